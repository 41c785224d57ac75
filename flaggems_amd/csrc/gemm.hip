// Host side of fg_gemm: validation, load-mode and tile selection, schedule selection, launches.
#include <mutex>
#include <type_traits>
#include "gemm_tile.h"

namespace fgk {

// implemented in gemm_skinny.hip
int skinny_supported(const GemmArgs& g, int dtype, int amode, int bmode);
size_t skinny_workspace_bytes(int64_t M, int64_t N, int64_t K, int num_cu);
int skinny_launch(const GemmArgs& g, int dtype, int b_kind, void* workspace, size_t workspace_bytes, int num_cu,
                  hipStream_t st);
// implemented in gemm_streamk.hip
size_t streamk_workspace_bytes(int64_t M, int64_t N, int64_t K, int dtype, int num_cu);
int streamk_launch(GemmArgs g, int dtype, int amode, int bmode, void* workspace, size_t workspace_bytes, int num_cu,
                   hipStream_t st);

// implemented in gemm_dma.hip
bool dma_supported(const GemmArgs& g, int elem_bytes);
bool dma_supported_ragged(const GemmArgs& g, int elem_bytes);
const void* dma_zeros();
double dma_pick_tile(int64_t M, int64_t N, int64_t K, int num_cu, int* bm, int* bn);
double dma_streamk_plan(int64_t sk_tiles, int64_t iters_per_tile, int num_cu, int* workers);
int dma_launch(const GemmArgs& g, int dtype, int bm, int bn, hipStream_t st);
int dma_streamk_launch(GemmArgs g, int dtype, void* workspace, size_t workspace_bytes, int num_cu, hipStream_t st);

int num_cus(int device) {
  static std::mutex mu;
  static int cached[64] = {0};
  int dev = device;
  if (dev < 0) {
    if (hipGetDevice(&dev) != hipSuccess) dev = 0;
  }
  if (dev >= 64) dev = 0;
  std::lock_guard<std::mutex> lk(mu);
  if (cached[dev] == 0) {
    int n = 0;
    if (hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || n <= 0) n = 256;
    cached[dev] = n;
  }
  return cached[dev];
}

template <typename T, int BM, int BN, int AMODE, int BMODE>
int launch_dp(const GemmArgs& g, hipStream_t st) {
  typedef TileCompute<T, BM, BN, AMODE, BMODE> TC;
  static std::once_flag once;
  static hipError_t attr_err = hipSuccess;
  auto kern = gemm_dp_kernel<T, BM, BN, AMODE, BMODE>;
  std::call_once(once, [&] {
    attr_err = hipFuncSetAttribute(reinterpret_cast<const void*>(kern), hipFuncAttributeMaxDynamicSharedMemorySize,
                                   TC::LDS_BYTES);
  });
  if (attr_err != hipSuccess) {
    fg_set_error("gemm: cannot reserve %d bytes of LDS: %s", TC::LDS_BYTES, hipGetErrorString(attr_err));
    return FG_ERR_LAUNCH;
  }
  const int64_t tiles = (int64_t)g.tiles_m * g.tiles_n;
  hipLaunchKernelGGL(kern, dim3((unsigned)tiles), dim3(kThreads), TC::LDS_BYTES, st, g);
  return fg_check_launch("gemm");
}

// (split in two so that the element-wise stager, the last resort of the small tile, is never instantiated for the
// large one: it would not be launched there, and it compiles to a kernel that spills a thousand registers)
template <typename T, int BM, int BN>
int launch_dp_small_modes(const GemmArgs& g, int amode, int bmode, hipStream_t st);

template <typename T, int BM, int BN>
int launch_dp_modes(const GemmArgs& g, int amode, int bmode, hipStream_t st) {
  if constexpr (BM == 256) {
    // the element-wise stager would not fit the register budget of the large tile
    if (amode == LOAD_K && bmode == LOAD_K) return launch_dp<T, BM, BN, LOAD_K, LOAD_K>(g, st);
    if (amode == LOAD_K && bmode == LOAD_MN) return launch_dp<T, BM, BN, LOAD_K, LOAD_MN>(g, st);
    if (amode == LOAD_MN && bmode == LOAD_K) return launch_dp<T, BM, BN, LOAD_MN, LOAD_K>(g, st);
    return launch_dp<T, BM, BN, LOAD_MN, LOAD_MN>(g, st);
  } else {
    return launch_dp_small_modes<T, BM, BN>(g, amode, bmode, st);
  }
}

template <typename T, int BM, int BN>
int launch_dp_small_modes(const GemmArgs& g, int amode, int bmode, hipStream_t st) {
  if constexpr (sizeof(T) == 2) {
    if (amode == LOAD_K && bmode == LOAD_K) return launch_dp<T, BM, BN, LOAD_K, LOAD_K>(g, st);
    if (amode == LOAD_K && bmode == LOAD_MN) return launch_dp<T, BM, BN, LOAD_K, LOAD_MN>(g, st);
    if (amode == LOAD_MN && bmode == LOAD_K) return launch_dp<T, BM, BN, LOAD_MN, LOAD_K>(g, st);
    if (amode == LOAD_MN && bmode == LOAD_MN) return launch_dp<T, BM, BN, LOAD_MN, LOAD_MN>(g, st);
    // operands contiguous along one axis but not aligned for the modes above
    if (amode == LOAD_KU && bmode == LOAD_KU) return launch_dp<T, BM, BN, LOAD_KU, LOAD_KU>(g, st);
    if (amode == LOAD_KU && bmode == LOAD_MNU) return launch_dp<T, BM, BN, LOAD_KU, LOAD_MNU>(g, st);
    if (amode == LOAD_MNU && bmode == LOAD_KU) return launch_dp<T, BM, BN, LOAD_MNU, LOAD_KU>(g, st);
    if (amode == LOAD_MNU && bmode == LOAD_MNU) return launch_dp<T, BM, BN, LOAD_MNU, LOAD_MNU>(g, st);
  } else {
    if (amode == LOAD_K && bmode == LOAD_K) return launch_dp<T, BM, BN, LOAD_K, LOAD_K>(g, st);
    if (amode == LOAD_KU && bmode == LOAD_KU) return launch_dp<T, BM, BN, LOAD_KU, LOAD_KU>(g, st);
    if (amode == LOAD_KU && bmode == LOAD_MNU) return launch_dp<T, BM, BN, LOAD_KU, LOAD_MNU>(g, st);
    if (amode == LOAD_MNU && bmode == LOAD_KU) return launch_dp<T, BM, BN, LOAD_MNU, LOAD_KU>(g, st);
    if (amode == LOAD_MNU && bmode == LOAD_MNU) return launch_dp<T, BM, BN, LOAD_MNU, LOAD_MNU>(g, st);
  }
  return launch_dp<T, BM, BN, LOAD_GEN, LOAD_GEN>(g, st);
}

// Load mode of an operand that pick_mode() turned away: the element-aligned vector modes when it is contiguous
// along K or along its row index, element-wise otherwise.
int pick_mode_unaligned(int64_t rows, int64_t K, int64_t s_row, int64_t s_k) {
  if (s_k == 1 || K == 1) return LOAD_KU;
  if (s_row == 1 || rows == 1) return LOAD_MNU;
  return LOAD_GEN;
}

// Load mode of an operand whose element (row, k) lives at base[row*s_row + k*s_k].
int pick_mode(const void* base, int64_t rows, int64_t K, int64_t s_row, int64_t s_k, int elem_bytes) {
  const int epc = 16 / elem_bytes;
  if (!fg_aligned(base, 16)) return LOAD_GEN;
  if ((s_k == 1 || K == 1) && K % epc == 0 && (rows == 1 || s_row % epc == 0)) return LOAD_K;
  if (elem_bytes == 2 && (s_row == 1 || rows == 1) && rows % 8 == 0 && rows >= 8 && (K == 1 || s_k % 8 == 0))
    return LOAD_MN;
  return LOAD_GEN;
}

constexpr int kDmaBKHost = 64;  // K step of the direct-to-LDS kernels

void set_tiles(GemmArgs& g, int BM, int BN, int BK) {
  g.tiles_m = (int)fg_cdiv(g.M, BM);
  g.tiles_n = (int)fg_cdiv(g.N, BN);
  g.iters_per_tile = (int)fg_cdiv(g.K, BK);
}

template <typename T>
int run_dp(GemmArgs g, int amode, int bmode, int num_cu, hipStream_t st) {
  constexpr int BK = kRowBytes / sizeof(T);
  if constexpr (sizeof(T) == 2) {
    // Aligned operands with K a multiple of 64 take the direct-to-LDS kernel, on the tile size that fills
    // the machine best (even a lone 128x128 workgroup per CU runs twice as fast as the register-staged kernel).
    if (amode != LOAD_GEN && dma_supported(g, (int)sizeof(T)) && !fg_options().gemm_no_dma) {
      int bm = 256, bn = 256;
      dma_pick_tile(g.M, g.N, g.K, num_cu, &bm, &bn);
      set_tiles(g, bm, bn, BK);
      return dma_launch(g, std::is_same<T, bf16_t>::value ? FG_BF16 : FG_F16, bm, bn, st);
    }
    // The 256x256 tile halves LDS and L2 traffic per flop; it pays once it can fill the machine.
    const int64_t big_tiles = fg_cdiv(g.M, 256) * fg_cdiv(g.N, 256);
    // K a multiple of 8 but not of 64: the direct-to-LDS kernel on one of two tiles, the last K step padded with zeros
    if (amode != LOAD_GEN && dma_supported_ragged(g, (int)sizeof(T)) && !fg_options().gemm_no_dma) {
      g.zeros = dma_zeros();
      if (g.zeros != nullptr) {
        const bool big = big_tiles * 10 >= (int64_t)num_cu * 9;
        set_tiles(g, big ? 256 : 128, big ? 256 : 128, BK);
        g.k_ragged = (int)(g.K % kDmaBKHost);
        return dma_launch(g, std::is_same<T, bf16_t>::value ? FG_BF16 : FG_F16, big ? 256 : 128, big ? 256 : 128, st);
      }
    }
    if (amode != LOAD_GEN && amode != LOAD_KU && amode != LOAD_MNU && g.M >= 256 && g.N >= 256 && big_tiles * 10 >= (int64_t)num_cu * 9) {
      set_tiles(g, 256, 256, BK);
      return launch_dp_modes<T, 256, 256>(g, amode, bmode, st);
    }
  }
  set_tiles(g, 128, 128, BK);
  FG_REQUIRE((int64_t)g.tiles_m * g.tiles_n < ((int64_t)1 << 31), FG_ERR_UNSUPPORTED, "gemm: too many tiles");
  return launch_dp_modes<T, 128, 128>(g, amode, bmode, st);
}

}  // namespace fgk

using namespace fgk;

extern "C" int fg_streamk_partition(int64_t tiles, int64_t iters_per_tile, int64_t workers, int64_t* sk_tiles,
                                    int64_t* begin, int64_t* end) {
  FG_REQUIRE(tiles >= 0 && iters_per_tile > 0 && workers > 0, FG_ERR_INVALID, "streamk_partition: bad sizes");
  // Cooperative tiles: the ragged last wave; plus one full wave when the remainder is small
  // (< half the workers), none when it nearly fills the machine (> 0.8 of the workers) and full
  // waves exist.  Same rule as the reference's streamk_mm.
  int64_t sk = tiles % workers;
  const int64_t full = tiles - sk;
  if (full > 0 && sk * 2 < workers) sk += workers;
  else if (full > 0 && sk * 10 > workers * 8) sk = 0;
  if (sk_tiles) *sk_tiles = sk;
  const int64_t total = sk * iters_per_tile;
  const int64_t per = total / workers, rem = total % workers;
  for (int64_t w = 0; w < workers; ++w) {
    // workers below `rem` take one extra iteration; ranges are contiguous in tile-major order
    const int64_t b = w * per + (w < rem ? w : rem);
    const int64_t e = b + per + (w < rem ? 1 : 0);
    if (begin) begin[w] = b;
    if (end) end[w] = e;
  }
  return FG_OK;
}

extern "C" size_t fg_gemm_workspace_bytes(int64_t M, int64_t N, int64_t K, int ab_dtype, int schedule, int device) {
  if (schedule == FG_SCHED_DATA_PARALLEL) return 0;
  const int cu = num_cus(device);
  size_t a = skinny_workspace_bytes(M, N, K, cu);
  size_t b = streamk_workspace_bytes(M, N, K, ab_dtype, cu);
  return a > b ? a : b;
}

extern "C" int fg_gemm_workspace_layout(int device, size_t* max_bytes, size_t* header_bytes) {
  // the largest request of either stream-K family: header + two fp32 128x128 partial tiles per CU
  const int cu = num_cus(device);
  if (max_bytes) *max_bytes = kPartialOffset + (size_t)(cu < kMaxWorkers ? cu : kMaxWorkers) * 2 * 128 * 128 * sizeof(float);
  if (header_bytes) *header_bytes = kPartialOffset;
  return FG_OK;
}

extern "C" int fg_gemm_tile_order(int tiles_m, int tiles_n, int b_k_contiguous, int* tile_m, int* tile_n) {
  FG_REQUIRE(tiles_m > 0 && tiles_n > 0 && (int64_t)tiles_m * tiles_n < ((int64_t)1 << 31), FG_ERR_INVALID,
             "gemm_tile_order: bad grid %d x %d", tiles_m, tiles_n);
  FG_REQUIRE(tile_m && tile_n, FG_ERR_INVALID, "gemm_tile_order: null pointer");
  const int total = tiles_m * tiles_n;
  // the direct-to-LDS kernels walk strips of 2 sub-block rows for a K-contiguous B and of 4 for a row-major one
  for (int id = 0; id < total; ++id) tile_coords(id, tiles_m, tiles_n, tile_m[id], tile_n[id], b_k_contiguous ? 2 : 4);
  return FG_OK;
}

// The automatic schedule's choice between the two direct-to-LDS launches (shared by fg_gemm and fg_gemm_plan).
static bool dma_auto_streamk(int64_t M, int64_t N, int64_t K, int cu, int* bm, int* bn, double* dp_us, int* workers,
                             double* sk_us) {
  const int64_t tiles = fg_cdiv(M, 128) * fg_cdiv(N, 128);
  const int64_t iters = fg_cdiv(K, 64);
  *dp_us = dma_pick_tile(M, N, K, cu, bm, bn);
  *workers = 0;
  *sk_us = 0.0;
  if (!(tiles <= cu && tiles * iters >= 4 * (int64_t)cu)) return false;
  *sk_us = dma_streamk_plan(tiles, iters, cu, workers);
  return *sk_us < *dp_us;
}

extern "C" int fg_gemm_plan(int64_t M, int64_t N, int64_t K, int num_cu, int* tile_m, int* tile_n, double* dp_us,
                            int* streamk_workers, double* streamk_us, int* streamk_chosen) {
  FG_REQUIRE(M > 0 && N > 0 && K > 0, FG_ERR_INVALID, "gemm_plan: sizes must be positive");
  FG_REQUIRE(K % 64 == 0, FG_ERR_UNSUPPORTED, "gemm_plan: K = %lld is not a multiple of 64", (long long)K);
  const int cu = num_cu > 0 ? num_cu : num_cus(-1);
  FG_REQUIRE(cu > 0, FG_ERR_INVALID, "gemm_plan: no device and no CU count given");
  int bm = 0, bn = 0, workers = 0;
  double dp = 0.0, sk = 0.0;
  const bool chosen = dma_auto_streamk(M, N, K, cu, &bm, &bn, &dp, &workers, &sk);
  if (tile_m) *tile_m = bm;
  if (tile_n) *tile_n = bn;
  if (dp_us) *dp_us = dp;
  if (streamk_workers) *streamk_workers = workers;
  if (streamk_us) *streamk_us = sk;
  if (streamk_chosen) *streamk_chosen = chosen ? 1 : 0;
  return FG_OK;
}

extern "C" int fg_stream_capture_id(void* stream, unsigned long long* id) {
  hipStreamCaptureStatus status = hipStreamCaptureStatusNone;
  unsigned long long cid = 0;
  const hipError_t e = hipStreamGetCaptureInfo((hipStream_t)stream, &status, &cid);
  if (e != hipSuccess) {
    (void)hipGetLastError();
    fg_set_error("stream_capture_id: %s", hipGetErrorString(e));
    return FG_ERR_INVALID;
  }
  if (id) *id = status == hipStreamCaptureStatusActive ? (cid != 0 ? cid : ~0ull) : 0;
  return FG_OK;
}

extern "C" int fg_gemm(const void* A, const void* B, const void* bias, void* C, int64_t M, int64_t N, int64_t K,
                       int64_t sam, int64_t sak, int64_t sbk, int64_t sbn, int64_t sim, int64_t sin_, int64_t scm,
                       int64_t scn, float alpha, float beta, int ab_dtype, int c_dtype, int bias_dtype, int schedule,
                       void* workspace, size_t workspace_bytes, int* schedule_used, void* stream) {
  FG_REQUIRE(M >= 0 && N >= 0 && K >= 0, FG_ERR_INVALID, "gemm: negative size");
  FG_REQUIRE(ab_dtype == FG_F16 || ab_dtype == FG_BF16 || ab_dtype == FG_F32, FG_ERR_INVALID, "gemm: bad dtype %d",
             ab_dtype);
  FG_REQUIRE(c_dtype == ab_dtype, FG_ERR_UNSUPPORTED, "gemm: output dtype %d must equal the input dtype %d", c_dtype,
             ab_dtype);
  FG_REQUIRE(bias == nullptr || bias_dtype == ab_dtype, FG_ERR_UNSUPPORTED,
             "gemm: bias dtype %d must equal the input dtype %d", bias_dtype, ab_dtype);
  FG_REQUIRE(schedule >= FG_SCHED_AUTO && schedule <= FG_SCHED_STREAM_K, FG_ERR_INVALID, "gemm: bad schedule %d",
             schedule);
  if (schedule_used) *schedule_used = FG_SCHED_DATA_PARALLEL;
  if (M == 0 || N == 0) return FG_OK;
  FG_REQUIRE(K > 0, FG_ERR_INVALID, "gemm: K must be positive (the caller handles K == 0)");
  FG_REQUIRE(A && B && C, FG_ERR_INVALID, "gemm: null pointer");
  FG_REQUIRE(M < ((int64_t)1 << 31) && N < ((int64_t)1 << 31) && K < ((int64_t)1 << 31), FG_ERR_UNSUPPORTED,
             "gemm: extent exceeds 2^31");
  hipStream_t st = (hipStream_t)stream;
  GemmArgs g = {};
  g.A = A; g.B = B; g.bias = bias; g.C = C;
  g.M = M; g.N = N; g.K = K;
  g.sam = sam; g.sak = sak; g.sbk = sbk; g.sbn = sbn; g.sim = sim; g.sin = sin_; g.scm = scm; g.scn = scn;
  g.alpha = alpha; g.beta = beta;
  const int eb = ab_dtype == FG_F32 ? 4 : 2;
  int amode = pick_mode(A, M, K, sam, sak, eb);
  int bmode = pick_mode(B, N, K, sbn, sbk, eb);
  if (amode == LOAD_GEN || bmode == LOAD_GEN || (eb == 4 && (amode != LOAD_K || bmode != LOAD_K))) {
    // one kernel serves both operands: either both take an element-aligned vector mode or both go element by element
    amode = pick_mode_unaligned(M, K, sam, sak);
    bmode = pick_mode_unaligned(N, K, sbn, sbk);
    if (amode == LOAD_GEN || bmode == LOAD_GEN) amode = bmode = LOAD_GEN;
  }
  const bool vec_unaligned = amode == LOAD_KU || amode == LOAD_MNU;
  const int cu = num_cus(-1);

  // ---- schedule --------------------------------------------------------------------------------
  // Skinny problems (M <= 16 rows) are bandwidth-bound streams of B: their own stream-K kernel.
  const int sk_ok = skinny_supported(g, ab_dtype, amode, bmode);
  bool use_skinny = false, use_streamk = false;
  if (schedule != FG_SCHED_DATA_PARALLEL && workspace != nullptr) {
    if (sk_ok) {
      use_skinny = workspace_bytes >= skinny_workspace_bytes(M, N, K, cu);
    } else if (eb == 2) {
      const size_t need = streamk_workspace_bytes(M, N, K, ab_dtype, cu);
      if (need > 0 && workspace_bytes >= need) {
        if (schedule == FG_SCHED_STREAM_K) {
          use_streamk = true;
        } else {
          // auto: stream-K when the tiles cannot fill the machine and K is deep enough to hand every workgroup
          // at least four K steps; fuller grids run data-parallel.  The register-staged main loop is worth
          // sharing up to half a wave of tiles; for the direct-to-LDS one the two duration models decide.
          const int64_t tiles = fg_cdiv(M, 128) * fg_cdiv(N, 128);
          const int64_t iters = fg_cdiv(K, 64);
          const bool dma = amode != LOAD_GEN && dma_supported(g, eb) && !fg_options().gemm_no_dma;
          if (dma) {
            int bm, bn, workers;
            double dp_us, sk_us;
            use_streamk = dma_auto_streamk(M, N, K, cu, &bm, &bn, &dp_us, &workers, &sk_us);
          } else {
            // (the stream-K kernels have no element-aligned vector modes: such operands stay data-parallel)
            use_streamk = !vec_unaligned && tiles * 2 <= (int64_t)cu && tiles * iters >= 4 * (int64_t)cu;
          }
        }
      }
    }
  }
  if (schedule == FG_SCHED_STREAM_K && !use_skinny && !use_streamk) {
    fg_set_error("gemm: the stream-K schedule needs 16-bit inputs and a workspace of %zu bytes (got %zu)",
                 fg_gemm_workspace_bytes(M, N, K, ab_dtype, schedule, -1), workspace_bytes);
    return workspace == nullptr || eb == 2 ? FG_ERR_WORKSPACE : FG_ERR_UNSUPPORTED;
  }
  if (use_skinny) {
    if (schedule_used) *schedule_used = FG_SCHED_STREAM_K;
    return skinny_launch(g, ab_dtype, sk_ok, workspace, workspace_bytes, cu, st);
  }
  if (use_streamk) {
    if (schedule_used) *schedule_used = FG_SCHED_STREAM_K;
    if (amode != LOAD_GEN && dma_supported(g, eb) && !fg_options().gemm_no_dma)
      return dma_streamk_launch(g, ab_dtype, workspace, workspace_bytes, cu, st);
    return streamk_launch(g, ab_dtype, amode, bmode, workspace, workspace_bytes, cu, st);
  }
  switch (ab_dtype) {
    case FG_F16: return run_dp<f16_t>(g, amode, bmode, cu, st);
    case FG_BF16: return run_dp<bf16_t>(g, amode, bmode, cu, st);
    default: return run_dp<float>(g, amode, bmode, cu, st);
  }
}

extern "C" int fg_bmm(const void* A, const void* B, void* C, int64_t batch, int64_t M, int64_t N, int64_t K,
                      int64_t sab, int64_t sam, int64_t sak, int64_t sbb, int64_t sbk, int64_t sbn, int64_t scb,
                      int64_t scm, int64_t scn, int dtype, void* stream) {
  FG_REQUIRE(batch >= 0 && M >= 0 && N >= 0 && K >= 0, FG_ERR_INVALID, "bmm: negative size");
  FG_REQUIRE(dtype == FG_F16 || dtype == FG_BF16 || dtype == FG_F32, FG_ERR_INVALID, "bmm: bad dtype %d", dtype);
  if (batch == 0 || M == 0 || N == 0) return FG_OK;
  FG_REQUIRE(K > 0, FG_ERR_INVALID, "bmm: K must be positive (the caller handles K == 0)");
  FG_REQUIRE(A && B && C, FG_ERR_INVALID, "bmm: null pointer");
  // The envelope the parity cases cover.  A larger batch (32 x 2048 x 2048 x 128 bf16, timed in a loop) once ended
  // in a GPU memory fault whose cause was not found in the kernels' address arithmetic; until it is, no binder can
  // reach that case through this entry.
  FG_REQUIRE(batch <= FG_BMM_MAX_BATCH && batch * M * N <= FG_BMM_MAX_OUT_ELEMS, FG_ERR_UNSUPPORTED,
             "bmm: %lld matrices of %lld x %lld are beyond the verified envelope (at most %d matrices and %lld output "
             "elements per call); split the batch or use the vendor library",
             (long long)batch, (long long)M, (long long)N, FG_BMM_MAX_BATCH, (long long)FG_BMM_MAX_OUT_ELEMS);
  // One data-parallel 2-D launch per matrix, back to back on the stream: every matrix takes the kernel and
  // tile size its own pointers and strides qualify for.
  const int64_t eb = dtype == FG_F32 ? 4 : 2;
  for (int64_t z = 0; z < batch; ++z) {
    const int rc = fg_gemm((const char*)A + z * sab * eb, (const char*)B + z * sbb * eb, nullptr,
                           (char*)C + z * scb * eb, M, N, K, sam, sak, sbk, sbn, 0, 0, scm, scn, 1.0f, 0.0f, dtype,
                           dtype, dtype, FG_SCHED_DATA_PARALLEL, nullptr, 0, nullptr, stream);
    if (rc != FG_OK) return rc;
  }
  return FG_OK;
}
