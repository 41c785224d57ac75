// Host side of the direct-to-LDS GEMM kernel: eligibility test and launch.
#include <cstdio>
#include <cstdlib>
#include <mutex>
#include "gemm_dma.h"

namespace fgk {

// The kernel's preconditions.  `elem_bytes` is the size of the A/B/C element type.
// `ragged`: K a multiple of 8 above 64 but not of 64 (the data-parallel 256x256 and 128x128 kernels only)
static bool dma_supported_k(const GemmArgs& g, int elem_bytes, bool ragged) {
  if (elem_bytes != 2) return false;
  if (ragged ? (g.K <= kDmaBK || g.K % 8 != 0 || g.K % kDmaBK == 0) : (g.K < kDmaBK || g.K % kDmaBK != 0)) return false;
  if (g.M < 1 || g.N < 8 || g.N % 8 != 0) return false;
  if (g.sak != 1 || g.sam % 8 != 0 || !fg_aligned(g.A, 16) || !fg_aligned(g.B, 16)) return false;
  if (g.scn != 1 || g.scm % 8 != 0 || !fg_aligned(g.C, 16)) return false;
  if (g.bias != nullptr && (g.sin != 1 || g.sim % 4 != 0 || !fg_aligned(g.bias, 8))) return false;
  // the kernels address a tile's rows through 32-bit byte offsets from a scalar base: 256 rows (64 for the k-rows
  // of an N-contiguous B) of the leading dimension, plus a row, must stay below 4 GiB
  const int64_t lim = ((int64_t)1 << 32) - 8192;
  if (g.sam * 2 * 256 + g.K * 2 >= lim) return false;
  if (g.sbk == 1) return g.sbn % 8 == 0 && g.sbn * 2 * 256 + g.K * 2 < lim;  // K-contiguous B
  if (g.sbn == 1) return g.sbk % 8 == 0 && g.sbk * 2 * 64 + g.N * 2 < lim;   // N-contiguous B
  return false;
}
bool dma_supported(const GemmArgs& g, int elem_bytes) { return dma_supported_k(g, elem_bytes, false); }
bool dma_supported_ragged(const GemmArgs& g, int elem_bytes) { return dma_supported_k(g, elem_bytes, true); }

// 4 KB of zeros per device: the source of the chunks past K in the last K step of a ragged problem
static __device__ __align__(256) unsigned char dma_zero_chunks[4096];
const void* dma_zeros() {
  static std::mutex mu;
  static const void* per_device[64] = {};
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) return nullptr;
  std::lock_guard<std::mutex> lock(mu);
  if (per_device[dev] == nullptr) {
    void* p = nullptr;
    if (hipGetSymbolAddress(&p, HIP_SYMBOL(dma_zero_chunks)) != hipSuccess) return nullptr;
    per_device[dev] = p;
  }
  return per_device[dev];
}

template <typename T, bool B_KC, int BM, int BN, int NS, bool RAGGED = false>
static int launch_dma_t(const GemmArgs& g, hipStream_t st) {
  constexpr int LDS = dma_lds_bytes(BM, BN, NS);
  static_assert(LDS <= 160 * 1024, "LDS of one CU");
  static std::once_flag once;
  static hipError_t attr_err = hipSuccess;
  auto kern = gemm_dma_kernel<T, B_KC, BM, BN, NS, RAGGED>;
  std::call_once(once, [&] {
    attr_err = hipFuncSetAttribute(reinterpret_cast<const void*>(kern), hipFuncAttributeMaxDynamicSharedMemorySize, LDS);
  });
  if (attr_err != hipSuccess) {
    fg_set_error("gemm: cannot reserve %d bytes of LDS: %s", LDS, hipGetErrorString(attr_err));
    return FG_ERR_LAUNCH;
  }
  const int64_t tiles = (int64_t)g.tiles_m * g.tiles_n;
  hipLaunchKernelGGL(kern, dim3((unsigned)tiles), dim3(256), LDS, st, g);
  return fg_check_launch("gemm");
}

template <typename T, int BM, int BN, int NS, bool RAGGED = false>
static int launch_dma_b(const GemmArgs& g, hipStream_t st) {
  return g.sbk == 1 ? launch_dma_t<T, true, BM, BN, NS, RAGGED>(g, st) : launch_dma_t<T, false, BM, BN, NS, RAGGED>(g, st);
}

// Duration model of a data-parallel launch, in microseconds.  A CU holds `per_cu` workgroups of a tile size, so the
// tiles run in rounds of per_cu * num_cu.  A K step of a round that is the whole launch costs `lone` when few CUs are
// busy and `loaded` when all are (the matrix cores then share the power budget); in between the cost follows the cube
// of the fill (half a round still runs at the lone rate).  A ragged round behind full ones starts while their
// stragglers finish: it adds 0.70 to 0.95 of a lone round on top of that.  Constants measured on MI355X on sustained
// clocks, bf16, K = 4096, weights not resident in the caches, 32 to 1024 tiles of each size (us per K step and
// round: 256x256 1.38 at 32-192 tiles, 1.57 at 256, 1.51-1.57 per round at 512-1024; 128x128 0.57 up to 256 tiles,
// 0.91 at 320, 0.94 at 384, 1.05 at 512, 1.00 per 512 tiles beyond).
struct DmaTileCost { int bm, bn, per_cu; double lone, loaded; };
static const DmaTileCost kDmaTiles[] = {
    {256, 256, 1, 1.38, 1.55},
    {192, 256, 1, 1.25, 1.26},
    {256, 128, 1, 0.78, 0.88},
    {128, 256, 1, 0.835, 0.89},
    {128, 128, 2, 0.57, 1.02},
};
static double dma_dp_cost(const DmaTileCost& t, int64_t M, int64_t N, int64_t K, int num_cu) {
  const int64_t tiles = fg_cdiv(M, t.bm) * fg_cdiv(N, t.bn);
  const int64_t cap = (int64_t)num_cu * t.per_cu;
  const int64_t full = tiles / cap, last = tiles % cap;
  const double f = (double)last / (double)cap;
  double steps = (double)full * t.loaded;
  if (last > 0) {
    const double behind = full > 0 ? 0.70 + 0.25 * f : 1.0;
    if (t.per_cu == 1) {
      steps += t.lone * behind + (t.loaded - t.lone) * f * f * f;
    } else {
      // two workgroups on a CU run at little more than half speed each: the cost steps up where the second ones arrive
      const double part = last <= num_cu ? t.lone : 0.90 + 0.15 * (double)(last - num_cu) / (double)num_cu;
      steps += part * behind;
    }
  }
  return steps * (double)(K / kDmaBK);
}
static bool dma_tile_exists(int bm, int bn) {
  for (const DmaTileCost& t : kDmaTiles)
    if (t.bm == bm && t.bn == bn) return true;
  return false;
}

// Tile choice: the candidate the model above finishes first.  Returns its estimated duration.
double dma_pick_tile(int64_t M, int64_t N, int64_t K, int num_cu, int* bm, int* bn) {
  const FgOptions& opt = fg_options();  // measurement aid: one of the tiles above forced
  if (opt.gemm_tile_bm > 0 && dma_tile_exists(opt.gemm_tile_bm, opt.gemm_tile_bn)) {
    *bm = opt.gemm_tile_bm; *bn = opt.gemm_tile_bn;
    return 0.0;
  }
  double best = 0.0;
  bool have = false;
  for (const DmaTileCost& t : kDmaTiles) {
    const double c = dma_dp_cost(t, M, N, K, num_cu);
    if (!have || c < best) { best = c; *bm = t.bm; *bn = t.bn; have = true; }
  }
  return best;
}

// Stream-K on 128x128 tiles: how many workgroups share the `sk_tiles` cooperative tiles, and the estimated duration of
// that launch in microseconds.  Either every CU takes an equal share of the K steps (tile boundaries then fall
// inside the shares: a workgroup restarts its pipeline in a second tile and more tiles need a fix-up), or each tile
// is cut into s equal parts, s a divisor of the K steps per tile, on sk_tiles * s <= num_cu workgroups.  Measured:
// ~20 us of launch, first fetch and fix-up (~10 us less when no tile is shared at all) and 0.42 us per K step for
// the aligned cut.  With equal shares the workgroups of one tile row read different K ranges at the same time, L2
// reuse drops and the launch can turn bandwidth-bound: ~7 us more and 0.6 us per K step.
double dma_streamk_plan(int64_t sk_tiles, int64_t iters_per_tile, int num_cu, int* workers) {
  const int64_t total = sk_tiles * iters_per_tile;
  if (total <= 0) { *workers = 0; return 0.0; }
  int64_t w = total < num_cu ? total : num_cu;
  const bool aligned = total % w == 0 && ((total / w) % iters_per_tile == 0 || iters_per_tile % (total / w) == 0);
  double best = aligned ? 20.0 + 0.42 * (double)(total / w) : 27.0 + 0.6 * (double)fg_cdiv(total, w);
  *workers = (int)w;
  if (fg_options().gemm_sk_even) return best;  // measurement and test aid: always equal shares
  for (int64_t s = 1; s <= iters_per_tile && sk_tiles * s <= num_cu; ++s) {
    if (iters_per_tile % s != 0) continue;
    const double c = (s == 1 ? 10.0 : 20.0) + 0.42 * (double)(iters_per_tile / s);
    if (c < best) { best = c; *workers = (int)(sk_tiles * s); }
  }
  return best;
}

// g.tiles_m / g.tiles_n must describe bm x bn tiles.  Every tile runs with as many LDS stages as one workgroup per CU
// can hold: two for 256x256 and 192x256, three for 256x128 and 128x256, four for 128x128.
int dma_launch(const GemmArgs& g, int dtype, int bm, int bn, hipStream_t st) {
#define FG_DMA(T)                                                                                         \
  do {                                                                                                    \
    if (g.k_ragged != 0) {                                                                                \
      if (bm == 256 && bn == 256) return launch_dma_b<T, 256, 256, 2, true>(g, st);                       \
      if (bm == 128 && bn == 128) return launch_dma_b<T, 128, 128, 4, true>(g, st);                       \
      break;                                                                                              \
    }                                                                                                     \
    if (bm == 256 && bn == 256) return launch_dma_b<T, 256, 256, 2>(g, st);                               \
    if (bm == 192 && bn == 256) return launch_dma_b<T, 192, 256, 2>(g, st);                               \
    if (bm == 256 && bn == 128) return launch_dma_b<T, 256, 128, 3>(g, st);                               \
    if (bm == 128 && bn == 256) return launch_dma_b<T, 128, 256, 3>(g, st);                               \
    if (bm == 128 && bn == 128) return launch_dma_b<T, 128, 128, 4>(g, st);                               \
  } while (0)
  if (dtype == FG_BF16) FG_DMA(bf16_t);
  else FG_DMA(f16_t);
#undef FG_DMA
  fg_set_error("gemm: no direct-to-LDS kernel for %d x %d tiles", bm, bn);
  return FG_ERR_UNSUPPORTED;
}


// Stream-K on the direct-to-LDS main loop, 128x128 tiles: the tiles of the ragged last wave (all tiles, when there
// is less than a wave of them) are shared K step by K step between one workgroup per CU; full waves in front of
// them run data-parallel.  `g` must satisfy dma_supported(); the workspace is the one streamk_workspace_bytes()
// sizes (tickets + two partial tiles per workgroup).
template <typename T, bool B_KC, int NS>
static int launch_dma_streamk_t(const GemmArgs& g, int dp_tiles, hipStream_t st) {
  constexpr int LDS = dma_lds_bytes(128, 128, 2), LDS_SK = dma_lds_bytes(128, 128, NS);
  static std::once_flag once;
  static hipError_t attr_err = hipSuccess;
  auto dp = gemm_dma_kernel<T, B_KC, 128, 128, 2>;
  auto sk = gemm_dma_streamk_kernel<T, B_KC, NS>;
  std::call_once(once, [&] {
    attr_err = hipFuncSetAttribute(reinterpret_cast<const void*>(dp), hipFuncAttributeMaxDynamicSharedMemorySize, LDS);
    if (attr_err == hipSuccess)
      attr_err = hipFuncSetAttribute(reinterpret_cast<const void*>(sk), hipFuncAttributeMaxDynamicSharedMemorySize, LDS_SK);
  });
  if (attr_err != hipSuccess) {
    fg_set_error("gemm(stream-K): cannot reserve %d bytes of LDS: %s", LDS, hipGetErrorString(attr_err));
    return FG_ERR_LAUNCH;
  }
  if (dp_tiles > 0) hipLaunchKernelGGL(dp, dim3((unsigned)dp_tiles), dim3(256), LDS, st, g);
  if (g.sk_tiles > 0) hipLaunchKernelGGL(sk, dim3((unsigned)g.sk_workers), dim3(256), LDS_SK, st, g);
  return fg_check_launch("gemm(stream-K)");
}

int dma_streamk_launch(GemmArgs g, int dtype, void* workspace, size_t workspace_bytes, int num_cu, hipStream_t st) {
  FG_REQUIRE(workspace != nullptr && fg_aligned(workspace, 256), FG_ERR_WORKSPACE,
             "gemm(stream-K): workspace must be 256-byte aligned");
  FG_REQUIRE(num_cu <= kMaxWorkers, FG_ERR_UNSUPPORTED, "gemm(stream-K): more CUs than ticket counters");
  FG_REQUIRE(workspace_bytes >= kPartialOffset + (size_t)num_cu * 2 * 128 * 128 * sizeof(float), FG_ERR_WORKSPACE,
             "gemm(stream-K): workspace too small");
  g.tiles_m = (int)fg_cdiv(g.M, 128);
  g.tiles_n = (int)fg_cdiv(g.N, 128);
  g.iters_per_tile = (int)(g.K / kDmaBK);
  const int64_t tiles = (int64_t)g.tiles_m * g.tiles_n;
  FG_REQUIRE(tiles < ((int64_t)1 << 30), FG_ERR_UNSUPPORTED, "gemm(stream-K): too many tiles");
  int64_t sk_tiles = 0;
  fg_streamk_partition(tiles, g.iters_per_tile, num_cu, &sk_tiles, nullptr, nullptr);
  const int64_t total_iters = sk_tiles * g.iters_per_tile;
  int workers = 0;
  dma_streamk_plan(sk_tiles, g.iters_per_tile, num_cu, &workers);
  g.sk_tiles = (int)sk_tiles;
  g.sk_workers = workers;
  g.sk_per = workers > 0 ? total_iters / workers : 0;
  g.sk_rem = workers > 0 ? total_iters % workers : 0;
  g.tile_base = (int)sk_tiles;
  char* ws = (char*)workspace;
  g.tickets = (unsigned*)(ws + kTicketOffset);
  g.partials = (float*)(ws + kPartialOffset);
  const int dp_tiles = (int)(tiles - sk_tiles);
  const bool kc = g.sbk == 1;
  // one workgroup per CU: all of its LDS goes into a four-stage ring
  if (dtype == FG_BF16)
    return kc ? launch_dma_streamk_t<bf16_t, true, 4>(g, dp_tiles, st) : launch_dma_streamk_t<bf16_t, false, 4>(g, dp_tiles, st);
  return kc ? launch_dma_streamk_t<f16_t, true, 4>(g, dp_tiles, st) : launch_dma_streamk_t<f16_t, false, 4>(g, dp_tiles, st);
}

}  // namespace fgk
