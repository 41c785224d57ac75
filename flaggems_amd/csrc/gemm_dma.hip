// Host side of the direct-to-LDS GEMM kernel: eligibility test and launch.
#include <cstdio>
#include <cstdlib>
#include <mutex>
#include "gemm_dma.h"

namespace fgk {

// The kernel's preconditions.  `elem_bytes` is the size of the A/B/C element type.
bool dma_supported(const GemmArgs& g, int elem_bytes) {
  if (elem_bytes != 2) return false;
  if (g.K < kDmaBK || g.K % kDmaBK != 0 || g.M < 1 || g.N < 8 || g.N % 8 != 0) return false;
  if (g.sak != 1 || g.sam % 8 != 0 || !fg_aligned(g.A, 16) || !fg_aligned(g.B, 16)) return false;
  if (g.scn != 1 || g.scm % 8 != 0 || !fg_aligned(g.C, 16)) return false;
  if (g.bias != nullptr && (g.sin != 1 || g.sim % 4 != 0 || !fg_aligned(g.bias, 8))) return false;
  if (g.sbk == 1) return g.sbn % 8 == 0;  // K-contiguous B
  if (g.sbn == 1) return g.sbk % 8 == 0;  // N-contiguous B
  return false;
}

template <typename T, bool B_KC, int BM, int BN>
static int launch_dma_t(const GemmArgs& g, hipStream_t st) {
  constexpr int LDS = dma_lds_bytes(BM, BN);
  static std::once_flag once;
  static hipError_t attr_err = hipSuccess;
  auto kern = gemm_dma_kernel<T, B_KC, BM, BN>;
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

template <typename T, int BM, int BN>
static int launch_dma_b(const GemmArgs& g, hipStream_t st) {
  return g.sbk == 1 ? launch_dma_t<T, true, BM, BN>(g, st) : launch_dma_t<T, false, BM, BN>(g, st);
}

// Tile choice: the candidate whose busiest CU finishes first.  A CU runs ceil(tiles / CUs) tiles; a tile
// costs its area over its efficiency relative to the 256x256 tile (the smaller tiles read more LDS bytes
// per flop).  Two 128x128 workgroups share a CU and overlap well; one alone leaves the matrix cores idle
// while it waits.  The efficiencies are measured on MI355X (1024..8192-row problems).
void dma_pick_tile(int64_t M, int64_t N, int num_cu, int* bm, int* bn) {
  *bm = 256; *bn = 256;
  if (const char* e = getenv("FG_GEMM_TILE")) {  // measurement aid: "256x256" | "256x128" | "128x128"
    int a = 0, b = 0;
    if (sscanf(e, "%dx%d", &a, &b) == 2 && (a == 256 || a == 128) && (b == 256 || b == 128) && a >= b) {
      *bm = a; *bn = b;
      return;
    }
  }
  auto per_cu = [&](int tm, int tn) { return (double)fg_cdiv(fg_cdiv(M, tm) * fg_cdiv(N, tn), (int64_t)num_cu); };
  const double c256 = per_cu(256, 256);
  const double c256x128 = per_cu(256, 128) * 0.5 / 0.90;
  const double t128 = per_cu(128, 128);
  const double c128 = 0.25 * (2.0 * (double)((int64_t)t128 / 2) / 0.86 + (double)((int64_t)t128 % 2) / 0.63);
  double best = c256;
  if (c256x128 < best) { best = c256x128; *bm = 256; *bn = 128; }
  if (c128 < best) { best = c128; *bm = 128; *bn = 128; }
}

// g.tiles_m / g.tiles_n must describe bm x bn tiles.
int dma_launch(const GemmArgs& g, int dtype, int bm, int bn, hipStream_t st) {
#define FG_DMA(T) (bm == 256 && bn == 256 ? launch_dma_b<T, 256, 256>(g, st) : bm == 256 ? launch_dma_b<T, 256, 128>(g, st) : launch_dma_b<T, 128, 128>(g, st))
  if (dtype == FG_BF16) return FG_DMA(bf16_t);
  return FG_DMA(f16_t);
#undef FG_DMA
}


// Stream-K on the direct-to-LDS main loop, 128x128 tiles: the tiles of the ragged last wave (all tiles, when there
// is less than a wave of them) are shared K step by K step between one workgroup per CU; full waves in front of
// them run data-parallel.  `g` must satisfy dma_supported(); the workspace is the one streamk_workspace_bytes()
// sizes (tickets + two partial tiles per workgroup).
template <typename T, bool B_KC>
static int launch_dma_streamk_t(const GemmArgs& g, int dp_tiles, hipStream_t st) {
  constexpr int LDS = dma_lds_bytes(128, 128);
  static std::once_flag once;
  static hipError_t attr_err = hipSuccess;
  auto dp = gemm_dma_kernel<T, B_KC, 128, 128>;
  auto sk = gemm_dma_streamk_kernel<T, B_KC>;
  std::call_once(once, [&] {
    attr_err = hipFuncSetAttribute(reinterpret_cast<const void*>(dp), hipFuncAttributeMaxDynamicSharedMemorySize, LDS);
    if (attr_err == hipSuccess)
      attr_err = hipFuncSetAttribute(reinterpret_cast<const void*>(sk), hipFuncAttributeMaxDynamicSharedMemorySize, LDS);
  });
  if (attr_err != hipSuccess) {
    fg_set_error("gemm(stream-K): cannot reserve %d bytes of LDS: %s", LDS, hipGetErrorString(attr_err));
    return FG_ERR_LAUNCH;
  }
  if (dp_tiles > 0) hipLaunchKernelGGL(dp, dim3((unsigned)dp_tiles), dim3(256), LDS, st, g);
  if (g.sk_tiles > 0) hipLaunchKernelGGL(sk, dim3((unsigned)g.sk_workers), dim3(256), LDS, st, g);
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
  int workers = num_cu;
  if (total_iters < workers) workers = (int)total_iters;
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
  if (dtype == FG_BF16)
    return kc ? launch_dma_streamk_t<bf16_t, true>(g, dp_tiles, st) : launch_dma_streamk_t<bf16_t, false>(g, dp_tiles, st);
  return kc ? launch_dma_streamk_t<f16_t, true>(g, dp_tiles, st) : launch_dma_streamk_t<f16_t, false>(g, dp_tiles, st);
}

}  // namespace fgk
