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

}  // namespace fgk
