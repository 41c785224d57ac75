// Host side of the direct-to-LDS GEMM kernel: eligibility test and launch.
#include <mutex>
#include "gemm_dma.h"

namespace fgk {

// The kernel's preconditions; the caller has already established that the problem is large enough
// for 256x256 tiles.  `elem_bytes` is the size of the A/B/C element type.
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

template <typename T, bool B_KC>
static int launch_dma_t(const GemmArgs& g, hipStream_t st) {
  static std::once_flag once;
  static hipError_t attr_err = hipSuccess;
  auto kern = gemm_dma_kernel<T, B_KC>;
  std::call_once(once, [&] {
    attr_err = hipFuncSetAttribute(reinterpret_cast<const void*>(kern), hipFuncAttributeMaxDynamicSharedMemorySize,
                                   kDmaLdsBytes);
  });
  if (attr_err != hipSuccess) {
    fg_set_error("gemm: cannot reserve %d bytes of LDS: %s", kDmaLdsBytes, hipGetErrorString(attr_err));
    return FG_ERR_LAUNCH;
  }
  const int64_t tiles = (int64_t)g.tiles_m * g.tiles_n;
  hipLaunchKernelGGL(kern, dim3((unsigned)tiles), dim3(256), kDmaLdsBytes, st, g);
  return fg_check_launch("gemm");
}

// g.tiles_m / g.tiles_n must describe 256x256 tiles.
int dma_launch(const GemmArgs& g, int dtype, hipStream_t st) {
  const bool b_kc = g.sbk == 1;
  if (dtype == FG_BF16) return b_kc ? launch_dma_t<bf16_t, true>(g, st) : launch_dma_t<bf16_t, false>(g, st);
  return b_kc ? launch_dma_t<f16_t, true>(g, st) : launch_dma_t<f16_t, false>(g, st);
}

}  // namespace fgk
