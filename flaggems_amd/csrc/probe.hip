// Calibration kernel for the matrix-core roofline: nothing but v_mfma_f32_16x16x32_bf16 (the instruction of the
// GEMM kernels) on operand fragments loaded once from a caller-supplied buffer, 64 independent accumulators per
// wave, one wave per SIMD.  What it sustains depends on the operand bits: the chip is power-limited, and random
// operands toggle far more logic than zeros, so the clock settles lower.  bench.py reports both; the rate with
// normally distributed operands is the ceiling a real bf16 GEMM can approach.  (The 32x32x16 shape reads and
// writes its accumulators twice as often per flop and sustains ~12 % less on the same operands: 1.78 against
// 2.02 PFLOP/s.)
#include "fg_common.h"

namespace {
__global__ __launch_bounds__(256) void mfma_probe_kernel(const bf16x8* src, float* out, int iters) {
  bf16x8 a[4], b[4];
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    a[i] = src[threadIdx.x + i * 256];
    b[i] = src[threadIdx.x + (4 + i) * 256];
  }
  f32x4 acc[8][8];
#pragma unroll
  for (int i = 0; i < 8; ++i)
#pragma unroll
    for (int j = 0; j < 8; ++j) acc[i][j] = f32x4{0.f, 0.f, 0.f, 0.f};
  for (int it = 0; it < iters; ++it) {
#pragma unroll
    for (int i = 0; i < 8; ++i)
#pragma unroll
      for (int j = 0; j < 8; ++j) acc[i][j] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a[i & 3], b[j & 3], acc[i][j], 0, 0, 0);
  }
  float s = 0.f;
#pragma unroll
  for (int i = 0; i < 8; ++i)
#pragma unroll
    for (int j = 0; j < 8; ++j)
#pragma unroll
      for (int e = 0; e < 4; ++e) s += acc[i][j][e];
  out[(size_t)blockIdx.x * 256 + threadIdx.x] = s;
}
}  // namespace

extern "C" int fg_mfma_probe(const void* operands, float* out, int blocks, int iters, double* flops, void* stream) {
  FG_REQUIRE(operands != nullptr && out != nullptr && blocks > 0 && iters > 0, FG_ERR_INVALID, "mfma_probe: bad arguments");
  FG_REQUIRE(fg_aligned(operands, 16), FG_ERR_UNSUPPORTED, "mfma_probe: operands must be 16-byte aligned");
  hipLaunchKernelGGL(mfma_probe_kernel, dim3((unsigned)blocks), dim3(256), 0, (hipStream_t)stream,
                     (const bf16x8*)operands, out, iters);
  // 4 waves x 64 MFMAs x 16*16*32*2 flops per iteration and block
  if (flops) *flops = (double)blocks * 4.0 * iters * 64.0 * 16384.0;
  return fg_check_launch("mfma_probe");
}
