// 2-D transpose of 16- and 32-bit elements for gfx950: dst[c, r] = src[r, c].
//
// mm's host side uses it to turn a column-major A into the K-contiguous layout that the direct-to-LDS and
// skinny GEMM kernels read.  A workgroup moves a 64 x 64 tile through LDS: 16-byte loads along the source's
// contiguous axis, 16-byte stores along the destination's.  Tiles on a ragged edge, and tensors whose rows
// are not 16-byte aligned, go element by element with bounds checks.
#include "fg_common.h"

namespace {

constexpr int kTS = 64;  // tile edge in elements

template <typename U, bool VEC_SRC, bool VEC_DST>
__global__ __launch_bounds__(256) void transpose_kernel(const U* __restrict__ src, U* __restrict__ dst, int64_t rows,
                                                       int64_t cols, int64_t ss, int64_t ds) {
  constexpr int EPC = 16 / sizeof(U);      // elements per 16-byte chunk
  constexpr int CPT = kTS / EPC;           // chunks per tile row
  constexpr int PITCH = kTS + 4 / sizeof(U);  // one dword of padding per tile row
  __shared__ U tile[kTS][PITCH];
  const int64_t r0 = (int64_t)blockIdx.y * kTS, c0 = (int64_t)blockIdx.x * kTS;
  const bool full = r0 + kTS <= rows && c0 + kTS <= cols;
  for (int idx = threadIdx.x; idx < kTS * CPT; idx += 256) {
    const int row = idx / CPT, ch = idx % CPT;
    const int64_t r = r0 + row, c = c0 + ch * EPC;
    if (VEC_SRC && full) {
      const Pack<U, EPC> p = ld_pack_nt<U, EPC>(src + r * ss + c);
#pragma unroll
      for (int e = 0; e < EPC; ++e) tile[row][ch * EPC + e] = p.v[e];
    } else {
#pragma unroll
      for (int e = 0; e < EPC; ++e)
        if (r < rows && c + e < cols) tile[row][ch * EPC + e] = src[r * ss + c + e];
    }
  }
  __syncthreads();
  for (int idx = threadIdx.x; idx < kTS * CPT; idx += 256) {
    const int col = idx / CPT, ch = idx % CPT;  // destination row c0 + col, destination columns r0 + ch * EPC ...
    const int64_t dr = c0 + col, dc = r0 + ch * EPC;
    if (VEC_DST && full) {
      Pack<U, EPC> p;
#pragma unroll
      for (int e = 0; e < EPC; ++e) p.v[e] = tile[ch * EPC + e][col];
      st_pack_nt<U, EPC>(dst + dr * ds + dc, p);
    } else {
#pragma unroll
      for (int e = 0; e < EPC; ++e)
        if (dr < cols && dc + e < rows) dst[dr * ds + dc + e] = tile[ch * EPC + e][col];
    }
  }
}

template <typename U>
int transpose_dispatch(const U* src, U* dst, int64_t rows, int64_t cols, int64_t ss, int64_t ds, hipStream_t st) {
  constexpr int EPC = 16 / sizeof(U);
  const bool vs = ss % EPC == 0 && fg_aligned(src, 16), vd = ds % EPC == 0 && fg_aligned(dst, 16);
  const dim3 grid((unsigned)fg_cdiv(cols, kTS), (unsigned)fg_cdiv(rows, kTS));
#define FG_T(A, B) hipLaunchKernelGGL((transpose_kernel<U, A, B>), grid, dim3(256), 0, st, src, dst, rows, cols, ss, ds)
  if (vs && vd) FG_T(true, true);
  else if (vs) FG_T(true, false);
  else if (vd) FG_T(false, true);
  else FG_T(false, false);
#undef FG_T
  return fg_check_launch("transpose2d");
}

}  // namespace

extern "C" int fg_transpose2d(const void* src, void* dst, int64_t rows, int64_t cols, int64_t src_row_stride,
                              int64_t dst_row_stride, int elem_bytes, void* stream) {
  FG_REQUIRE(rows >= 0 && cols >= 0, FG_ERR_INVALID, "transpose2d: negative size");
  if (rows == 0 || cols == 0) return FG_OK;
  FG_REQUIRE(src && dst, FG_ERR_INVALID, "transpose2d: null pointer");
  FG_REQUIRE(src_row_stride >= cols && dst_row_stride >= rows, FG_ERR_INVALID,
             "transpose2d: a row stride is smaller than its row");
  FG_REQUIRE(fg_cdiv(rows, kTS) < 65536 && fg_cdiv(cols, kTS) < ((int64_t)1 << 31), FG_ERR_UNSUPPORTED,
             "transpose2d: %lld x %lld exceeds the grid limits", (long long)rows, (long long)cols);
  hipStream_t st = (hipStream_t)stream;
  if (elem_bytes == 2)
    return transpose_dispatch((const uint16_t*)src, (uint16_t*)dst, rows, cols, src_row_stride, dst_row_stride, st);
  if (elem_bytes == 4)
    return transpose_dispatch((const uint32_t*)src, (uint32_t*)dst, rows, cols, src_row_stride, dst_row_stride, st);
  fg_set_error("transpose2d: element size %d", elem_bytes);
  return FG_ERR_INVALID;
}
