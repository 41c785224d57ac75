// silu_and_mul for gfx950: out[r, c] = a[r, c] / (1 + exp(-a[r, c])) * b[r, c] in fp32.
//
// a, b and out are [rows, cols] with unit column stride and independent row strides, which covers
// the two halves of a fused gate-up projection without a copy.  Packs of 16 bytes are numbered
// row-major and dealt one per thread.  Rows that defeat 16-byte alignment keep the scheme with accesses
// declared element-aligned.
#include "fg_common.h"

namespace {

__device__ __forceinline__ float silu_mul(float x, float y) { return x / (1.0f + __expf(-x)) * y; }

template <typename T, int VEC>
__global__ __launch_bounds__(256) void silu_mul_kernel(const T* a, const T* b, T* out,
                                                      int64_t rows, int64_t cols, int64_t as, int64_t bs, int64_t os) {
  const int64_t ppr = cols / VEC;  // packs per row
  const int64_t item = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (item >= rows * ppr) return;
  const int64_t r = item / ppr;
  const int64_t c = (item - r * ppr) * VEC;
  Pack<T, VEC> x = ld_pack_nt<T, VEC>(a + r * as + c), y = ld_pack_nt<T, VEC>(b + r * bs + c), o;
#pragma unroll
  for (int e = 0; e < VEC; ++e) o.v[e] = (T)silu_mul((float)x.v[e], (float)y.v[e]);
  st_pack_nt<T, VEC>(out + r * os + c, o);
}

// Rows that defeat 16-byte alignment (odd column count, row stride or base address): the same numbering with
// ceil(cols / VEC) packs per row, 16-byte accesses declared element-aligned, the ragged last pack of a row element
// by element.
template <typename T, int VEC>
__global__ __launch_bounds__(256) void silu_mul_unaligned_kernel(const T* a, const T* b, T* out, int64_t rows, int64_t cols,
                                                                int64_t as, int64_t bs, int64_t os) {
  const int64_t ppr = (cols + VEC - 1) / VEC;
  const int64_t item = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (item >= rows * ppr) return;
  const int64_t r = item / ppr;
  const int64_t c = (item - r * ppr) * VEC;
  if (c + VEC <= cols) {
    Pack<T, VEC> x = ld_pack_u<T, VEC>(a + r * as + c), y = ld_pack_u<T, VEC>(b + r * bs + c), o;
#pragma unroll
    for (int e = 0; e < VEC; ++e) o.v[e] = (T)silu_mul((float)x.v[e], (float)y.v[e]);
    st_pack_u<T, VEC>(out + r * os + c, o);
  } else {
    for (int64_t cc = c; cc < cols; ++cc)
      out[r * os + cc] = (T)silu_mul((float)a[r * as + cc], (float)b[r * bs + cc]);
  }
}

template <typename T>
int silu_dispatch(const T* a, const T* b, T* out, int64_t rows, int64_t cols, int64_t as, int64_t bs, int64_t os,
                  hipStream_t st) {
  constexpr int VEC = 16 / sizeof(T);
  const bool vec_ok = cols % VEC == 0 && as % VEC == 0 && bs % VEC == 0 && os % VEC == 0 && fg_aligned(a, 16) &&
                      fg_aligned(b, 16) && fg_aligned(out, 16);
  const int64_t items = vec_ok ? rows * (cols / VEC) : rows * fg_cdiv(cols, VEC);
  const int64_t grid = fg_cdiv(items, 256);
  FG_REQUIRE(grid < ((int64_t)1 << 31), FG_ERR_UNSUPPORTED, "silu_and_mul: problem too large for one launch");
  if (vec_ok)
    hipLaunchKernelGGL((silu_mul_kernel<T, VEC>), dim3((unsigned)grid), dim3(256), 0, st, a, b, out, rows, cols, as, bs, os);
  else
    hipLaunchKernelGGL((silu_mul_unaligned_kernel<T, VEC>), dim3((unsigned)grid), dim3(256), 0, st, a, b, out, rows, cols, as,
                       bs, os);
  return fg_check_launch("silu_and_mul");
}

#if FG_V_SILU_GRAD_KERNEL
// Backward (variants.h, FG_V_SILU_GRAD_KERNEL): with s = 1 / (1 + exp(-a)),
//   grad_a = g * b * s * (1 + a * (1 - s)),   grad_b = g * a * s,   in fp32.
// Same numbering of 16-byte packs as the forward; five rows of independent stride.
__device__ __forceinline__ void silu_mul_grad(float x, float y, float g, float& dx, float& dy) {
  const float s = 1.0f / (1.0f + __expf(-x));
  dx = s * (1.0f + x * (1.0f - s)) * g * y;
  dy = g * (x * s);
}

struct SiluGradArgs {
  const void *a, *b, *g;
  void *da, *db;
  int64_t rows, cols, as, bs, gs, das, dbs;
};

template <typename T, int VEC, bool ALIGNED>
__global__ __launch_bounds__(256) void silu_mul_grad_kernel(SiluGradArgs k) {
  const T *a = (const T*)k.a, *b = (const T*)k.b, *g = (const T*)k.g;
  T *da = (T*)k.da, *db = (T*)k.db;
  const int64_t ppr = ALIGNED ? k.cols / VEC : (k.cols + VEC - 1) / VEC;
  const int64_t item = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (item >= k.rows * ppr) return;
  const int64_t r = item / ppr;
  const int64_t c = (item - r * ppr) * VEC;
  if (ALIGNED || c + VEC <= k.cols) {
    Pack<T, VEC> x, y, go, ox, oy;
    if constexpr (ALIGNED) {
      x = ld_pack_nt<T, VEC>(a + r * k.as + c); y = ld_pack_nt<T, VEC>(b + r * k.bs + c); go = ld_pack_nt<T, VEC>(g + r * k.gs + c);
    } else {
      x = ld_pack_u<T, VEC>(a + r * k.as + c); y = ld_pack_u<T, VEC>(b + r * k.bs + c); go = ld_pack_u<T, VEC>(g + r * k.gs + c);
    }
#pragma unroll
    for (int e = 0; e < VEC; ++e) {
      float dx, dy;
      silu_mul_grad((float)x.v[e], (float)y.v[e], (float)go.v[e], dx, dy);
      ox.v[e] = (T)dx;
      oy.v[e] = (T)dy;
    }
    if constexpr (ALIGNED) {
      st_pack_nt<T, VEC>(da + r * k.das + c, ox); st_pack_nt<T, VEC>(db + r * k.dbs + c, oy);
    } else {
      st_pack_u<T, VEC>(da + r * k.das + c, ox); st_pack_u<T, VEC>(db + r * k.dbs + c, oy);
    }
  } else {
    for (int64_t cc = c; cc < k.cols; ++cc) {
      float dx, dy;
      silu_mul_grad((float)a[r * k.as + cc], (float)b[r * k.bs + cc], (float)g[r * k.gs + cc], dx, dy);
      da[r * k.das + cc] = (T)dx;
      db[r * k.dbs + cc] = (T)dy;
    }
  }
}

template <typename T>
int silu_grad_dispatch(const SiluGradArgs& k, hipStream_t st) {
  constexpr int VEC = 16 / sizeof(T);
  const bool vec_ok = k.cols % VEC == 0 && k.as % VEC == 0 && k.bs % VEC == 0 && k.gs % VEC == 0 && k.das % VEC == 0 &&
                      k.dbs % VEC == 0 && fg_aligned(k.a, 16) && fg_aligned(k.b, 16) && fg_aligned(k.g, 16) &&
                      fg_aligned(k.da, 16) && fg_aligned(k.db, 16);
  const int64_t items = vec_ok ? k.rows * (k.cols / VEC) : k.rows * fg_cdiv(k.cols, VEC);
  const int64_t grid = fg_cdiv(items, 256);
  FG_REQUIRE(grid < ((int64_t)1 << 31), FG_ERR_UNSUPPORTED, "silu_and_mul_backward: problem too large for one launch");
  if (vec_ok) hipLaunchKernelGGL((silu_mul_grad_kernel<T, VEC, true>), dim3((unsigned)grid), dim3(256), 0, st, k);
  else hipLaunchKernelGGL((silu_mul_grad_kernel<T, VEC, false>), dim3((unsigned)grid), dim3(256), 0, st, k);
  return fg_check_launch("silu_and_mul_backward");
}
#endif  // FG_V_SILU_GRAD_KERNEL

}  // namespace

extern "C" int fg_silu_and_mul_backward(const void* a, const void* b, const void* grad_out, void* grad_a, void* grad_b,
                                        int64_t rows, int64_t cols, int64_t a_row_stride, int64_t b_row_stride,
                                        int64_t g_row_stride, int64_t ga_row_stride, int64_t gb_row_stride, int dtype,
                                        void* stream) {
  FG_REQUIRE(rows >= 0 && cols >= 0, FG_ERR_INVALID, "silu_and_mul_backward: negative size");
  FG_REQUIRE(dtype == FG_F16 || dtype == FG_BF16 || dtype == FG_F32, FG_ERR_INVALID,
             "silu_and_mul_backward: unsupported dtype %d", dtype);
#if FG_V_SILU_GRAD_KERNEL
  if (rows == 0 || cols == 0) return FG_OK;
  FG_REQUIRE(a && b && grad_out && grad_a && grad_b, FG_ERR_INVALID, "silu_and_mul_backward: null pointer");
  const SiluGradArgs k = {a, b, grad_out, grad_a, grad_b, rows, cols, a_row_stride, b_row_stride, g_row_stride,
                          ga_row_stride, gb_row_stride};
  hipStream_t st = (hipStream_t)stream;
  if (dtype == FG_F16) return silu_grad_dispatch<f16_t>(k, st);
  if (dtype == FG_BF16) return silu_grad_dispatch<bf16_t>(k, st);
  return silu_grad_dispatch<float>(k, st);
#else
  (void)a; (void)b; (void)grad_out; (void)grad_a; (void)grad_b; (void)a_row_stride; (void)b_row_stride;
  (void)g_row_stride; (void)ga_row_stride; (void)gb_row_stride; (void)stream;
  fg_set_error("silu_and_mul_backward: the kernel is not part of this build (FG_V_SILU_GRAD_KERNEL, csrc/variants.h)");
  return FG_ERR_UNSUPPORTED;
#endif
}

extern "C" int fg_silu_and_mul(const void* a, const void* b, void* out, int64_t rows, int64_t cols,
                               int64_t a_row_stride, int64_t b_row_stride, int64_t o_row_stride, int dtype,
                               void* stream) {
  FG_REQUIRE(rows >= 0 && cols >= 0, FG_ERR_INVALID, "silu_and_mul: negative size");
  if (rows == 0 || cols == 0) return FG_OK;
  FG_REQUIRE(a && b && out, FG_ERR_INVALID, "silu_and_mul: null pointer");
  hipStream_t st = (hipStream_t)stream;
  switch (dtype) {
    case FG_F16:
      return silu_dispatch((const f16_t*)a, (const f16_t*)b, (f16_t*)out, rows, cols, a_row_stride, b_row_stride,
                           o_row_stride, st);
    case FG_BF16:
      return silu_dispatch((const bf16_t*)a, (const bf16_t*)b, (bf16_t*)out, rows, cols, a_row_stride, b_row_stride,
                           o_row_stride, st);
    case FG_F32:
      return silu_dispatch((const float*)a, (const float*)b, (float*)out, rows, cols, a_row_stride, b_row_stride,
                           o_row_stride, st);
  }
  fg_set_error("silu_and_mul: unsupported dtype %d", dtype);
  return FG_ERR_INVALID;
}
