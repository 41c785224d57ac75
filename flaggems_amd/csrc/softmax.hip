// softmax and log_softmax forward for gfx950 (LOG selects out = (x - max) - log(sum) instead of e / sum).
//
// Inner axis (K == 1): the row lives in registers as fp32 (TPR threads per row, ITERS packs of VEC
// elements per thread, same column interleave as the norm kernels), so HBM is read once and
// written once.  max and sum use wave64 butterflies plus one LDS step when a row spans waves.
// Rows that do not fit registers, or that defeat 16-byte access, use a looped online-softmax
// kernel (two reads of the row, the second from L2).
// Middle axis (K > 1): threads run along the contiguous K axis and walk N with stride K.
//
// Arithmetic follows the reference kernels: fp32, e = exp(x - max), out = e / sum.  -inf inputs
// give exact zeros; a row of only -inf gives NaN (0/0) exactly as torch does.
#include "fg_common.h"

namespace {

// v_exp_f32 (2^x) path for 16-bit inputs; libm-accurate expf when the data is fp32.
template <bool ACCURATE>
__device__ __forceinline__ float fast_exp(float x) {
  if constexpr (ACCURATE) return expf(x);
  else return __expf(x);
}

template <int TPR, typename Op>
__device__ __forceinline__ float row_reduce(float v, float* smem, int row_in_block, int t, Op op, float ident) {
  v = wave_allreduce(v, op);
  if constexpr (TPR > 64) {
    constexpr int WPR = TPR / 64;
    __syncthreads();
    if ((t & 63) == 0) smem[row_in_block * WPR + (t >> 6)] = v;
    __syncthreads();
    float s = ident;
#pragma unroll
    for (int i = 0; i < WPR; ++i) s = op(s, smem[row_in_block * WPR + i]);
    v = s;
  }
  return v;
}

template <typename TI, typename TO, int VEC, int ITERS, int TPR, bool LOG>
__global__ __launch_bounds__(TPR < 256 ? 256 : TPR) void softmax_rows_kernel(const TI* __restrict__ in,
                                                                              TO* __restrict__ out, int64_t M,
                                                                              int N) {
  constexpr int BLOCK = TPR < 256 ? 256 : TPR;
  constexpr int RPB = BLOCK / TPR;
  __shared__ float smem[BLOCK / 64];
  const int tid = threadIdx.x;
  const int row_in_block = tid / TPR;
  const int t = tid % TPR;
  const int64_t row = (int64_t)blockIdx.x * RPB + row_in_block;
  const bool row_ok = row < M;
  const TI* xr = in + row * (int64_t)N;

  float v[ITERS][VEC];
  float m = -INFINITY;
#pragma unroll
  for (int j = 0; j < ITERS; ++j) {
    const int col = (j * TPR + t) * VEC;
    if (row_ok && col < N) {
      Pack<TI, VEC> px = ld_pack_nt<TI, VEC>(xr + col);
#pragma unroll
      for (int e = 0; e < VEC; ++e) {
        v[j][e] = (float)px.v[e];
        m = fmaxf(m, v[j][e]);
      }
    } else {
#pragma unroll
      for (int e = 0; e < VEC; ++e) v[j][e] = -INFINITY;
    }
  }
  // fmaxf drops NaN operands, but exp(NaN - m) below puts the NaN into the row sum, so a NaN
  // element poisons its whole row like torch.
  m = row_reduce<TPR>(m, smem, row_in_block, t, OpMax(), -INFINITY);
  float s = 0.f;
#pragma unroll
  for (int j = 0; j < ITERS; ++j) {
#pragma unroll
    for (int e = 0; e < VEC; ++e) {
      if constexpr (LOG) {
        v[j][e] -= m;
        s += fast_exp<sizeof(TI) == 4>(v[j][e]);
      } else {
        v[j][e] = fast_exp<sizeof(TI) == 4>(v[j][e] - m);
        s += v[j][e];
      }
    }
  }
  s = row_reduce<TPR>(s, smem, row_in_block, t, OpSum(), 0.f);
  if (!row_ok) return;
  const float inv = 1.0f / s;
  const float log_s = LOG ? logf(s) : 0.f;
  TO* yr = out + row * (int64_t)N;
#pragma unroll
  for (int j = 0; j < ITERS; ++j) {
    const int col = (j * TPR + t) * VEC;
    if (col < N) {
      Pack<TO, VEC> po;
#pragma unroll
      for (int e = 0; e < VEC; ++e) {
        // 16-bit results hide the last fp32 ulp, so the reciprocal multiply is exact enough there.
        if constexpr (LOG) po.v[e] = (TO)(v[j][e] - log_s);
        else if constexpr (sizeof(TO) == 4) po.v[e] = (TO)(v[j][e] / s);
        else po.v[e] = (TO)(v[j][e] * inv);
      }
      st_pack_nt<TO, VEC>(yr + col, po);
    }
  }
}

// Any N: one block per row, online (max, sum) then a second sweep.
template <typename TI, typename TO, bool LOG>
__global__ __launch_bounds__(256) void softmax_looped_kernel(const TI* __restrict__ in, TO* __restrict__ out,
                                                            int64_t M, int64_t N) {
  __shared__ float smem[4];
  const int64_t row = blockIdx.x;
  const TI* xr = in + row * N;
  TO* yr = out + row * N;
  float m = -INFINITY, z = 0.f;
  for (int64_t c = threadIdx.x; c < N; c += 256) {
    const float x = (float)xr[c];
    const float mn = fmaxf(m, x);
    // mn == -inf only while every element seen so far is -inf: keep z at 0 instead of NaN.
    if (mn != -INFINITY) z = z * __expf(m - mn) + __expf(x - mn);
    if (x != x) z = x;
    m = mn;
  }
  const float mr = row_reduce<256>(m, smem, 0, threadIdx.x, OpMax(), -INFINITY);
  float zz = (m == -INFINITY) ? 0.f : z * __expf(m - mr);
  if (z != z) zz = z;
  const float s = row_reduce<256>(zz, smem, 0, threadIdx.x, OpSum(), 0.f);
  const float log_s = LOG ? logf(s) : 0.f;
  for (int64_t c = threadIdx.x; c < N; c += 256) {
    const float d = (float)xr[c] - mr;
    yr[c] = LOG ? (TO)(d - log_s) : (TO)(__expf(d) / s);
  }
}

// Middle axis: in viewed as [M, N, K], K contiguous.  Thread = one (m, k) column.
template <typename TI, typename TO, bool LOG>
__global__ __launch_bounds__(256) void softmax_non_inner_kernel(const TI* __restrict__ in, TO* __restrict__ out,
                                                               int64_t M, int64_t N, int64_t K) {
  const int64_t k = (int64_t)blockIdx.x * 256 + threadIdx.x;
  const int64_t mrow = blockIdx.y;
  if (k >= K) return;
  const TI* x = in + mrow * N * K + k;
  TO* y = out + mrow * N * K + k;
  float m = -INFINITY, z = 0.f;
  for (int64_t n = 0; n < N; ++n) {
    const float v = (float)x[n * K];
    const float mn = fmaxf(m, v);
    if (mn != -INFINITY) z = z * __expf(m - mn) + __expf(v - mn);
    if (v != v) z = v;
    m = mn;
  }
  const float log_z = LOG ? logf(z) : 0.f;
  for (int64_t n = 0; n < N; ++n) {
    const float d = (float)x[n * K] - m;
    y[n * K] = LOG ? (TO)(d - log_z) : (TO)(__expf(d) / z);
  }
}

template <typename TI, typename TO, int VEC, int ITERS, int TPR, bool LOG>
void launch_rows(const TI* in, TO* out, int64_t M, int N, hipStream_t st) {
  constexpr int BLOCK = TPR < 256 ? 256 : TPR;
  constexpr int RPB = BLOCK / TPR;
  hipLaunchKernelGGL((softmax_rows_kernel<TI, TO, VEC, ITERS, TPR, LOG>), dim3((unsigned)fg_cdiv(M, RPB)), dim3(BLOCK), 0,
                     st, in, out, M, N);
}

template <typename TI, typename TO, bool LOG>
int softmax_dispatch(const TI* in, TO* out, int64_t M, int64_t N, int64_t K, hipStream_t st) {
  if (K > 1) {
    FG_REQUIRE(M < 65536, FG_ERR_UNSUPPORTED, "softmax: leading extent %lld too large for the middle-axis kernel",
               (long long)M);
    hipLaunchKernelGGL((softmax_non_inner_kernel<TI, TO, LOG>), dim3((unsigned)fg_cdiv(K, 256), (unsigned)M), dim3(256), 0,
                       st, in, out, M, N, K);
    return fg_check_launch("softmax(non-inner)");
  }
  FG_REQUIRE(M < ((int64_t)1 << 31), FG_ERR_UNSUPPORTED, "softmax: M=%lld exceeds the grid limit", (long long)M);
  // One pack = 16 bytes of the narrower side so both the load and the store are single instructions.
  constexpr int VEC = 16 / sizeof(TI);
  const bool vec_ok = (N % VEC == 0) && fg_aligned(in, 16) && fg_aligned(out, sizeof(TO) * VEC);
  const int64_t packs = vec_ok ? N / VEC : 0;
#define FG_ROWS(ITERS, TPR) launch_rows<TI, TO, VEC, ITERS, TPR, LOG>(in, out, M, (int)N, st)
  if (!vec_ok || packs > 1024 * 8) {
    hipLaunchKernelGGL((softmax_looped_kernel<TI, TO, LOG>), dim3((unsigned)M), dim3(256), 0, st, in, out, M, N);
  } else if (packs <= 64) {
    FG_ROWS(1, 64);
  } else if (packs <= 128) {
    FG_ROWS(2, 64);
  } else if (packs <= 256) {
    // two packs per thread, two waves per row: 166.7 us on [131072, 2048] bf16 against 170.4 us
    // (four packs, one wave) and 175.7 us (one pack, four waves) on MI355X
    FG_ROWS(2, 128);
  } else if (packs <= 512) {
    FG_ROWS(2, 256);
  } else if (packs <= 1024) {
    FG_ROWS(2, 512);
  } else if (packs <= 2048) {
    FG_ROWS(2, 1024);
  } else if (packs <= 4096) {
    FG_ROWS(4, 1024);
  } else {
    FG_ROWS(8, 1024);
  }
#undef FG_ROWS
  return fg_check_launch("softmax");
}

template <bool LOG>
int softmax_entry(const void* in, void* out, int64_t M, int64_t N, int64_t K, int in_dtype, int out_dtype, void* stream) {
  const char* name = LOG ? "log_softmax" : "softmax";
  FG_REQUIRE(M >= 0 && N >= 0 && K >= 0, FG_ERR_INVALID, "%s: negative size", name);
  if (M == 0 || N == 0 || K == 0) return FG_OK;
  FG_REQUIRE(in && out, FG_ERR_INVALID, "%s: null pointer", name);
  FG_REQUIRE(N < ((int64_t)1 << 31), FG_ERR_UNSUPPORTED, "%s: N=%lld too large", name, (long long)N);
  FG_REQUIRE(out_dtype == in_dtype || out_dtype == FG_F32, FG_ERR_INVALID,
             "%s: out dtype %d must equal in dtype %d or be fp32", name, out_dtype, in_dtype);
  hipStream_t st = (hipStream_t)stream;
  if (in_dtype == FG_F16 && out_dtype == FG_F16) return softmax_dispatch<f16_t, f16_t, LOG>((const f16_t*)in, (f16_t*)out, M, N, K, st);
  if (in_dtype == FG_F16 && out_dtype == FG_F32) return softmax_dispatch<f16_t, float, LOG>((const f16_t*)in, (float*)out, M, N, K, st);
  if (in_dtype == FG_BF16 && out_dtype == FG_BF16) return softmax_dispatch<bf16_t, bf16_t, LOG>((const bf16_t*)in, (bf16_t*)out, M, N, K, st);
  if (in_dtype == FG_BF16 && out_dtype == FG_F32) return softmax_dispatch<bf16_t, float, LOG>((const bf16_t*)in, (float*)out, M, N, K, st);
  if (in_dtype == FG_F32 && out_dtype == FG_F32) return softmax_dispatch<float, float, LOG>((const float*)in, (float*)out, M, N, K, st);
  fg_set_error("%s: unsupported dtype pair (%d, %d)", name, in_dtype, out_dtype);
  return FG_ERR_INVALID;
}

}  // namespace

extern "C" int fg_softmax(const void* in, void* out, int64_t M, int64_t N, int64_t K, int in_dtype, int out_dtype,
                          void* stream) {
  return softmax_entry<false>(in, out, M, N, K, in_dtype, out_dtype, stream);
}

extern "C" int fg_log_softmax(const void* in, void* out, int64_t M, int64_t N, int64_t K, int in_dtype, int out_dtype,
                              void* stream) {
  return softmax_entry<true>(in, out, M, N, K, in_dtype, out_dtype, stream);
}
