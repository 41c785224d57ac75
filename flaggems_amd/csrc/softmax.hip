// softmax and log_softmax forward for gfx950 (LOG selects out = (x - max) - log(sum) instead of e / sum).
//
// Inner axis (K == 1): the row lives in registers as fp32 (TPR threads per row, ITERS packs of VEC
// elements per thread, same column interleave as the norm kernels), so HBM is read once and
// written once.  max and sum use wave64 butterflies plus one LDS step when a row spans waves.
// Rows that do not fit registers, or whose start is only element-aligned, take a two-sweep online-softmax
// kernel with one workgroup per row (the second read comes from L2), or, up to 1024 elements, a kernel
// with one wave per row.
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

  // All packs of the thread are requested before the first is used.  The loads are unconditional (a pack past the
  // end of the row or of the matrix is read from the start of the input and discarded): with a branch around each
  // load the compiler finishes pack j, wait included, before it requests pack j + 1, one trip to memory per pack.
  // (variant FG_V_ROWS_UPFRONT, variants.h; off: every pack is loaded where it is used, under its bounds check)
  constexpr bool UPFRONT = FG_V_ROWS_UPFRONT != 0;
  Pack<TI, VEC> px[ITERS];
  if constexpr (UPFRONT) {
#pragma unroll
    for (int j = 0; j < ITERS; ++j) {
      const int col = (j * TPR + t) * VEC;
      px[j] = ld_pack_nt<TI, VEC>(row_ok && col < N ? xr + col : in);
    }
    // the output pointer is fetched with the other kernel arguments, not by a scalar load behind the last reduction
    asm volatile("" : : "s"(out));
  }
  float v[ITERS][VEC];
  float m = -INFINITY;
#pragma unroll
  for (int j = 0; j < ITERS; ++j) {
    const int col = (j * TPR + t) * VEC;
    if constexpr (UPFRONT) {
      const bool ok = row_ok && col < N;
#pragma unroll
      for (int e = 0; e < VEC; ++e) {
        v[j][e] = ok ? (float)px[j].v[e] : -INFINITY;
        m = fmaxf(m, v[j][e]);
      }
    } else if (row_ok && col < N) {
      px[j] = ld_pack_nt<TI, VEC>(xr + col);
#pragma unroll
      for (int e = 0; e < VEC; ++e) {
        v[j][e] = (float)px[j].v[e];
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

// Rows that do not fit the registers of one workgroup (more than 8192 packs of 16 bytes) or whose
// start is only element-aligned (N not a multiple of the pack): one workgroup per row, two sweeps.  The first keeps a
// running (max, sum) per thread, rescaled once per 16-byte pack; the second reads the row again (from L2 for all but
// the longest rows), and writes.  Loads and stores are 16-byte accesses declared element-aligned; up to four of them
// per thread are in flight.  The N % VEC elements behind the last full pack go one per thread.
template <typename TI, typename TO, bool LOG, int BLOCK>
__global__ __launch_bounds__(BLOCK) void softmax_long_kernel(const TI* __restrict__ in, TO* __restrict__ out, int64_t M,
                                                            int64_t N) {
  constexpr int VEC = 16 / sizeof(TI);
  constexpr int UNROLL = 4;
  __shared__ float smem[BLOCK / 64];
  const int64_t row = blockIdx.x;
  const TI* xr = in + row * N;
  TO* yr = out + row * N;
  const int64_t packs = N / VEC;
  const int64_t tail0 = packs * VEC;
  const int t = threadIdx.x;
  float m = -INFINITY, z = 0.f;
  for (int64_t p0 = t; p0 < packs; p0 += (int64_t)BLOCK * UNROLL) {
    Pack<TI, VEC> px[UNROLL];
#pragma unroll
    for (int u = 0; u < UNROLL; ++u)
      if (p0 + (int64_t)u * BLOCK < packs) px[u] = ld_pack_u<TI, VEC>(xr + (p0 + (int64_t)u * BLOCK) * VEC);
#pragma unroll
    for (int u = 0; u < UNROLL; ++u) {
      if (p0 + (int64_t)u * BLOCK < packs) {
        float x[VEC];
        float pm = -INFINITY;
#pragma unroll
        for (int e = 0; e < VEC; ++e) {
          x[e] = (float)px[u].v[e];
          pm = fmaxf(pm, x[e]);
        }
        const float mn = fmaxf(m, pm);
        // mn == -inf only while every element seen so far is -inf: keep z at 0 instead of NaN.
        if (mn != -INFINITY) {
          float acc = 0.f;
#pragma unroll
          for (int e = 0; e < VEC; ++e) acc += __expf(x[e] - mn);
          z = z * __expf(m - mn) + acc;
        }
#pragma unroll
        for (int e = 0; e < VEC; ++e)
          if (x[e] != x[e]) z = x[e];  // fmaxf drops a NaN: put it into the sum by hand
        m = mn;
      }
    }
  }
  if (t < N - tail0) {
    const float x = (float)xr[tail0 + t];
    const float mn = fmaxf(m, x);
    if (mn != -INFINITY) z = z * __expf(m - mn) + __expf(x - mn);
    if (x != x) z = x;
    m = mn;
  }
  const float mr = row_reduce<BLOCK>(m, smem, 0, t, OpMax(), -INFINITY);
  float zz = (m == -INFINITY) ? 0.f : z * __expf(m - mr);
  if (z != z) zz = z;
  const float s = row_reduce<BLOCK>(zz, smem, 0, t, OpSum(), 0.f);
  const float log_s = LOG ? logf(s) : 0.f;
  const float inv = 1.0f / s;
  auto result = [&](float x) -> TO {
    const float d = x - mr;
    if constexpr (LOG) return (TO)(d - log_s);
    else if constexpr (sizeof(TO) == 4) return (TO)(__expf(d) / s);
    else return (TO)(__expf(d) * inv);
  };
  for (int64_t p0 = t; p0 < packs; p0 += (int64_t)BLOCK * UNROLL) {
    Pack<TI, VEC> px[UNROLL];
#pragma unroll
    for (int u = 0; u < UNROLL; ++u)
      if (p0 + (int64_t)u * BLOCK < packs) px[u] = ld_pack_u<TI, VEC>(xr + (p0 + (int64_t)u * BLOCK) * VEC);
#pragma unroll
    for (int u = 0; u < UNROLL; ++u) {
      if (p0 + (int64_t)u * BLOCK < packs) {
        Pack<TO, VEC> po;
#pragma unroll
        for (int e = 0; e < VEC; ++e) po.v[e] = result((float)px[u].v[e]);
        st_pack_u<TO, VEC>(yr + (p0 + (int64_t)u * BLOCK) * VEC, po);
      }
    }
  }
  if (t < N - tail0) yr[tail0 + t] = result((float)xr[tail0 + t]);
}

// Short rows whose start is only element-aligned (N <= 1024, not a multiple of the pack): one wave per row, element
// j * 64 + lane in register j, no LDS and no barrier.
template <typename TI, typename TO, bool LOG, int ITERS>
__global__ __launch_bounds__(256) void softmax_short_kernel(const TI* __restrict__ in, TO* __restrict__ out, int64_t M,
                                                           int N) {
  const int lane = threadIdx.x & 63;
  const int64_t row = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
  if (row >= M) return;  // the whole wave leaves
  const TI* xr = in + row * (int64_t)N;
  TO* yr = out + row * (int64_t)N;
  // unconditional loads (a column past the end reads the row's first element and is discarded): with a branch
  // around each the compiler waits for one before it requests the next, up to ITERS trips to memory per row
  // (variant FG_V_SHORT_UPFRONT, variants.h; off: every element is loaded where it is used, under its bounds check)
  constexpr bool UPFRONT = FG_V_SHORT_UPFRONT != 0;
  TI raw[ITERS];
  if constexpr (UPFRONT) {
#pragma unroll
    for (int j = 0; j < ITERS; ++j) {
      const int c = j * 64 + lane;
      raw[j] = xr[c < N ? c : 0];
    }
  }
  float v[ITERS];
  float m = -INFINITY;
#pragma unroll
  for (int j = 0; j < ITERS; ++j) {
    const int c = j * 64 + lane;
    if constexpr (UPFRONT) v[j] = c < N ? (float)raw[j] : -INFINITY;
    else v[j] = c < N ? (float)xr[c] : -INFINITY;
    m = fmaxf(m, v[j]);
  }
  m = wave_max(m);
  float s = 0.f;
#pragma unroll
  for (int j = 0; j < ITERS; ++j) {
    if constexpr (LOG) {
      v[j] -= m;
      s += fast_exp<sizeof(TI) == 4>(v[j]);
    } else {
      v[j] = fast_exp<sizeof(TI) == 4>(v[j] - m);
      s += v[j];
    }
  }
  s = wave_sum(s);
  const float inv = 1.0f / s;
  const float log_s = LOG ? logf(s) : 0.f;
#pragma unroll
  for (int j = 0; j < ITERS; ++j) {
    const int c = j * 64 + lane;
    if (c < N) {
      if constexpr (LOG) yr[c] = (TO)(v[j] - log_s);
      else if constexpr (sizeof(TO) == 4) yr[c] = (TO)(v[j] / s);
      else yr[c] = (TO)(v[j] * inv);
    }
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
  if (!vec_ok && N <= 1024) {
#define FG_SHORT(ITERS)                                                                                                  \
  hipLaunchKernelGGL((softmax_short_kernel<TI, TO, LOG, ITERS>), dim3((unsigned)fg_cdiv(M, 4)), dim3(256), 0, st, in, out, \
                     M, (int)N)
    if (N <= 64) FG_SHORT(1);
    else if (N <= 128) FG_SHORT(2);
    else if (N <= 256) FG_SHORT(4);
    else if (N <= 512) FG_SHORT(8);
    else FG_SHORT(16);
#undef FG_SHORT
  } else if (!vec_ok || packs > 1024 * 8) {
    if (N >= 2048)
      hipLaunchKernelGGL((softmax_long_kernel<TI, TO, LOG, 1024>), dim3((unsigned)M), dim3(1024), 0, st, in, out, M, N);
    else
      hipLaunchKernelGGL((softmax_long_kernel<TI, TO, LOG, 256>), dim3((unsigned)M), dim3(256), 0, st, in, out, M, N);
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
