// Row-wise backward passes for gfx950: softmax, log_softmax and rms_norm.
//
// All three have the shape of their forward kernels: two inputs in the forward's row layout, one
// fp32 sum per row, one output.
//   softmax:      dx = y * (dy - sum(y * dy))
//   log_softmax:  dx = dy - exp(y) * sum(dy)
//   rms_norm:     g = dy * w, xh = x * inv_rms, dx = (g - xh * sum(xh * g) / N) * inv_rms
// Inner axis (K == 1): the two rows live in registers as fp32 (TPR threads per row, ITERS packs of
// VEC elements per thread), so HBM is read once per input and written once.  Rows that do not fit,
// or that defeat 16-byte access, use a looped kernel that reads the row twice (the second time from
// L2).  Middle axis (softmax only, K > 1): one thread per (m, k) column, walking N with stride K.
// The weight gradient of rms_norm is a column sum over all rows.  The rms kernel therefore walks a
// group of consecutive rows per workgroup and keeps the running column sums of x * inv_rms * dy for its
// columns in registers; each group leaves one fp32 partial row and the caller adds the partial rows up.
// x and dy are read once for both gradients (3 accesses per element instead of 5).
#include "fg_common.h"

namespace fgk {
int num_cus(int device);  // gemm.hip
}

namespace {

enum { BWD_SOFTMAX = 0, BWD_LOG_SOFTMAX = 1, BWD_RMS = 2 };

// Barrier that orders LDS traffic only: global loads issued before it (the next row's prefetch) stay in flight,
// where __syncthreads() would wait for them.
__device__ __forceinline__ void lds_barrier() {
  __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup", "local");
  __builtin_amdgcn_s_barrier();
  __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup", "local");
}

// LIGHT: the barriers order LDS traffic only (for the kernel that keeps global loads in flight across them).
template <int TPR, bool LIGHT = false>
__device__ __forceinline__ float row_sum(float v, float* smem, int row_in_block, int t) {
  v = wave_sum(v);
  if constexpr (TPR > 64) {
    constexpr int WPR = TPR / 64;  // waves per row
    if constexpr (LIGHT) lds_barrier();
    else __syncthreads();
    if ((t & 63) == 0) smem[row_in_block * WPR + (t >> 6)] = v;
    if constexpr (LIGHT) lds_barrier();
    else __syncthreads();
    float s = 0.f;
#pragma unroll
    for (int i = 0; i < WPR; ++i) s += smem[row_in_block * WPR + i];
    v = s;
  }
  return v;
}

template <typename T> __device__ __forceinline__ float exp_like_forward(float x) {
  if constexpr (sizeof(T) == 4) return expf(x);
  else return __expf(x);
}

// softmax / log_softmax; a: the forward's output y, g: dy.
template <typename TI, typename TO, int VEC, int ITERS, int TPR, int MODE>
__global__ __launch_bounds__(TPR < 256 ? 256 : TPR) void bwd_rows_kernel(const TI* __restrict__ a,
                                                                          const TI* __restrict__ g,
                                                                          TO* __restrict__ out, int64_t M, int N) {
  constexpr int BLOCK = TPR < 256 ? 256 : TPR;
  constexpr int RPB = BLOCK / TPR;
  __shared__ float smem[BLOCK / 64];
  const int tid = threadIdx.x;
  const int row_in_block = tid / TPR;
  const int t = tid % TPR;
  const int64_t row = (int64_t)blockIdx.x * RPB + row_in_block;
  const bool row_ok = row < M;
  const TI* ar = a + row * (int64_t)N;
  const TI* gr = g + row * (int64_t)N;
  // All packs of the thread are requested before the first is used; the loads are unconditional (a pack past the end
  // of the row or of the matrix is read from the start of the input and discarded).  With a branch around each pair
  // of loads the compiler finishes pack j, wait included, before it requests pack j + 1.
  // (variant FG_V_ROWS_UPFRONT, variants.h; off: every pair of packs is loaded where it is used, under its bounds check)
  constexpr bool UPFRONT = FG_V_ROWS_UPFRONT != 0;
  Pack<TI, VEC> pa[ITERS], pg[ITERS];
  if constexpr (UPFRONT) {
#pragma unroll
    for (int j = 0; j < ITERS; ++j) {
      const int col = (j * TPR + t) * VEC;
      const bool ok = row_ok && col < N;
      pa[j] = ld_pack_nt<TI, VEC>(ok ? ar + col : a);
      pg[j] = ld_pack_nt<TI, VEC>(ok ? gr + col : g);
    }
    asm volatile("" : : "s"(out));  // fetched with the other kernel arguments, not behind the reduction
    if constexpr (sizeof(TI) * VEC == 16) {
      // (the registers pass through an empty asm: without it the compiler moves a load whose value is only needed
      // behind the reduction down to that use, where it costs a trip to memory of its own)
#pragma unroll
      for (int j = 0; j < ITERS; ++j)
        asm volatile("" : "+v"(*reinterpret_cast<u32x4*>(&pa[j])), "+v"(*reinterpret_cast<u32x4*>(&pg[j])));
    }
  }
  float va[ITERS][VEC], vg[ITERS][VEC];
  float s = 0.f;
#pragma unroll
  for (int j = 0; j < ITERS; ++j) {
    const int col = (j * TPR + t) * VEC;
    if constexpr (UPFRONT) {
      const bool ok = row_ok && col < N;
#pragma unroll
      for (int e = 0; e < VEC; ++e) {
        va[j][e] = ok ? (float)pa[j].v[e] : 0.f;
        vg[j][e] = ok ? (float)pg[j].v[e] : 0.f;
        s += MODE == BWD_SOFTMAX ? va[j][e] * vg[j][e] : vg[j][e];
      }
    } else if (row_ok && col < N) {
      pa[j] = ld_pack_nt<TI, VEC>(ar + col);
      pg[j] = ld_pack_nt<TI, VEC>(gr + col);
#pragma unroll
      for (int e = 0; e < VEC; ++e) {
        va[j][e] = (float)pa[j].v[e];
        vg[j][e] = (float)pg[j].v[e];
        s += MODE == BWD_SOFTMAX ? va[j][e] * vg[j][e] : vg[j][e];
      }
    } else {
#pragma unroll
      for (int e = 0; e < VEC; ++e) va[j][e] = vg[j][e] = 0.f;
    }
  }
  s = row_sum<TPR>(s, smem, row_in_block, t);
  if (!row_ok) return;
  TO* orow = out + row * (int64_t)N;
#pragma unroll
  for (int j = 0; j < ITERS; ++j) {
    const int col = (j * TPR + t) * VEC;
    if (col < N) {
      Pack<TO, VEC> po;
#pragma unroll
      for (int e = 0; e < VEC; ++e) {
        float r;
        if constexpr (MODE == BWD_SOFTMAX) r = va[j][e] * (vg[j][e] - s);
        else r = vg[j][e] - exp_like_forward<TI>(va[j][e]) * s;
        po.v[e] = (TO)r;
      }
      st_pack_nt<TO, VEC>(orow + col, po);
    }
  }
}

// rms_norm: dx for the rows of one group, and the group's column sums for the weight gradient.
// Group = rows [group * rows_per_group, ...); a block holds RPB groups (one per TPR threads).  Every thread
// of a block runs the same number of iterations, so the barriers inside row_sum are uniform.  The packs of a
// row are requested one row ahead (two buffers, the loop advances two rows per trip), so that they travel while
// the current row is reduced.
// The loads are unconditional (a row past the end is read from the last row, a column past the end from column
// 0, both discarded later): without branches around them the compiler's wait counts stay exact and the requests of
// the next row really remain in flight across the reduction.
template <typename T, int VEC, int ITERS, int TPR, bool CLAMP>
__device__ __forceinline__ void rms_bwd_fetch(Pack<T, VEC> (&px)[ITERS], Pack<T, VEC> (&pd)[ITERS], float& pinv, bool ok,
                                              int64_t row, int64_t M, const T* __restrict__ x, const T* __restrict__ dy,
                                              const float* __restrict__ inv_rms, int N, int t) {
  if constexpr (CLAMP) {
    const int64_t rr = ok ? row : M - 1;
    const float v = inv_rms[rr];
    pinv = ok ? v : 0.f;
#pragma unroll
    for (int j = 0; j < ITERS; ++j) {
      const int col = (j * TPR + t) * VEC;
      const int cc = col < N ? col : 0;
      px[j] = ld_pack_nt<T, VEC>(x + rr * (int64_t)N + cc);
      pd[j] = ld_pack_nt<T, VEC>(dy + rr * (int64_t)N + cc);
    }
  } else {
    pinv = ok ? inv_rms[row] : 0.f;
#pragma unroll
    for (int j = 0; j < ITERS; ++j) {
      const int col = (j * TPR + t) * VEC;
      if (ok && col < N) {
        px[j] = ld_pack_nt<T, VEC>(x + row * (int64_t)N + col);
        pd[j] = ld_pack_nt<T, VEC>(dy + row * (int64_t)N + col);
      } else {
#if FG_V_RMS_BWD_ZERO_PACK
        // (variant, variants.h: whole packs, not element by element: a pack that is written both as one 16-byte value
        // and as 16-bit elements is left in scratch memory by the compiler)
        Pack<T, VEC> zero;
        __builtin_memset(&zero, 0, sizeof(zero));
        px[j] = zero;
        pd[j] = zero;
#else
#pragma unroll
        for (int e = 0; e < VEC; ++e) px[j].v[e] = pd[j].v[e] = (T)0.f;
#endif
      }
    }
  }
}

template <typename T, int VEC, int ITERS, int TPR, bool LIGHT>
__device__ __forceinline__ void rms_bwd_row(const Pack<T, VEC> (&cx)[ITERS], const Pack<T, VEC> (&cd)[ITERS], float inv,
                                            bool row_ok, int64_t row, const float (&wv)[ITERS][VEC],
                                            float (&acc)[ITERS][VEC], float* smem, T* __restrict__ dx, int N, int t,
                                            int row_in_block) {
  float xh[ITERS][VEC], d[ITERS][VEC];
  float s = 0.f;
#pragma unroll
  for (int j = 0; j < ITERS; ++j) {
    const bool col_ok = (j * TPR + t) * VEC < N;
#pragma unroll
    for (int e = 0; e < VEC; ++e) {
      xh[j][e] = col_ok ? (float)cx[j].v[e] * inv : 0.f;
      d[j][e] = col_ok ? (float)cd[j].v[e] : 0.f;
      s += xh[j][e] * d[j][e] * wv[j][e];
    }
  }
  s = row_sum<TPR, LIGHT>(s, smem, row_in_block, t);
  const float mean = s / (float)N;
  if (row_ok) {
#pragma unroll
    for (int j = 0; j < ITERS; ++j) {
      const int col = (j * TPR + t) * VEC;
      if (col < N) {
        Pack<T, VEC> po;
#pragma unroll
        for (int e = 0; e < VEC; ++e) {
          po.v[e] = (T)((d[j][e] * wv[j][e] - xh[j][e] * mean) * inv);
          acc[j][e] += xh[j][e] * d[j][e];
        }
        st_pack_nt<T, VEC>(dx + row * (int64_t)N + col, po);
      }
    }
  }
}

template <typename T, int VEC, int ITERS, int TPR, bool PREFETCH>
__global__ __launch_bounds__(TPR < 256 ? 256 : TPR) void rms_bwd_rows_kernel(
    const T* __restrict__ x, const T* __restrict__ dy, const T* __restrict__ w, const float* __restrict__ inv_rms,
    T* __restrict__ dx, float* __restrict__ dw_partial, int64_t partial_rows, int64_t M, int N, int rows_per_group) {
  constexpr int BLOCK = TPR < 256 ? 256 : TPR;
  constexpr int RPB = BLOCK / TPR;
  __shared__ float smem[BLOCK / 64];
  const int tid = threadIdx.x;
  const int row_in_block = tid / TPR;
  const int t = tid % TPR;
  const int64_t group = (int64_t)blockIdx.x * RPB + row_in_block;
  const int64_t r0 = group * rows_per_group;

  float wv[ITERS][VEC], acc[ITERS][VEC];
#pragma unroll
  for (int j = 0; j < ITERS; ++j) {
    const int col = (j * TPR + t) * VEC;
    if (w != nullptr && col < N) {
      const Pack<T, VEC> pw = ld_pack<T, VEC>(w + col);
#pragma unroll
      for (int e = 0; e < VEC; ++e) wv[j][e] = (float)pw.v[e];
    } else {
#pragma unroll
      for (int e = 0; e < VEC; ++e) wv[j][e] = 1.0f;
    }
#pragma unroll
    for (int e = 0; e < VEC; ++e) acc[j][e] = 0.f;
  }

  if constexpr (PREFETCH) {
    Pack<T, VEC> ax[ITERS], ad[ITERS], bx[ITERS], bd[ITERS];
    float ainv, binv = 0.f;
    rms_bwd_fetch<T, VEC, ITERS, TPR, true>(ax, ad, ainv, r0 < M, r0, M, x, dy, inv_rms, N, t);
    for (int i = 0; i < rows_per_group; i += 2) {
      const int64_t row = r0 + i;
      const bool second = i + 1 < rows_per_group;  // uniform over the block, like every branch in this loop
      if (second) rms_bwd_fetch<T, VEC, ITERS, TPR, true>(bx, bd, binv, row + 1 < M, row + 1, M, x, dy, inv_rms, N, t);
      rms_bwd_row<T, VEC, ITERS, TPR, true>(ax, ad, ainv, row < M, row, wv, acc, smem, dx, N, t, row_in_block);
      if (second) {
        if (i + 2 < rows_per_group)
          rms_bwd_fetch<T, VEC, ITERS, TPR, true>(ax, ad, ainv, row + 2 < M, row + 2, M, x, dy, inv_rms, N, t);
        rms_bwd_row<T, VEC, ITERS, TPR, true>(bx, bd, binv, row + 1 < M, row + 1, wv, acc, smem, dx, N, t, row_in_block);
      }
    }
  } else {
    // one row per group (no weight gradient wanted: a leaner kernel, three workgroups per CU instead of two), or
    // two packs per thread, where a second buffer would not fit the registers of a 1024-thread block: fetch and use
    for (int i = 0; i < rows_per_group; ++i) {
      const int64_t row = r0 + i;
      Pack<T, VEC> ax[ITERS], ad[ITERS];
      float ainv;
      rms_bwd_fetch<T, VEC, ITERS, TPR, false>(ax, ad, ainv, row < M, row, M, x, dy, inv_rms, N, t);
      rms_bwd_row<T, VEC, ITERS, TPR, false>(ax, ad, ainv, row < M, row, wv, acc, smem, dx, N, t, row_in_block);
    }
  }
  if (dw_partial != nullptr && group < partial_rows) {
#pragma unroll
    for (int j = 0; j < ITERS; ++j) {
      const int col = (j * TPR + t) * VEC;
      if (col < N) {
        Pack<float, VEC> pa;
#pragma unroll
        for (int e = 0; e < VEC; ++e) pa.v[e] = acc[j][e];
        st_pack<float, VEC>(dw_partial + group * (int64_t)N + col, pa);
      }
    }
  }
}

// Rows too long for the registers of one workgroup, or whose start is only element-aligned: one workgroup per row,
// two sweeps of element-aligned 16-byte accesses (the second sweep reads from L2 for all but the longest rows); the
// N % VEC elements behind the last full pack go one per thread.
template <typename TI, typename TO, int MODE, int BLOCK>
__global__ __launch_bounds__(BLOCK) void bwd_looped_kernel(const TI* __restrict__ a, const TI* __restrict__ g,
                                                          const TI* __restrict__ w, const float* __restrict__ inv_rms,
                                                          TO* __restrict__ out, int64_t M, int64_t N) {
  constexpr int VEC = 16 / sizeof(TI);
  constexpr int UNROLL = 2;
  __shared__ float smem[BLOCK / 64];
  const int64_t row = blockIdx.x;
  const TI* ar = a + row * N;
  const TI* gr = g + row * N;
  TO* orow = out + row * N;
  const int64_t packs = N / VEC, tail0 = packs * VEC;
  const int t = threadIdx.x;
  const float inv = MODE == BWD_RMS ? inv_rms[row] : 1.0f;
  const bool has_w = MODE == BWD_RMS && w != nullptr;
  float s = 0.f;
  for (int64_t p0 = t; p0 < packs; p0 += (int64_t)BLOCK * UNROLL) {
    Pack<TI, VEC> pa[UNROLL], pg[UNROLL], pw[UNROLL];
#pragma unroll
    for (int u = 0; u < UNROLL; ++u) {
      const int64_t p = p0 + (int64_t)u * BLOCK;
      if (p < packs) {
        pa[u] = ld_pack_u<TI, VEC>(ar + p * VEC);
        pg[u] = ld_pack_u<TI, VEC>(gr + p * VEC);
        if (has_w) pw[u] = ld_pack_u<TI, VEC>(w + p * VEC);
      }
    }
#pragma unroll
    for (int u = 0; u < UNROLL; ++u) {
      if (p0 + (int64_t)u * BLOCK < packs) {
#pragma unroll
        for (int e = 0; e < VEC; ++e) {
          const float x = (float)pa[u].v[e], d = (float)pg[u].v[e];
          if constexpr (MODE == BWD_SOFTMAX) s += x * d;
          else if constexpr (MODE == BWD_LOG_SOFTMAX) s += d;
          else s += x * inv * d * (has_w ? (float)pw[u].v[e] : 1.0f);
        }
      }
    }
  }
  if (t < N - tail0) {
    const int64_t c = tail0 + t;
    const float x = (float)ar[c], d = (float)gr[c];
    if constexpr (MODE == BWD_SOFTMAX) s += x * d;
    else if constexpr (MODE == BWD_LOG_SOFTMAX) s += d;
    else s += x * inv * d * (has_w ? (float)w[c] : 1.0f);
  }
  s = row_sum<BLOCK>(s, smem, 0, t);
  const float mean = s / (float)N;
  auto result = [&](float x, float d, float wv) -> TO {
    if constexpr (MODE == BWD_SOFTMAX) return (TO)(x * (d - s));
    else if constexpr (MODE == BWD_LOG_SOFTMAX) return (TO)(d - exp_like_forward<TI>(x) * s);
    else return (TO)((d * wv - x * inv * mean) * inv);
  };
  for (int64_t p0 = t; p0 < packs; p0 += (int64_t)BLOCK * UNROLL) {
    Pack<TI, VEC> pa[UNROLL], pg[UNROLL], pw[UNROLL];
#pragma unroll
    for (int u = 0; u < UNROLL; ++u) {
      const int64_t p = p0 + (int64_t)u * BLOCK;
      if (p < packs) {
        pa[u] = ld_pack_u<TI, VEC>(ar + p * VEC);
        pg[u] = ld_pack_u<TI, VEC>(gr + p * VEC);
        if (has_w) pw[u] = ld_pack_u<TI, VEC>(w + p * VEC);
      }
    }
#pragma unroll
    for (int u = 0; u < UNROLL; ++u) {
      const int64_t p = p0 + (int64_t)u * BLOCK;
      if (p < packs) {
        Pack<TO, VEC> po;
#pragma unroll
        for (int e = 0; e < VEC; ++e)
          po.v[e] = result((float)pa[u].v[e], (float)pg[u].v[e], has_w ? (float)pw[u].v[e] : 1.0f);
        st_pack_u<TO, VEC>(orow + p * VEC, po);
      }
    }
  }
  if (t < N - tail0) {
    const int64_t c = tail0 + t;
    orow[c] = result((float)ar[c], (float)gr[c], has_w ? (float)w[c] : 1.0f);
  }
}

// Short rows whose start is only element-aligned (N <= 512): one wave per row, element j * 64 + lane in
// register j, no LDS and no barrier.  Softmax and log_softmax only.
template <typename TI, typename TO, int MODE, int ITERS>
__global__ __launch_bounds__(256) void bwd_short_kernel(const TI* __restrict__ a, const TI* __restrict__ g,
                                                       TO* __restrict__ out, int64_t M, int N) {
  const int lane = threadIdx.x & 63;
  const int64_t row = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
  if (row >= M) return;  // the whole wave leaves
  const TI* ar = a + row * (int64_t)N;
  const TI* gr = g + row * (int64_t)N;
  TO* orow = out + row * (int64_t)N;
  // unconditional loads (a column past the end reads column 0 and is discarded): with a branch around each the
  // compiler waits for one before it requests the next, a trip to memory per element
  // (variant FG_V_SHORT_UPFRONT, variants.h; off: every element is loaded where it is used, under its bounds check)
  constexpr bool UPFRONT = FG_V_SHORT_UPFRONT != 0;
  TI araw[ITERS], graw[ITERS];
  if constexpr (UPFRONT) {
#pragma unroll
    for (int j = 0; j < ITERS; ++j) {
      const int c = j * 64 + lane;
      const int cc = c < N ? c : 0;
      araw[j] = ar[cc];
      graw[j] = gr[cc];
    }
  }
  float x[ITERS], d[ITERS];
  float s = 0.f;
#pragma unroll
  for (int j = 0; j < ITERS; ++j) {
    const int c = j * 64 + lane;
    if constexpr (UPFRONT) {
      x[j] = c < N ? (float)araw[j] : 0.f;
      d[j] = c < N ? (float)graw[j] : 0.f;
    } else {
      x[j] = c < N ? (float)ar[c] : 0.f;
      d[j] = c < N ? (float)gr[c] : 0.f;
    }
    s += MODE == BWD_SOFTMAX ? x[j] * d[j] : d[j];
  }
  s = wave_sum(s);
#pragma unroll
  for (int j = 0; j < ITERS; ++j) {
    const int c = j * 64 + lane;
    if (c < N) orow[c] = MODE == BWD_SOFTMAX ? (TO)(x[j] * (d[j] - s)) : (TO)(d[j] - exp_like_forward<TI>(x[j]) * s);
  }
}

// Middle axis: tensors viewed as [M, N, K], K contiguous.  Thread = one (m, k) column.
template <typename TI, typename TO, int MODE>
__global__ __launch_bounds__(256) void bwd_non_inner_kernel(const TI* __restrict__ y, const TI* __restrict__ g,
                                                           TO* __restrict__ out, int64_t M, int64_t N, int64_t K) {
  const int64_t k = (int64_t)blockIdx.x * 256 + threadIdx.x;
  const int64_t mrow = blockIdx.y;
  if (k >= K) return;
  const int64_t base = mrow * N * K + k;
  float s = 0.f;
  for (int64_t n = 0; n < N; ++n) {
    const float x = (float)y[base + n * K], d = (float)g[base + n * K];
    s += MODE == BWD_SOFTMAX ? x * d : d;
  }
  for (int64_t n = 0; n < N; ++n) {
    const float x = (float)y[base + n * K], d = (float)g[base + n * K];
    out[base + n * K] = MODE == BWD_SOFTMAX ? (TO)(x * (d - s)) : (TO)(d - exp_like_forward<TI>(x) * s);
  }
}

// Partial weight gradient of rms_norm: block (rb, cb) sums x * dy * inv_rms over rows
// [rb * rows_per_block, ...) for its 256 columns and writes row rb of `partial` [row_blocks, N].
template <typename T>
__global__ __launch_bounds__(256) void rms_dw_partial_kernel(const T* __restrict__ x, const T* __restrict__ dy,
                                                            const float* __restrict__ inv_rms,
                                                            float* __restrict__ partial, int64_t M, int64_t N,
                                                            int rows_per_block) {
  const int64_t c = (int64_t)blockIdx.y * 256 + threadIdx.x;
  if (c >= N) return;
  const int64_t r0 = (int64_t)blockIdx.x * rows_per_block;
  int64_t r1 = r0 + rows_per_block;
  if (r1 > M) r1 = M;
  float s = 0.f;
  for (int64_t r = r0; r < r1; ++r) s += (float)x[r * N + c] * (float)dy[r * N + c] * inv_rms[r];
  partial[(int64_t)blockIdx.x * N + c] = s;
}

// Column sums of the partial rows: out[c] = sum over r of partial[r, c], rounded once to T.  A workgroup owns 32
// columns (one 128-byte line per row); its 32 row lanes each add every 32nd row, then lane 0 adds the 32 sums in
// order, so the result does not depend on timing.
template <typename T>
__global__ __launch_bounds__(1024) void column_sum_kernel(const float* __restrict__ partial, T* __restrict__ out,
                                                          int64_t rows, int64_t N) {
  __shared__ float part[32][33];
  const int tx = threadIdx.x & 31, ty = threadIdx.x >> 5;
  const int64_t c = (int64_t)blockIdx.x * 32 + tx;
  float s = 0.f;
  if (c < N)
    for (int64_t r = ty; r < rows; r += 32) s += partial[r * N + c];
  part[ty][tx] = s;
  __syncthreads();
  if (ty == 0 && c < N) {
    float t = 0.f;
#pragma unroll
    for (int i = 0; i < 32; ++i) t += part[i][tx];
    out[c] = (T)t;
  }
}

template <typename TI, typename TO, int VEC, int ITERS, int TPR, int MODE>
void launch_rows(const TI* a, const TI* g, TO* out, int64_t M, int N, hipStream_t st) {
  constexpr int BLOCK = TPR < 256 ? 256 : TPR;
  constexpr int RPB = BLOCK / TPR;
  hipLaunchKernelGGL((bwd_rows_kernel<TI, TO, VEC, ITERS, TPR, MODE>), dim3((unsigned)fg_cdiv(M, RPB)), dim3(BLOCK), 0,
                     st, a, g, out, M, N);
}

// Inner-axis dispatch of the softmax modes.  The caller has checked sizes and pointers.
template <typename TI, typename TO, int MODE>
int bwd_rows_dispatch(const TI* a, const TI* g, TO* out, int64_t M, int64_t N, hipStream_t st, const char* what) {
  FG_REQUIRE(M < ((int64_t)1 << 31), FG_ERR_UNSUPPORTED, "%s: M=%lld exceeds the grid limit", what, (long long)M);
  constexpr int VEC = 16 / sizeof(TI);
  const bool vec_ok = (N % VEC == 0) && fg_aligned(a, 16) && fg_aligned(g, 16) && fg_aligned(out, sizeof(TO) * VEC);
  const int64_t packs = vec_ok ? N / VEC : 0;
#define FG_ROWS(ITERS, TPR) launch_rows<TI, TO, VEC, ITERS, TPR, MODE>(a, g, out, M, (int)N, st)
  // two input streams: one pack per thread from each, as in the fused add + norm forward
  if (!vec_ok && N <= 512) {  // from there on the two-sweep kernel with 256 threads measures faster
#define FG_SHORT(ITERS)                                                                                                \
  hipLaunchKernelGGL((bwd_short_kernel<TI, TO, MODE, ITERS>), dim3((unsigned)fg_cdiv(M, 4)), dim3(256), 0, st, a, g, out, \
                     M, (int)N)
    if (N <= 64) FG_SHORT(1);
    else if (N <= 128) FG_SHORT(2);
    else if (N <= 256) FG_SHORT(4);
    else FG_SHORT(8);
#undef FG_SHORT
  } else if (!vec_ok || packs > 4096) {
    if (N >= 2048)
      hipLaunchKernelGGL((bwd_looped_kernel<TI, TO, MODE, 1024>), dim3((unsigned)M), dim3(1024), 0, st, a, g,
                         (const TI*)nullptr, (const float*)nullptr, out, M, N);
    else
      hipLaunchKernelGGL((bwd_looped_kernel<TI, TO, MODE, 256>), dim3((unsigned)M), dim3(256), 0, st, a, g,
                         (const TI*)nullptr, (const float*)nullptr, out, M, N);
  } else if (packs > 2048) {
    FG_ROWS(4, 1024);  // vocabulary-sized rows (32000 16-bit elements)
  } else if (packs <= 64) {
    FG_ROWS(1, 64);
  } else if (packs <= 128) {
    FG_ROWS(1, 128);
  } else if (packs <= 256) {
    FG_ROWS(1, 256);
  } else if (packs <= 512) {
    FG_ROWS(1, 512);
  } else if (packs <= 1024) {
    FG_ROWS(1, 1024);
  } else {
    FG_ROWS(2, 1024);
  }
#undef FG_ROWS
  return fg_check_launch(what);
}

// Threads per row of the rms kernel for a row of `packs` 16-byte packs (at most 2048).
int rms_bwd_tpr(int64_t packs) { return packs <= 64 ? 64 : packs <= 128 ? 128 : packs <= 256 ? 256 : packs <= 512 ? 512 : 1024; }

template <typename T, int VEC, int ITERS, int TPR>
void launch_rms_rows(const T* x, const T* dy, const T* w, const float* inv_rms, T* dx, float* dw_partial,
                     int64_t partial_rows, int64_t M, int N, int rows_per_group, hipStream_t st) {
  constexpr int BLOCK = TPR < 256 ? 256 : TPR;
  constexpr int RPB = BLOCK / TPR;
  // every partial row gets written (groups past the last row write zeros); without partial rows one row per group
  const int64_t groups = dw_partial != nullptr ? partial_rows : fg_cdiv(M, rows_per_group);
  if (ITERS == 1 && rows_per_group > 1)
    hipLaunchKernelGGL((rms_bwd_rows_kernel<T, VEC, ITERS, TPR, ITERS == 1>), dim3((unsigned)fg_cdiv(groups, RPB)),
                       dim3(BLOCK), 0, st, x, dy, w, inv_rms, dx, dw_partial, partial_rows, M, N, rows_per_group);
  else
    hipLaunchKernelGGL((rms_bwd_rows_kernel<T, VEC, ITERS, TPR, false>), dim3((unsigned)fg_cdiv(groups, RPB)),
                       dim3(BLOCK), 0, st, x, dy, w, inv_rms, dx, dw_partial, partial_rows, M, N, rows_per_group);
}

// dw_partial (may be null) has partial_rows rows of N floats; every one of them is written.
template <typename T>
int rms_bwd_dispatch(const T* x, const T* dy, const T* w, const float* inv_rms, T* dx, float* dw_partial,
                     int64_t partial_rows, int64_t M, int64_t N, hipStream_t st) {
  constexpr int VEC = 16 / sizeof(T);
  const bool vec_ok = (N % VEC == 0) && fg_aligned(x, 16) && fg_aligned(dy, 16) && fg_aligned(dx, 16) &&
                      (w == nullptr || fg_aligned(w, 16)) && (dw_partial == nullptr || fg_aligned(dw_partial, 32));
  const int64_t packs = vec_ok ? N / VEC : 0;
  // rows summed into one partial row: with partial_rows groups of that many rows all M rows are covered
  const int64_t rows_per_group = dw_partial != nullptr ? fg_cdiv(M, partial_rows) : 1;
  if (!vec_ok || packs > 2048) {
    if (N >= 2048)
      hipLaunchKernelGGL((bwd_looped_kernel<T, T, BWD_RMS, 1024>), dim3((unsigned)M), dim3(1024), 0, st, x, dy, w, inv_rms,
                         dx, M, N);
    else
      hipLaunchKernelGGL((bwd_looped_kernel<T, T, BWD_RMS, 256>), dim3((unsigned)M), dim3(256), 0, st, x, dy, w, inv_rms,
                         dx, M, N);
    if (dw_partial != nullptr)
      hipLaunchKernelGGL((rms_dw_partial_kernel<T>), dim3((unsigned)partial_rows, (unsigned)fg_cdiv(N, 256)), dim3(256),
                         0, st, x, dy, inv_rms, dw_partial, M, N, (int)rows_per_group);
    return fg_check_launch("rms_norm_backward");
  }
#define FG_ROWS(ITERS, TPR)   launch_rms_rows<T, VEC, ITERS, TPR>(x, dy, w, inv_rms, dx, dw_partial, partial_rows, M, (int)N, (int)rows_per_group, st)
  switch (rms_bwd_tpr(packs)) {
    case 64: FG_ROWS(1, 64); break;
    case 128: FG_ROWS(1, 128); break;
    case 256: FG_ROWS(1, 256); break;
    case 512: FG_ROWS(1, 512); break;
    default:
      if (packs <= 1024) FG_ROWS(1, 1024);
      else FG_ROWS(2, 1024);
  }
#undef FG_ROWS
  return fg_check_launch("rms_norm_backward");
}

template <typename TI, typename TO, int MODE>
int softmax_bwd_dispatch(const TI* y, const TI* g, TO* out, int64_t M, int64_t N, int64_t K, hipStream_t st,
                         const char* what) {
  if (K > 1) {
    FG_REQUIRE(M < 65536, FG_ERR_UNSUPPORTED, "%s: leading extent %lld too large for the middle-axis kernel", what,
               (long long)M);
    hipLaunchKernelGGL((bwd_non_inner_kernel<TI, TO, MODE>), dim3((unsigned)fg_cdiv(K, 256), (unsigned)M), dim3(256), 0,
                       st, y, g, out, M, N, K);
    return fg_check_launch(what);
  }
  return bwd_rows_dispatch<TI, TO, MODE>(y, g, out, M, N, st, what);
}

template <int MODE>
int softmax_bwd_entry(const void* y, const void* g, void* out, int64_t M, int64_t N, int64_t K, int dtype,
                      int out_dtype, void* stream) {
  const char* what = MODE == BWD_SOFTMAX ? "softmax_backward" : "log_softmax_backward";
  FG_REQUIRE(M >= 0 && N >= 0 && K >= 0, FG_ERR_INVALID, "%s: negative size", what);
  if (M == 0 || N == 0 || K == 0) return FG_OK;
  FG_REQUIRE(y && g && out, FG_ERR_INVALID, "%s: null pointer", what);
  FG_REQUIRE(N < ((int64_t)1 << 31), FG_ERR_UNSUPPORTED, "%s: N=%lld too large", what, (long long)N);
  FG_REQUIRE(out_dtype == dtype || dtype == FG_F32, FG_ERR_INVALID,
             "%s: gradient dtype %d must equal the output dtype %d unless that is fp32", what, out_dtype, dtype);
  hipStream_t st = (hipStream_t)stream;
#define FG_CASE(DI, DO, TI, TO) \
  if (dtype == DI && out_dtype == DO) \
    return softmax_bwd_dispatch<TI, TO, MODE>((const TI*)y, (const TI*)g, (TO*)out, M, N, K, st, what)
  FG_CASE(FG_F16, FG_F16, f16_t, f16_t);
  FG_CASE(FG_BF16, FG_BF16, bf16_t, bf16_t);
  FG_CASE(FG_F32, FG_F32, float, float);
  FG_CASE(FG_F32, FG_F16, float, f16_t);
  FG_CASE(FG_F32, FG_BF16, float, bf16_t);
#undef FG_CASE
  fg_set_error("%s: unsupported dtype pair (%d, %d)", what, dtype, out_dtype);
  return FG_ERR_INVALID;
}

}  // namespace

extern "C" int fg_softmax_backward(const void* out, const void* grad_out, void* grad_in, int64_t M, int64_t N,
                                   int64_t K, int dtype, int grad_in_dtype, void* stream) {
  return softmax_bwd_entry<BWD_SOFTMAX>(out, grad_out, grad_in, M, N, K, dtype, grad_in_dtype, stream);
}

extern "C" int fg_log_softmax_backward(const void* out, const void* grad_out, void* grad_in, int64_t M, int64_t N,
                                       int64_t K, int dtype, int grad_in_dtype, void* stream) {
  return softmax_bwd_entry<BWD_LOG_SOFTMAX>(out, grad_out, grad_in, M, N, K, dtype, grad_in_dtype, stream);
}

extern "C" int64_t fg_rms_norm_backward_partial_rows(int64_t M, int64_t N, int dtype, int device) {
  if (M <= 0 || N <= 0) return 0;
  const int64_t vec = dtype == FG_F32 ? 4 : 8;
  if (N % vec != 0 || N / vec > 2048) return fg_cdiv(M, 64);
  const int tpr = rms_bwd_tpr(N / vec);
  const int block = tpr < 256 ? 256 : tpr;
  // enough groups to give every CU its 2048 threads once, 8 to 64 rows each
  const int64_t target = (int64_t)fgk::num_cus(device) * (2048 / block) * (block / tpr);
  int64_t rows_per_group = fg_cdiv(M, target);
  rows_per_group = rows_per_group < 8 ? 8 : rows_per_group > 64 ? 64 : rows_per_group;
  return fg_cdiv(M, rows_per_group);
}

extern "C" int fg_rms_norm_backward_dw(const float* dw_partial, int64_t partial_rows, int64_t N, void* dw, int dtype,
                                       void* stream) {
  FG_REQUIRE(partial_rows >= 0 && N >= 0, FG_ERR_INVALID, "rms_norm_backward_dw: negative size");
  if (N == 0) return FG_OK;
  FG_REQUIRE(dw && (dw_partial || partial_rows == 0), FG_ERR_INVALID, "rms_norm_backward_dw: null pointer");
  FG_REQUIRE(fg_cdiv(N, 32) < ((int64_t)1 << 31), FG_ERR_UNSUPPORTED, "rms_norm_backward_dw: N=%lld too large",
             (long long)N);
  hipStream_t st = (hipStream_t)stream;
  const dim3 grid((unsigned)fg_cdiv(N, 32));
  switch (dtype) {
    case FG_F16:
      hipLaunchKernelGGL(column_sum_kernel<f16_t>, grid, dim3(1024), 0, st, dw_partial, (f16_t*)dw, partial_rows, N);
      break;
    case FG_BF16:
      hipLaunchKernelGGL(column_sum_kernel<bf16_t>, grid, dim3(1024), 0, st, dw_partial, (bf16_t*)dw, partial_rows, N);
      break;
    case FG_F32:
      hipLaunchKernelGGL(column_sum_kernel<float>, grid, dim3(1024), 0, st, dw_partial, (float*)dw, partial_rows, N);
      break;
    default:
      fg_set_error("rms_norm_backward_dw: bad dtype %d", dtype);
      return FG_ERR_INVALID;
  }
  return fg_check_launch("rms_norm_backward_dw");
}

extern "C" int fg_rms_norm_backward(const void* x, const void* dy, const float* inv_rms, const void* w, void* dx,
                                    float* dw_partial, int64_t partial_rows, int64_t M, int64_t N, int dtype,
                                    void* stream) {
  FG_REQUIRE(M >= 0 && N >= 0, FG_ERR_INVALID, "rms_norm_backward: negative size");
  if (M == 0 || N == 0) return FG_OK;
  FG_REQUIRE(x && dy && inv_rms && dx, FG_ERR_INVALID, "rms_norm_backward: null pointer");
  FG_REQUIRE(M < ((int64_t)1 << 31) && N < ((int64_t)1 << 31), FG_ERR_UNSUPPORTED,
             "rms_norm_backward: extent exceeds 2^31");
  FG_REQUIRE(dw_partial == nullptr || (partial_rows >= 1 && partial_rows <= M), FG_ERR_INVALID,
             "rms_norm_backward: partial_rows=%lld must lie in [1, M]", (long long)partial_rows);
  FG_REQUIRE(fg_cdiv(N, 256) < 65536, FG_ERR_UNSUPPORTED, "rms_norm_backward: N=%lld too large", (long long)N);
  hipStream_t st = (hipStream_t)stream;
  switch (dtype) {
    case FG_F16:
      return rms_bwd_dispatch<f16_t>((const f16_t*)x, (const f16_t*)dy, (const f16_t*)w, inv_rms, (f16_t*)dx, dw_partial,
                                     partial_rows, M, N, st);
    case FG_BF16:
      return rms_bwd_dispatch<bf16_t>((const bf16_t*)x, (const bf16_t*)dy, (const bf16_t*)w, inv_rms, (bf16_t*)dx,
                                      dw_partial, partial_rows, M, N, st);
    case FG_F32:
      return rms_bwd_dispatch<float>((const float*)x, (const float*)dy, (const float*)w, inv_rms, (float*)dx, dw_partial,
                                     partial_rows, M, N, st);
  }
  fg_set_error("rms_norm_backward: unsupported dtype %d", dtype);
  return FG_ERR_INVALID;
}
