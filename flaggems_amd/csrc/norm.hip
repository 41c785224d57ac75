// rms_norm and fused_add_rms_norm for gfx950: single pass over HBM, the row lives in registers.
//
// Layout: x [M, N] with unit column stride and arbitrary row stride.  TPR threads share one row
// (TPR = 64 .. 1024, a power of two); each thread holds ITERS packs of VEC elements, pack j of
// thread t covering columns (j*TPR + t)*VEC .. +VEC, so every load instruction of a wave reads
// 64*VEC*sizeof(T) contiguous bytes (1 KiB at 16 B per lane).  Blocks are 256 threads, so
// 256/TPR rows share a block when TPR < 256.  Rows too long for the register variant
// (N > 1024*VEC*8) and rows that defeat vector access (N or strides not a multiple of VEC,
// unaligned base) go through a two-pass kernel that re-reads the row from L2 (16-byte accesses
// declared element-aligned, one workgroup per row), or, up to 512 elements, one wave per row.
#include "fg_common.h"

namespace {

template <int TPR>
__device__ __forceinline__ float row_sum(float v, float* smem, int row_in_block, int t) {
  v = wave_sum(v);
  if constexpr (TPR > 64) {
    constexpr int WPR = TPR / 64;  // waves per row
    const int wave_in_row = t >> 6;
    __syncthreads();
    if ((t & 63) == 0) smem[row_in_block * WPR + wave_in_row] = v;
    __syncthreads();
    float s = 0.f;
#pragma unroll
    for (int i = 0; i < WPR; ++i) s += smem[row_in_block * WPR + i];
    v = s;
  }
  return v;
}

// FUSED = false: y = x * rrms * w, optional inv_rms.   FUSED = true: r = x + r (stored), x = r*rrms*w.
template <typename T, int VEC, int ITERS, int TPR, bool FUSED>
__global__ __launch_bounds__(TPR < 256 ? 256 : TPR) void rms_rows_kernel(
    const T* x, T* res, const T* __restrict__ w, T* y,
    float* __restrict__ inv_rms, int64_t M, int N, int64_t xs, int64_t rs, int64_t ys, float eps) {
  constexpr int BLOCK = TPR < 256 ? 256 : TPR;
  constexpr int RPB = BLOCK / TPR;
  __shared__ float smem[BLOCK / 64];
  const int tid = threadIdx.x;
  const int row_in_block = tid / TPR;
  const int t = tid % TPR;
  const int64_t row = (int64_t)blockIdx.x * RPB + row_in_block;
  const bool row_ok = row < M;
  const T* xr = x + row * xs;

  // Variant FG_V_ROWS_UPFRONT (variants.h; off: every pack is loaded where it is used, under its bounds check).
  // What the tail of the kernel needs is requested before the row is read.  Fetched where it is used, the weight
  // pack costs every workgroup a round trip to L2 behind the reduction, when it has no other request in flight, and
  // each kernel argument first touched there a round trip to the scalar cache.  Up to two packs a thread (4 registers
  // each for 16-bit types); longer rows keep the late fetch.
  constexpr bool UPFRONT = FG_V_ROWS_UPFRONT != 0;
  constexpr bool EARLY_W = UPFRONT && ITERS <= 2 && sizeof(T) * VEC == 16;
  u32x4 pw_early[EARLY_W ? ITERS : 1];
  if constexpr (EARLY_W) {
    const T* wp = w != nullptr ? w : x;  // no weight: any readable address, the value is not used
#pragma unroll
    for (int j = 0; j < ITERS; ++j) {
      const int col = (j * TPR + t) * VEC;
      pw_early[j] = *reinterpret_cast<const u32x4*>(wp + (col < N ? col : 0));  // columns past the end are never stored
    }
  }
  if constexpr (UPFRONT) asm volatile("" : : "s"(eps), "s"(y), "s"(ys), "s"(inv_rms));

  // All packs of the thread are requested before the first is used.  The loads are unconditional (a pack past the
  // end of the row or of the matrix is read from the start of x and discarded): with a branch around each load the
  // compiler finishes pack j, wait included, before it requests pack j + 1, one trip to memory per pack.
  Pack<T, VEC> px[ITERS], pr[FUSED ? ITERS : 1];
  if constexpr (UPFRONT) {
#pragma unroll
    for (int j = 0; j < ITERS; ++j) {
      const int col = (j * TPR + t) * VEC;
      const bool ok = row_ok && col < N;
      px[j] = ld_pack_nt<T, VEC>(ok ? xr + col : x);
      if constexpr (FUSED) pr[j] = ld_pack_nt<T, VEC>(ok ? res + row * rs + col : x);
    }
  }
  if constexpr (UPFRONT && FUSED && ITERS == 1 && sizeof(T) * VEC == 16) {
    // with one pack of each, the scheduler otherwise starts converting x before it has requested the residual;
    // the empty asm needs both registers, so both requests go out first
    asm volatile("" : "+v"(*reinterpret_cast<u32x4*>(&px[0])), "+v"(*reinterpret_cast<u32x4*>(&pr[0])));
  }
  float v[ITERS][VEC];
  float ss = 0.f;
#pragma unroll
  for (int j = 0; j < ITERS; ++j) {
    const int col = (j * TPR + t) * VEC;
    if (row_ok && col < N) {
      if constexpr (!UPFRONT) px[j] = ld_pack_nt<T, VEC>(xr + col);
      if constexpr (FUSED) {
        if constexpr (!UPFRONT) pr[j] = ld_pack_nt<T, VEC>(res + row * rs + col);
        Pack<T, VEC> po;
#pragma unroll
        for (int e = 0; e < VEC; ++e) {
          v[j][e] = (float)px[j].v[e] + (float)pr[j].v[e];
          po.v[e] = (T)v[j][e];
        }
        st_pack_nt<T, VEC>(res + row * rs + col, po);
      } else {
#pragma unroll
        for (int e = 0; e < VEC; ++e) v[j][e] = (float)px[j].v[e];
      }
#pragma unroll
      for (int e = 0; e < VEC; ++e) ss += v[j][e] * v[j][e];
    } else {
#pragma unroll
      for (int e = 0; e < VEC; ++e) v[j][e] = 0.f;
    }
  }
  ss = row_sum<TPR>(ss, smem, row_in_block, t);
  const float rrms = 1.0f / sqrtf(ss / (float)N + eps);
  if (!row_ok) return;
  if constexpr (!FUSED) {
    if (inv_rms != nullptr && t == 0) inv_rms[row] = rrms;
  }
  T* yr = y + row * ys;
#pragma unroll
  for (int j = 0; j < ITERS; ++j) {
    const int col = (j * TPR + t) * VEC;
    if (col < N) {
      Pack<T, VEC> po;
      if (w != nullptr) {
        Pack<T, VEC> pw;
        if constexpr (EARLY_W) {
          // (the registers pass through an empty asm so that the conversion to fp32, and with it the wait for the
          // load, stays down here)
          u32x4 raw = pw_early[j];
          asm volatile("" : "+v"(raw));
          pw = *reinterpret_cast<Pack<T, VEC>*>(&raw);
        } else {
          pw = ld_pack<T, VEC>(w + col);
        }
#pragma unroll
        for (int e = 0; e < VEC; ++e) po.v[e] = (T)(v[j][e] * rrms * (float)pw.v[e]);
      } else {
#pragma unroll
        for (int e = 0; e < VEC; ++e) po.v[e] = (T)(v[j][e] * rrms);
      }
      st_pack_nt<T, VEC>(yr + col, po);
    }
  }
}

#if FG_V_RMS_TWO_ROWS
// Variant FG_V_RMS_TWO_ROWS (variants.h): rows of one 16-byte pack per thread on 256 to 1024 threads, two rows per
// workgroup.  A matrix of a few thousand rows is a handful of rounds of workgroups on this part (a CU holds 2048
// threads: [4096, 4096] bf16 at 512 threads a row is four rounds), and every round pays its start and its drain.  Two
// rows per workgroup halve the rounds; both rows' packs and the weight pack are requested before anything is
// used, so a thread has four requests in flight instead of two, and the two row sums share one LDS exchange (two
// barriers per workgroup instead of two per row).  Arithmetic and rounding are those of rms_rows_kernel.
template <typename T, int VEC, int TPR, bool FUSED>
__global__ __launch_bounds__(TPR) void rms_rows2_kernel(const T* x, T* res, const T* __restrict__ w, T* y,
                                                       float* __restrict__ inv_rms, int64_t M, int N, int64_t xs,
                                                       int64_t rs, int64_t ys, float eps) {
  static_assert(TPR >= 256 && TPR % 64 == 0 && sizeof(T) * VEC == 16, "one 16-byte pack per thread, whole waves");
  constexpr int WPR = TPR / 64;
  __shared__ float smem[2][WPR];
  const int t = threadIdx.x;
  const int64_t row0 = (int64_t)blockIdx.x * 2;
  const int col = t * VEC;
  const bool col_ok = col < N;
  bool ok[2];
  Pack<T, VEC> px[2], pr[FUSED ? 2 : 1];
  const T* wp = w != nullptr ? w : x;  // no weight: any readable address, the value is not used
  const u32x4 wraw = *reinterpret_cast<const u32x4*>(wp + (col_ok ? col : 0));
  asm volatile("" : : "s"(eps), "s"(y), "s"(ys), "s"(inv_rms));  // the tail's arguments are fetched with the others
#pragma unroll
  for (int r = 0; r < 2; ++r) {
    ok[r] = row0 + r < M && col_ok;
    // unconditional loads: a pack past the end of the row or of the matrix is read from the start of x and discarded
    px[r] = ld_pack_nt<T, VEC>(ok[r] ? x + (row0 + r) * xs + col : x);
    if constexpr (FUSED) pr[r] = ld_pack_nt<T, VEC>(ok[r] ? res + (row0 + r) * rs + col : x);
  }
  float v[2][VEC], ss[2];
#pragma unroll
  for (int r = 0; r < 2; ++r) {
    ss[r] = 0.f;
    if constexpr (FUSED) {
      Pack<T, VEC> po;
#pragma unroll
      for (int e = 0; e < VEC; ++e) {
        v[r][e] = ok[r] ? (float)px[r].v[e] + (float)pr[r].v[e] : 0.f;
        po.v[e] = (T)v[r][e];
      }
      if (ok[r]) st_pack_nt<T, VEC>(res + (row0 + r) * rs + col, po);
    } else {
#pragma unroll
      for (int e = 0; e < VEC; ++e) v[r][e] = ok[r] ? (float)px[r].v[e] : 0.f;
    }
#pragma unroll
    for (int e = 0; e < VEC; ++e) ss[r] += v[r][e] * v[r][e];
    ss[r] = wave_sum(ss[r]);
  }
  // (a row's sum is added up over its waves in wave order, as row_sum does)
  if ((t & 63) == 0) {
    smem[0][t >> 6] = ss[0];
    smem[1][t >> 6] = ss[1];
  }
  __syncthreads();
  Pack<T, VEC> pw = *reinterpret_cast<const Pack<T, VEC>*>(&wraw);
#pragma unroll
  for (int r = 0; r < 2; ++r) {
    float s = 0.f;
#pragma unroll
    for (int i = 0; i < WPR; ++i) s += smem[r][i];
    const float rrms = 1.0f / sqrtf(s / (float)N + eps);
    if (row0 + r >= M) continue;
    if constexpr (!FUSED) {
      if (inv_rms != nullptr && t == 0) inv_rms[row0 + r] = rrms;
    }
    if (!col_ok) continue;
    Pack<T, VEC> po;
    if (w != nullptr) {
#pragma unroll
      for (int e = 0; e < VEC; ++e) po.v[e] = (T)(v[r][e] * rrms * (float)pw.v[e]);
    } else {
#pragma unroll
      for (int e = 0; e < VEC; ++e) po.v[e] = (T)(v[r][e] * rrms);
    }
    st_pack_nt<T, VEC>(y + (row0 + r) * ys + col, po);
  }
}
#endif

// Any N, any alignment: one 256-thread block per row, element-wise coalesced access, two passes.
// Short rows that defeat 16-byte access (N <= 512): one wave per row, element j * 64 + lane in register j.
template <typename T, bool FUSED, int ITERS>
__global__ __launch_bounds__(256) void rms_short_kernel(const T* x, T* res, const T* __restrict__ w, T* y,
                                                       float* __restrict__ inv_rms, int64_t M, int N, int64_t xs,
                                                       int64_t rs, int64_t ys, float eps) {
  const int lane = threadIdx.x & 63;
  const int64_t row = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
  if (row >= M) return;  // the whole wave leaves
  const T* xr = x + row * xs;
  T* rr = FUSED ? res + row * rs : nullptr;
  T* yr = y + row * ys;
  // Variant FG_V_SHORT_UPFRONT (variants.h; off: every element is loaded where it is used, under its bounds check):
  // unconditional loads, the weights included (a column past the end reads column 0 and is discarded): with a
  // branch around each the compiler waits for one before it requests the next, a trip to memory per element
  constexpr bool UPFRONT = FG_V_SHORT_UPFRONT != 0;
  T xraw[ITERS], rraw[FUSED ? ITERS : 1], wraw[ITERS];
  if constexpr (UPFRONT) {
    const T* wp = w != nullptr ? w : x;  // no weight: any readable address, the value is not used
    asm volatile("" : : "s"(eps), "s"(y), "s"(ys), "s"(inv_rms));  // the tail's arguments are fetched with the others
#pragma unroll
    for (int j = 0; j < ITERS; ++j) {
      const int c = j * 64 + lane;
      const int cc = c < N ? c : 0;
      xraw[j] = xr[cc];
      if constexpr (FUSED) rraw[j] = rr[cc];
      wraw[j] = wp[cc];
    }
  }
  float v[ITERS];
  float ss = 0.f;
#pragma unroll
  for (int j = 0; j < ITERS; ++j) {
    const int c = j * 64 + lane;
    if constexpr (UPFRONT) {
      v[j] = c < N ? (float)xraw[j] : 0.f;
      if constexpr (FUSED) {
        if (c < N) v[j] += (float)rraw[j];
      }
    } else {
      v[j] = c < N ? (float)xr[c] : 0.f;
      if constexpr (FUSED) {
        if (c < N) v[j] += (float)rr[c];
      }
    }
    ss += v[j] * v[j];
  }
  ss = wave_sum(ss);
  const float rrms = 1.0f / sqrtf(ss / (float)N + eps);
  if constexpr (!FUSED) {
    if (inv_rms != nullptr && lane == 0) inv_rms[row] = rrms;
  }
#pragma unroll
  for (int j = 0; j < ITERS; ++j) {
    const int c = j * 64 + lane;
    if (c < N) {
      if constexpr (FUSED) rr[c] = (T)v[j];
      if constexpr (UPFRONT) yr[c] = (T)(v[j] * rrms * (w != nullptr ? (float)wraw[j] : 1.0f));
      else yr[c] = (T)(v[j] * rrms * (w != nullptr ? (float)w[c] : 1.0f));
    }
  }
}

template <typename T, bool FUSED, int BLOCK>
__global__ __launch_bounds__(BLOCK) void rms_looped_kernel(const T* x, T* res,
                                                          const T* __restrict__ w, T* y,
                                                          float* __restrict__ inv_rms, int64_t M, int64_t N,
                                                          int64_t xs, int64_t rs, int64_t ys, float eps) {
  constexpr int VEC = 16 / sizeof(T);
  constexpr int UNROLL = FUSED ? 2 : 4;
  __shared__ float smem[BLOCK / 64];
  const int64_t row = blockIdx.x;
  const T* xr = x + row * xs;
  T* rr = FUSED ? res + row * rs : nullptr;
  T* yr = y + row * ys;
  const int64_t packs = N / VEC, tail0 = packs * VEC;
  const int t = threadIdx.x;
  // 16-byte accesses declared element-aligned; the N % VEC elements behind the last full pack go one per thread
  float ss = 0.f;
  for (int64_t p0 = t; p0 < packs; p0 += (int64_t)BLOCK * UNROLL) {
    Pack<T, VEC> px[UNROLL], pr[UNROLL];
#pragma unroll
    for (int u = 0; u < UNROLL; ++u) {
      const int64_t p = p0 + (int64_t)u * BLOCK;
      if (p < packs) {
        px[u] = ld_pack_u<T, VEC>(xr + p * VEC);
        if constexpr (FUSED) pr[u] = ld_pack_u<T, VEC>(rr + p * VEC);
      }
    }
#pragma unroll
    for (int u = 0; u < UNROLL; ++u) {
      if (p0 + (int64_t)u * BLOCK < packs) {
#pragma unroll
        for (int e = 0; e < VEC; ++e) {
          float v = (float)px[u].v[e];
          if constexpr (FUSED) v += (float)pr[u].v[e];
          ss += v * v;
        }
      }
    }
  }
  if (t < N - tail0) {
    float v = (float)xr[tail0 + t];
    if constexpr (FUSED) v += (float)rr[tail0 + t];
    ss += v * v;
  }
  ss = row_sum<BLOCK>(ss, smem, 0, t);
  const float rrms = 1.0f / sqrtf(ss / (float)N + eps);
  if constexpr (!FUSED) {
    if (inv_rms != nullptr && t == 0) inv_rms[row] = rrms;
  }
  // Second pass recomputes the fp32 sum from the still-unmodified inputs (each element is read
  // and then written by the same thread, so in-place operation is safe).
  for (int64_t p0 = t; p0 < packs; p0 += (int64_t)BLOCK * UNROLL) {
    Pack<T, VEC> px[UNROLL], pr[UNROLL], pw[UNROLL];
#pragma unroll
    for (int u = 0; u < UNROLL; ++u) {
      const int64_t p = p0 + (int64_t)u * BLOCK;
      if (p < packs) {
        px[u] = ld_pack_u<T, VEC>(xr + p * VEC);
        if constexpr (FUSED) pr[u] = ld_pack_u<T, VEC>(rr + p * VEC);
        if (w != nullptr) pw[u] = ld_pack_u<T, VEC>(w + p * VEC);
      }
    }
#pragma unroll
    for (int u = 0; u < UNROLL; ++u) {
      const int64_t p = p0 + (int64_t)u * BLOCK;
      if (p < packs) {
        Pack<T, VEC> po, ps;
#pragma unroll
        for (int e = 0; e < VEC; ++e) {
          float v = (float)px[u].v[e];
          if constexpr (FUSED) {
            v += (float)pr[u].v[e];
            ps.v[e] = (T)v;
          }
          po.v[e] = (T)(v * rrms * (w != nullptr ? (float)pw[u].v[e] : 1.0f));
        }
        if constexpr (FUSED) st_pack_u<T, VEC>(rr + p * VEC, ps);
        st_pack_u<T, VEC>(yr + p * VEC, po);
      }
    }
  }
  if (t < N - tail0) {
    const int64_t c = tail0 + t;
    float v = (float)xr[c];
    if constexpr (FUSED) {
      v += (float)rr[c];
      rr[c] = (T)v;
    }
    yr[c] = (T)(v * rrms * (w != nullptr ? (float)w[c] : 1.0f));
  }
}

template <typename T, int VEC, int ITERS, int TPR, bool FUSED>
void launch_rows(const T* x, T* res, const T* w, T* y, float* inv_rms, int64_t M, int N, int64_t xs, int64_t rs,
                 int64_t ys, float eps, hipStream_t st) {
#if FG_V_RMS_TWO_ROWS
  if constexpr (ITERS == 1 && TPR >= 256) {
    // matrices of up to a few rounds of workgroups: beyond that the rounds overlap and one row per workgroup is as good
    if (M >= 2 && M <= 32768) {
      hipLaunchKernelGGL((rms_rows2_kernel<T, VEC, TPR, FUSED>), dim3((unsigned)fg_cdiv(M, 2)), dim3(TPR), 0, st, x, res,
                         w, y, inv_rms, M, N, xs, rs, ys, eps);
      return;
    }
  }
#endif
  constexpr int BLOCK = TPR < 256 ? 256 : TPR;
  constexpr int RPB = BLOCK / TPR;
  const int64_t grid = fg_cdiv(M, RPB);
  hipLaunchKernelGGL((rms_rows_kernel<T, VEC, ITERS, TPR, FUSED>), dim3((unsigned)grid), dim3(BLOCK), 0, st, x, res,
                     w, y, inv_rms, M, N, xs, rs, ys, eps);
}

template <typename T, bool FUSED>
int rms_dispatch(const T* x, T* res, const T* w, T* y, float* inv_rms, int64_t M, int64_t N, int64_t xs, int64_t rs,
                 int64_t ys, float eps, hipStream_t st) {
  constexpr int VEC = 16 / sizeof(T);
  const bool vec_ok = (N % VEC == 0) && (xs % VEC == 0) && (ys % VEC == 0) && (!FUSED || rs % VEC == 0) &&
                      fg_aligned(x, 16) && fg_aligned(y, 16) && (!FUSED || fg_aligned(res, 16)) &&
                      (w == nullptr || fg_aligned(w, 16));
  const int64_t packs = vec_ok ? N / VEC : 0;
  if (M >= (int64_t)1 << 31) {
    fg_set_error("rms_norm: M=%lld exceeds the grid limit", (long long)M);
    return FG_ERR_UNSUPPORTED;
  }
#define FG_ROWS(ITERS, TPR) launch_rows<T, VEC, ITERS, TPR, FUSED>(x, res, w, y, inv_rms, M, (int)N, xs, rs, ys, eps, st)
  if (!vec_ok || packs > 1024 * 8) {
    if (N <= 512) {  // from there on the two-pass kernel with 256 threads measures faster
#define FG_SHORT(ITERS)                                                                                              \
  hipLaunchKernelGGL((rms_short_kernel<T, FUSED, ITERS>), dim3((unsigned)fg_cdiv(M, 4)), dim3(256), 0, st, x, res, w, y, \
                     inv_rms, M, (int)N, xs, rs, ys, eps)
      if (N <= 64) FG_SHORT(1);
      else if (N <= 128) FG_SHORT(2);
      else if (N <= 256) FG_SHORT(4);
      else FG_SHORT(8);
#undef FG_SHORT
    } else if (N >= 2048)
      hipLaunchKernelGGL((rms_looped_kernel<T, FUSED, 1024>), dim3((unsigned)M), dim3(1024), 0, st, x, res, w, y, inv_rms,
                         M, N, xs, rs, ys, eps);
    else
      hipLaunchKernelGGL((rms_looped_kernel<T, FUSED, 256>), dim3((unsigned)M), dim3(256), 0, st, x, res, w, y, inv_rms,
                         M, N, xs, rs, ys, eps);
  } else if (FUSED) {
    // Two input streams: one pack per thread from each wherever a row fits 1024 threads.  Measured on
    // MI355X this beats fewer threads holding several packs (16384 x 4096 bf16: 84.8 us at 1 x 512
    // threads per row against 92.8 us at 4 x 128), the extra waves keeping more requests in flight.
    if (packs <= 64) FG_ROWS(1, 64);
    else if (packs <= 128) FG_ROWS(1, 128);
    else if (packs <= 256) FG_ROWS(1, 256);
    else if (packs <= 512) FG_ROWS(1, 512);
    else if (packs <= 1024) FG_ROWS(1, 1024);
    else if (packs <= 2048) FG_ROWS(2, 1024);
    else if (packs <= 4096) FG_ROWS(4, 1024);
    else FG_ROWS(8, 1024);
  } else {
    // One input stream: two packs per thread give the same two 16-byte requests in flight per thread
    // (65536 x 4096 bf16: 171 us at 2 x 256 threads per row against 197 us at 1 x 512).
    if (packs <= 64) FG_ROWS(1, 64);
    else if (packs <= 128) FG_ROWS(2, 64);
    else if (packs <= 256) FG_ROWS(2, 128);
    else if (packs <= 512) FG_ROWS(2, 256);
    else if (packs <= 1024) FG_ROWS(2, 512);
    else if (packs <= 2048) FG_ROWS(2, 1024);
    else if (packs <= 4096) FG_ROWS(4, 1024);
    else FG_ROWS(8, 1024);
  }
#undef FG_ROWS
  return fg_check_launch(FUSED ? "fused_add_rms_norm" : "rms_norm");
}

}  // namespace

extern "C" int fg_rms_norm(const void* x, const void* w, void* y, float* inv_rms, int64_t M, int64_t N,
                           int64_t x_row_stride, int64_t y_row_stride, float eps, int dtype, void* stream) {
  FG_REQUIRE(M >= 0 && N >= 0, FG_ERR_INVALID, "rms_norm: negative size M=%lld N=%lld", (long long)M, (long long)N);
  if (M == 0 || N == 0) return FG_OK;
  FG_REQUIRE(x && y, FG_ERR_INVALID, "rms_norm: null pointer");
  FG_REQUIRE(N < ((int64_t)1 << 31), FG_ERR_UNSUPPORTED, "rms_norm: N=%lld too large", (long long)N);
  hipStream_t st = (hipStream_t)stream;
  switch (dtype) {
    case FG_F16:
      return rms_dispatch<f16_t, false>((const f16_t*)x, nullptr, (const f16_t*)w, (f16_t*)y, inv_rms, M, N,
                                        x_row_stride, 0, y_row_stride, eps, st);
    case FG_BF16:
      return rms_dispatch<bf16_t, false>((const bf16_t*)x, nullptr, (const bf16_t*)w, (bf16_t*)y, inv_rms, M, N,
                                         x_row_stride, 0, y_row_stride, eps, st);
    case FG_F32:
      return rms_dispatch<float, false>((const float*)x, nullptr, (const float*)w, (float*)y, inv_rms, M, N,
                                        x_row_stride, 0, y_row_stride, eps, st);
  }
  fg_set_error("rms_norm: unsupported dtype %d", dtype);
  return FG_ERR_INVALID;
}

extern "C" int fg_fused_add_rms_norm(void* x, void* residual, const void* w, int64_t M, int64_t N,
                                     int64_t x_row_stride, int64_t r_row_stride, float eps, int dtype, void* stream) {
  FG_REQUIRE(M >= 0 && N >= 0, FG_ERR_INVALID, "fused_add_rms_norm: negative size");
  if (M == 0 || N == 0) return FG_OK;
  FG_REQUIRE(x && residual && w, FG_ERR_INVALID, "fused_add_rms_norm: null pointer");
  FG_REQUIRE(N < ((int64_t)1 << 31), FG_ERR_UNSUPPORTED, "fused_add_rms_norm: N=%lld too large", (long long)N);
  hipStream_t st = (hipStream_t)stream;
  switch (dtype) {
    case FG_F16:
      return rms_dispatch<f16_t, true>((const f16_t*)x, (f16_t*)residual, (const f16_t*)w, (f16_t*)x, nullptr, M, N,
                                       x_row_stride, r_row_stride, x_row_stride, eps, st);
    case FG_BF16:
      return rms_dispatch<bf16_t, true>((const bf16_t*)x, (bf16_t*)residual, (const bf16_t*)w, (bf16_t*)x, nullptr, M,
                                        N, x_row_stride, r_row_stride, x_row_stride, eps, st);
    case FG_F32:
      return rms_dispatch<float, true>((const float*)x, (float*)residual, (const float*)w, (float*)x, nullptr, M, N,
                                       x_row_stride, r_row_stride, x_row_stride, eps, st);
  }
  fg_set_error("fused_add_rms_norm: unsupported dtype %d", dtype);
  return FG_ERR_INVALID;
}
