// Variable-length attention forward over a paged KV cache for gfx950 (FA2 semantics).
//
// Work split.  A workgroup is 4 waves; a wave owns RW = 32 query rows of one query head and keeps
// their running max / sum and the output accumulator in registers for the whole KV sweep.  The 4
// waves of a workgroup share every K/V tile through LDS, and they are chosen to need the same
// keys: with grouped-query attention the workgroup takes HPB = 4 (or 2) query heads that map to
// the same KV head over one 32-row (64-row) block, so each K/V byte fetched from the cache feeds
// 4 heads; with HPB = 1 the waves take 4 consecutive row blocks of one head.
//
// Matrix products (MFMA 32x32x16, fp32 accumulate), both computed transposed so that a lane owns
// ONE query row (lane % 32) and the softmax reductions stay inside the lane:
//   S^T[key, q] = K[key, :] . Q[q, :]      A operand = K tile rows (LDS, d-contiguous),
//                                          B operand = Q (registers, loaded once);
//   O^T[d, q]  += V^T[d, key] . P^T[key, q] A operand = V^T tile rows (LDS, key-contiguous),
//                                          B operand = P^T straight from the S^T accumulators.
// The S^T accumulator of lane (q, h = lane/32) holds rows (i/4)*8 + 4h + i%4, i = 0..15.  K rows
// are fed to the MFMA through the bit permutation sigma below so that those 16 values are keys
// 16*(i/8) + 8h + i%8: registers 8t..8t+7 are then exactly the 8 consecutive keys the B operand
// of the t-th PV MFMA wants from this lane, and no data moves between the two products.
//
// Softmax runs in the base-2 domain: t = logit * log2(e), p = exp2(t - max), with the logit being
// scale*S, or softcap*tanh(scale*S/softcap), plus the ALiBi bias, and -inf where masked (keys
// past the sequence, causal / sliding-window bounds aligned to the bottom-right corner).
// lse = max*ln2 + ln(sum); rows with no visible key give out = 0, lse = +inf.
//
// K/V tiles of 64 keys are gathered page by page (block_table -> page -> row), 16 bytes per lane,
// zero-filled past the sequence end so stale cache contents can never reach the accumulators.
// V is transposed on its way into LDS (8x8 register transposes with v_perm_b32).
#include <stdint.h>
#include <stdlib.h>
#include "fg_common.h"

namespace {

constexpr int kBN = 64;        // keys per tile
constexpr int kRW = 32;        // query rows per wave
constexpr int kVtPitch = 144;  // V^T tile: row = 64 keys * 2 B + 16 B pad
constexpr int kPageTabMaxBytes = 16384;  // LDS the asynchronous kernel may spend on block-table entries

template <typename T> struct AttnMfma;
template <> struct AttnMfma<bf16_t> {
  typedef bf16x8 Frag;
  static __device__ __forceinline__ f32x16 mma(Frag a, Frag b, f32x16 c) {
    return __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, c, 0, 0, 0);
  }
  // 16x16 outputs over 32 k: A = 16 rows x 8 k per lane group of 16, B likewise by column, C column-major by lane
  static __device__ __forceinline__ f32x4 mma16(Frag a, Frag b, f32x4 c) {
    return __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, b, c, 0, 0, 0);
  }
};
template <> struct AttnMfma<f16_t> {
  typedef f16x8 Frag;
  static __device__ __forceinline__ f32x16 mma(Frag a, Frag b, f32x16 c) {
    return __builtin_amdgcn_mfma_f32_32x32x16_f16(a, b, c, 0, 0, 0);
  }
  static __device__ __forceinline__ f32x4 mma16(Frag a, Frag b, f32x4 c) {
    return __builtin_amdgcn_mfma_f32_16x16x32_f16(a, b, c, 0, 0, 0);
  }
};

struct AttnArgs {
  FgFlashParams p;
  int hpb;            // query heads per workgroup (1, 2 or 4)
  int rows_per_block; // query rows per workgroup = 128 / hpb
  int has_right, has_left;  // mask bounds in use
  int right_off_w, left_off_w;  // window_right / window_left as used by the bounds
  float scale_log2;   // softmax_scale * log2(e)   (softcap == 0)
  float cap_in, cap_out_log2;  // softcap: t = cap_out_log2 * tanh(S * cap_in)
  int page_shift;     // log2(page_size) when it is a power of two, else -1
  int use_async;      // take the asynchronous-tile kernel (head dims 64, 96, 128, 192, 256)
  int nw, nst;        // waves per workgroup and LDS stages of the asynchronous kernel
  int page_tab_entries;  // block-table entries the asynchronous kernel keeps in LDS (0: read them from global memory)
  int use_fast;       // take the lean kernel (head dim 64/128, power-of-two pages, no ALiBi, no soft-cap)
  int skip_single;    // mixed batch: sequences with one query token are left to the single-token kernel
  int xcd_remap;      // lean kernel: workgroup order regrouped per XCD
};

// MFMA row slot s (0..31) of a K sub-tile -> key offset inside the 32-key sub-tile.
__device__ __forceinline__ int sigma(int s) {
  return ((s >> 4) & 1) * 16 + ((s >> 2) & 1) * 8 + ((s >> 3) & 1) * 4 + (s & 3);
}

template <typename T, int DP>
__global__ __launch_bounds__(256) void attn_varlen_kernel(AttnArgs a) {
  typedef typename AttnMfma<T>::Frag Frag;
  constexpr int KPITCH = DP * 2 + 16;  // bytes per K tile row
  constexpr int KS = DP / 16;          // MFMA k-steps over the head dim
  constexpr int DT = DP / 32;          // 32-row output sub-tiles over the head dim
  __shared__ __attribute__((aligned(16))) char k_lds[kBN * KPITCH];
  __shared__ __attribute__((aligned(16))) char vt_lds[DP * kVtPitch];

  const FgFlashParams& p = a.p;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int half = lane >> 5, ql = lane & 31;
  const int b = blockIdx.y, hgroup = blockIdx.z;
  // rotated per (sequence, head group) so that sequences of one row block do not all land on one XCD
  const int m_block = (int)((blockIdx.x + (unsigned)(b * 5 + hgroup * 3)) % gridDim.x);

  const int q_bos = p.cu_seqlens_q[b];
  const int q_len = p.cu_seqlens_q[b + 1] - q_bos;
  const int k_len = p.seqused_k[b];
  const int block_row0 = m_block * a.rows_per_block;
  if (block_row0 >= q_len || (a.skip_single && q_len == 1)) return;

  // wave -> (head, row block)
  const int waves_per_head = 4 / a.hpb;
  const int head = hgroup * a.hpb + wave / waves_per_head;
  const int row0 = block_row0 + (wave % waves_per_head) * kRW;  // first row of this wave in the sequence
  const int kv_head = head / (p.Hq / p.Hk);
  const int D = p.D;

  // ---- key range of the workgroup --------------------------------------------------------------
  const int shift = k_len - q_len;  // bottom-right alignment
  int n_max = (k_len + kBN - 1) / kBN;
  if (a.has_right) {
    const int last = block_row0 + a.rows_per_block + shift + a.right_off_w;  // exclusive key bound
    const int lim = last <= 0 ? 0 : (last + kBN - 1) / kBN;
    n_max = n_max < lim ? n_max : lim;
  }
  int n_min = 0;
  if (a.has_left) {
    const int first = block_row0 + shift - a.left_off_w;
    n_min = first <= 0 ? 0 : first / kBN;
  }

  // ---- Q fragments (B operand): lane (q = ql, half) holds d = 16*ks + 8*half .. +8 ----------------
  Frag qf[KS];
  {
    const int qrow = row0 + ql;
    const bool row_ok = qrow < q_len;
    const T* qp = (const T*)p.q + (int64_t)(q_bos + (row_ok ? qrow : 0)) * p.q_row_stride + (int64_t)head * p.q_head_stride;
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) {
      const int d = ks * 16 + half * 8;
      u32x4 v = {0u, 0u, 0u, 0u};
      if (row_ok && d < D) v = *reinterpret_cast<const u32x4*>(qp + d);
      qf[ks] = __builtin_bit_cast(Frag, v);
    }
  }

  f32x16 o_acc[DT];
#pragma unroll
  for (int dt = 0; dt < DT; ++dt)
#pragma unroll
    for (int e = 0; e < 16; ++e) o_acc[dt][e] = 0.f;
  float m_run = -INFINITY, l_run = 0.f;

  float slope = 0.f;
  if (p.alibi_slopes != nullptr) slope = p.alibi_slopes[(int64_t)b * p.alibi_batch_stride + head] * 1.4426950408889634f;
  const bool softcap = p.softcap > 0.f;

  const int32_t* btab = p.block_table + (int64_t)b * p.block_table_stride;
  const T* kbase = (const T*)p.k_cache + (int64_t)kv_head * p.k_head_stride;
  const T* vbase = (const T*)p.v_cache + (int64_t)kv_head * p.v_head_stride;
  const int page_size = p.page_size;
  const int CPR = D / 8;  // 16-byte chunks per K/V row

  const bool wave_rows_ok = row0 < q_len;
  const int wave_row_last = (row0 + kRW - 1 < q_len ? row0 + kRW - 1 : q_len - 1);

  for (int nb = n_min; nb < n_max; ++nb) {
    const int key0 = nb * kBN;
    __syncthreads();  // the previous tile is fully consumed
    if (tid >= 128) {
      // K tile: 16-byte chunks, row-major copy.  chunk index -> (key, d-chunk)
      for (int idx = tid - 128; idx < kBN * (DP / 8); idx += 128) {
        const int r = idx / (DP / 8), c = idx - r * (DP / 8);
        const int key = key0 + r;
        u32x4 v = {0u, 0u, 0u, 0u};
        if (key < k_len && c < CPR) {
          const int pg = key / page_size;
          const int64_t page = btab[pg];
          v = *reinterpret_cast<const u32x4*>(kbase + page * p.k_page_stride + (int64_t)(key - pg * page_size) * p.k_row_stride + c * 8);
        }
        *reinterpret_cast<u32x4*>(k_lds + r * KPITCH + c * 16) = v;
      }
    } else {
      // V tile: 8(key) x 8(d) blocks, transposed to V^T[d][key].  block index -> (d-chunk, key block)
      for (int blk = tid; blk < (kBN / 8) * (DP / 8); blk += 128) {
        const int c = blk % (DP / 8), kb = blk / (DP / 8);
        u32x4 v[8];
#pragma unroll
        for (int j = 0; j < 8; ++j) {
          const int key = key0 + kb * 8 + j;
          v[j] = u32x4{0u, 0u, 0u, 0u};
          if (key < k_len && c < CPR) {
            const int pg = key / page_size;
            const int64_t page = btab[pg];
            v[j] = *reinterpret_cast<const u32x4*>(vbase + page * p.v_page_stride + (int64_t)(key - pg * page_size) * p.v_row_stride + c * 8);
          }
        }
#pragma unroll
        for (int dd = 0; dd < 8; ++dd) {
          const unsigned sel = (dd & 1) ? 0x07060302u : 0x05040100u;
          u32x4 o;
#pragma unroll
          for (int w = 0; w < 4; ++w) o[w] = __builtin_amdgcn_perm(v[2 * w + 1][dd >> 1], v[2 * w][dd >> 1], sel);
          *reinterpret_cast<u32x4*>(vt_lds + (c * 8 + dd) * kVtPitch + kb * 16) = o;
        }
      }
    }
    __syncthreads();

    if (!wave_rows_ok) continue;
    // tile visibility for this wave's rows
    if (a.has_right && key0 > wave_row_last + shift + a.right_off_w) continue;
    if (a.has_left && key0 + kBN - 1 < row0 + shift - a.left_off_w) continue;

    // ---- S^T = K . Q^T ---------------------------------------------------------------------------
    f32x16 s_acc[2];
#pragma unroll
    for (int kt = 0; kt < 2; ++kt) {
#pragma unroll
      for (int e = 0; e < 16; ++e) s_acc[kt][e] = 0.f;
      const char* krow = k_lds + (kt * 32 + sigma(ql)) * KPITCH + half * 16;
#pragma unroll
      for (int ks = 0; ks < KS; ++ks) {
        Frag kf = *reinterpret_cast<const Frag*>(krow + ks * 32);
        s_acc[kt] = AttnMfma<T>::mma(kf, qf[ks], s_acc[kt]);
      }
    }

    // ---- logits in the base-2 domain, masks ------------------------------------------------------
    const int qrow = row0 + ql;  // this lane's query row
    const bool need_mask = (key0 + kBN > k_len) || (a.has_right && key0 + kBN - 1 > row0 + shift + a.right_off_w) ||
                           (a.has_left && key0 < wave_row_last + shift - a.left_off_w);
    const int col_hi = a.has_right ? (qrow + shift + a.right_off_w < k_len - 1 ? qrow + shift + a.right_off_w : k_len - 1)
                                   : k_len - 1;
    const int col_lo = a.has_left ? qrow + shift - a.left_off_w : 0;
    float tmax = -INFINITY;
#pragma unroll
    for (int kt = 0; kt < 2; ++kt)
#pragma unroll
      for (int e = 0; e < 16; ++e) {
        const int col = key0 + kt * 32 + (e >> 3) * 16 + half * 8 + (e & 7);
        float t = s_acc[kt][e];
        if (softcap) t = a.cap_out_log2 * tanhf(t * a.cap_in);
        else t = t * a.scale_log2;
        if (p.alibi_slopes != nullptr) {
          if (p.is_causal) t += slope * (float)(col - k_len + 1);
          else t -= slope * fabsf((float)(col - shift - qrow));
        }
        if (need_mask && (col > col_hi || col < col_lo)) t = -INFINITY;
        s_acc[kt][e] = t;
        tmax = fmaxf(tmax, t);
      }
    tmax = fmaxf(tmax, __shfl_xor(tmax, 32, 64));
    const float m_new = fmaxf(m_run, tmax);
    const float m_use = m_new == -INFINITY ? 0.f : m_new;
    const float alpha = exp2f(m_run - m_use);
    float psum = 0.f;
    Frag pf[4];
#pragma unroll
    for (int kt = 0; kt < 2; ++kt)
#pragma unroll
      for (int t2 = 0; t2 < 2; ++t2) {
        T tmp[8];
#pragma unroll
        for (int e = 0; e < 8; ++e) {
          const float pv = exp2f(s_acc[kt][t2 * 8 + e] - m_use);
          psum += pv;
          tmp[e] = (T)pv;
        }
        pf[kt * 2 + t2] = *reinterpret_cast<Frag*>(tmp);
      }
    psum += __shfl_xor(psum, 32, 64);
    l_run = l_run * alpha + psum;
    m_run = m_new;

    // ---- O^T = O^T * alpha + V^T . P^T ------------------------------------------------------------
#pragma unroll
    for (int dt = 0; dt < DT; ++dt) {
#pragma unroll
      for (int e = 0; e < 16; ++e) o_acc[dt][e] *= alpha;
      const char* vrow = vt_lds + (dt * 32 + ql) * kVtPitch + half * 16;
#pragma unroll
      for (int t4 = 0; t4 < 4; ++t4) {
        Frag vf = *reinterpret_cast<const Frag*>(vrow + t4 * 32);
        o_acc[dt] = AttnMfma<T>::mma(vf, pf[t4], o_acc[dt]);
      }
    }
  }

  // ---- epilogue -----------------------------------------------------------------------------------
  const int qrow = row0 + ql;
  if (qrow >= q_len) return;
  const bool empty = l_run == 0.f || l_run != l_run;
  const float inv = empty ? 1.f : 1.f / l_run;
  if (p.lse != nullptr && half == 0) {
    p.lse[(int64_t)head * p.total_q + q_bos + qrow] = empty ? INFINITY : m_run * 0.6931471805599453f + logf(l_run);
  }
  T* op = (T*)p.out + (int64_t)(q_bos + qrow) * p.o_row_stride + (int64_t)head * p.o_head_stride;
#pragma unroll
  for (int dt = 0; dt < DT; ++dt)
#pragma unroll
    for (int g = 0; g < 4; ++g) {
      const int d = dt * 32 + g * 8 + half * 4;
      if (d < D) {  // D is a multiple of 8, so a group of 4 is all inside or all outside
        Pack<T, 4> o;
#pragma unroll
        for (int e = 0; e < 4; ++e) o.v[e] = (T)(o_acc[dt][g * 4 + e] * inv);
        st_pack<T, 4>(op + d, o);
      }
    }
}

// =============================================================================================
// Fast path: asynchronous K/V tiles.
//
// Same work split and the same two transposed products as the kernel above; what changes is how
// the tiles travel and how the waves overlap:
//   * K and V tiles (64 keys x D) go from the paged cache straight into LDS with
//     global_load_lds_dwordx4 (no staging registers, no LDS store instructions), two stages deep:
//     the tile for step j+1 is in flight while step j computes; one s_waitcnt vmcnt + one barrier
//     per step.  Keys past the sequence end are clamped to the last valid key: their scores are
//     masked to -inf, so their probability is an exact zero and the duplicate rows never count.
//   * LDS rows are RB = 2*D bytes rounded up to a power of two, with the 16-byte chunks of row
//     `key` stored at position chunk ^ swz(key).  swz is a bit permutation of key & 15 chosen so
//     that (a) the 16 keys a quarter-wave reads for one K fragment and (b) the 4 keys x 32 bytes a
//     16-lane group reads for one transposed V fragment both fall into disjoint banks.
//   * V stays in its natural [key][d] layout; the V^T MFMA operand (8 consecutive keys of one d
//     per lane) is produced by ds_read_b64_tr_b16, which hands lane i of a 16-lane group the i-th
//     16-bit column of the 4 rows x 64 bits the group addresses.
//   * exp2 is the bare v_exp_f32; the softmax scale is folded into one fma per score; the output
//     accumulator is rescaled only when a row maximum actually moved.
//   * at most 256 VGPRs, so two workgroups share a CU and one workgroup's softmax (VALU) overlaps
//     the other's MFMAs.
// =============================================================================================
#define FG_LDSP(p) ((__attribute__((address_space(3))) void*)(p))
#define FG_GLBP(p) ((const __attribute__((address_space(1))) void*)(p))
#define FG_WAIT_VM(N) __builtin_amdgcn_s_waitcnt(((N) & 0xF) | (7 << 4) | (0xF << 8) | (((N) >> 4) << 14))
typedef short s16x4 __attribute__((ext_vector_type(4)));

// ---- LDS reads the compiler must not reorder or guard ------------------------------------------------
// The tile DMAs of later steps are still in flight while a step computes.  The compiler cannot tell
// that they target other LDS stages and would wait for all of them (vmcnt(0)) before a transposing
// LDS read; and left to itself it sinks every fragment read next to its first use.  So fragment
// reads are issued through inline asm in groups, software-pipelined by hand: wait for group g (a full
// lgkmcnt(0), tied to the group's registers), issue the reads of group g+1, then issue the MFMAs of
// group g, which execute while the next reads are in flight.
__device__ __forceinline__ uint32_t lds_off(const void* p) {
  return (uint32_t)(uintptr_t)(__attribute__((address_space(3))) const char*)p;
}
__device__ __forceinline__ u32x4 lds_read_b128(uint32_t addr) {
  u32x4 v;
  asm volatile("ds_read_b128 %0, %1" : "=v"(v) : "v"(addr));
  return v;
}
__device__ __forceinline__ u32x2 lds_read_tr_b64(uint32_t addr) {
  u32x2 v;
  asm volatile("ds_read_b64_tr_b16 %0, %1" : "=v"(v) : "v"(addr));
  return v;
}
// Combine a value with the one held by lane ^ 32 without going through LDS: v_permlane32_swap
// exchanges the upper half of its first register with the lower half of its second, so with both
// holding v on entry the first ends as the lower-half value and the second as the upper-half value
// of every lane position.  Written as asm because the builtin's second result is not usable with
// this compiler; the no-ops cover the VALU-write -> permlane-read distance the compiler would
// otherwise insert itself.
__device__ __forceinline__ void xhalf_split(float v, float& lo, float& hi) {
  lo = v;
  hi = v;
  asm volatile("s_nop 1\n\tv_permlane32_swap_b32 %0, %1\n\ts_nop 1" : "+v"(lo), "+v"(hi));
}
__device__ __forceinline__ float xhalf_max(float v) {
  float lo, hi;
  xhalf_split(v, lo, hi);
  return fmaxf(lo, hi);
}
__device__ __forceinline__ float xhalf_sum(float v) {
  float lo, hi;
  xhalf_split(v, lo, hi);
  return lo + hi;
}

// Wait for every outstanding LDS read (and scalar load: they share the counter, and scalar loads
// retire out of order, so a partial count can never be trusted here), tied to a group's registers.
template <typename V>
__device__ __forceinline__ void lds_wait_all(V (&r)[8]) {
  asm volatile("s_waitcnt lgkmcnt(0)"
               : "+v"(r[0]), "+v"(r[1]), "+v"(r[2]), "+v"(r[3]), "+v"(r[4]), "+v"(r[5]), "+v"(r[6]), "+v"(r[7]));
}

// Chunk swizzle: 16-byte chunk c of LDS row `key` is stored at position c ^ swz(key).
// Written with key bits k3 k2 k1 k0:
//   rows of 16 or 32 chunks: swz = (k1, k0, k3, k2).  The 16 keys of one K-fragment read get 16
//     different values (a bit permutation), so a quarter-wave of ds_read_b128 covers all banks once.
//     For a transposed V read the 32-byte pair index is swz >> 1 = (k1, k0, k3): the 4 consecutive keys
//     of a 16-lane group land in pairs P ^ {0, 2, 4, 6} (+k3), and the neighbouring group, which
//     reads pair P + 1 of the same keys in the same cycle, in (P + 1) ^ {0, 2, 4, 6}: disjoint.
//   rows of 8 chunks (two rows per 256 bytes of banks, row parity = k0): swz = (k1, k2, k3); the
//     same two properties hold with the row parity taking the place of the missing bit.
template <int CPR>
__device__ __forceinline__ int swz(int key) {
  if constexpr (CPR >= 16) return ((key & 3) << 2) | (((key >> 3) & 1) << 1) | ((key >> 2) & 1);
  else return (((key >> 1) & 1) << 2) | (((key >> 2) & 1) << 1) | ((key >> 3) & 1);
}

template <typename T, int D, int RB, int NW, int NST, bool LP>
__global__ __launch_bounds__(NW * 64, (RB <= 256 ? 2 : 1)) void attn_varlen_async_kernel(AttnArgs a) {
  typedef typename AttnMfma<T>::Frag Frag;
  constexpr int CPR = RB / 16;          // 16-byte chunks per LDS row
  constexpr int VALID_C = D / 8;        // chunks that hold data
  constexpr int KS = D / 16;            // MFMA k-steps over the head dim
  constexpr int DT = (D + 31) / 32;     // 32-row output sub-tiles over the head dim
  constexpr int OPB = kBN * RB;         // bytes of one operand tile
  constexpr int STAGEB = 2 * OPB;       // K tile + V tile
  constexpr int IPW = RB / 16 / NW;     // DMA instructions per wave per operand per tile
  extern __shared__ __attribute__((aligned(16))) char lds[];

  const FgFlashParams& p = a.p;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int half = lane >> 5, ql = lane & 31;
  // long (late) row blocks first: they take the most steps under a causal mask
  // Long (late) row blocks first, and the order rotated per (sequence, head group): workgroups go round-robin to the
  // 8 XCDs by their linear id, so without the rotation a batch whose sequences have one row block each (and
  // gridDim.x a multiple of 8) would put all of its work on one XCD.
  const int b = blockIdx.y, hgroup = blockIdx.z;
  const int m_block = (int)((gridDim.x - 1 - blockIdx.x + (unsigned)(b * 5 + hgroup * 3)) % gridDim.x);

  const int q_bos = p.cu_seqlens_q[b];
  const int q_len = p.cu_seqlens_q[b + 1] - q_bos;
  const int k_len = p.seqused_k[b];
  const int block_row0 = m_block * a.rows_per_block;
  if (block_row0 >= q_len || (a.skip_single && q_len == 1)) return;

  const int waves_per_head = NW / a.hpb;
  const int head = hgroup * a.hpb + wave / waves_per_head;
  const int row0 = block_row0 + (wave % waves_per_head) * kRW;
  const int kv_head = head / (p.Hq / p.Hk);

  const int shift = k_len - q_len;
  int n_max = (k_len + kBN - 1) / kBN;
  if (a.has_right) {
    const int last = block_row0 + a.rows_per_block + shift + a.right_off_w;
    const int lim = last <= 0 ? 0 : (last + kBN - 1) / kBN;
    n_max = n_max < lim ? n_max : lim;
  }
  int n_min = 0;
  if (a.has_left) {
    const int first = block_row0 + shift - a.left_off_w;
    n_min = first <= 0 ? 0 : first / kBN;
  }

  // ---- Q fragments (async kernel) -----------------------------------------------------------------
  Frag qf[KS];
  {
    const int qrow = row0 + ql;
    const bool row_ok = qrow < q_len;
    const T* qp = (const T*)p.q + (int64_t)(q_bos + (row_ok ? qrow : 0)) * p.q_row_stride + (int64_t)head * p.q_head_stride;
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) {
      u32x4 v = {0u, 0u, 0u, 0u};
      if (row_ok) v = *reinterpret_cast<const u32x4*>(qp + ks * 16 + half * 8);
      qf[ks] = __builtin_bit_cast(Frag, v);
    }
  }

  f32x16 o_acc[DT];
#pragma unroll
  for (int dt = 0; dt < DT; ++dt)
#pragma unroll
    for (int e = 0; e < 16; ++e) o_acc[dt][e] = 0.f;
  float m_run = -INFINITY, l_run = 0.f;  // running max (base-2 logits) and running sum

  float slope = 0.f;
  if (p.alibi_slopes != nullptr) slope = p.alibi_slopes[(int64_t)b * p.alibi_batch_stride + head] * 1.4426950408889634f;
  const bool softcap = p.softcap > 0.f;

  const int32_t* btab = p.block_table + (int64_t)b * p.block_table_stride;
  const char* kbase = (const char*)((const T*)p.k_cache + (int64_t)kv_head * p.k_head_stride);
  const char* vbase = (const char*)((const T*)p.v_cache + (int64_t)kv_head * p.v_head_stride);
  const int page_size = p.page_size;
  const int page_shift = a.page_shift;  // log2(page_size) or -1

  // ---- DMA lane geometry (fixed per thread) -------------------------------------------------------
  // instruction n = wave*IPW + j of an operand tile fills LDS bytes [n*1024, n*1024 + 1024); lane L
  // lands at n*1024 + L*16 -> (key_l, position) and fetches the chunk that belongs there.
  int dma_key[IPW], dma_coff[IPW];
#pragma unroll
  for (int j = 0; j < IPW; ++j) {
    const int off = (wave * IPW + j) * 1024 + lane * 16;
    const int key_l = off / RB, pos = (off % RB) / 16;
    int c = pos ^ swz<CPR>(key_l);
    if (c >= VALID_C) c = 0;  // padding region of the row: any finite data will do
    dma_key[j] = key_l;
    dma_coff[j] = c * 16;
  }
  // Page ids.  The slice of the block table this workgroup walks is copied into LDS once, behind the
  // tile stages, and every DMA lane looks its page up there: LDS reads retire on their own counter
  // (lgkmcnt), so waiting for a page id never waits for a tile DMA (vmcnt), whereas a page id read
  // from global memory after a DMA would, because memory operations retire in order.  When the
  // slice does not fit the space reserved for it (LP == false) the ids are read from global memory.
  int32_t* lds_pages = reinterpret_cast<int32_t*>(lds + NST * STAGEB);
  const int pg_base = page_shift >= 0 ? ((n_min * kBN) >> page_shift) : (n_min * kBN) / page_size;
  if constexpr (LP) {
    const int last_key = (n_max * kBN < k_len ? n_max * kBN : k_len) - 1;
    const int pg_last = last_key < 0 ? pg_base - 1 : (page_shift >= 0 ? (last_key >> page_shift) : last_key / page_size);
    int count = pg_last - pg_base + 1;
    count = count < a.page_tab_entries ? count : a.page_tab_entries;
    for (int i = tid; i < count; i += NW * 64) lds_pages[i] = btab[pg_base + i];
    __syncthreads();
  }
  int pg_id[IPW], pg_idx[IPW];
  auto fetch_pages = [&](int nb) {
    const int key0 = nb * kBN;
#pragma unroll
    for (int j = 0; j < IPW; ++j) {
      int key = key0 + dma_key[j];
      key = key < k_len ? key : k_len - 1;
      const int pg = page_shift >= 0 ? (key >> page_shift) : key / page_size;
      pg_idx[j] = pg;
      if constexpr (LP) {
        int rel = pg - pg_base;
        rel = rel < a.page_tab_entries ? rel : a.page_tab_entries - 1;  // never read past the table
        pg_id[j] = lds_pages[rel];
      } else {
        pg_id[j] = btab[pg];
      }
    }
  };
  auto issue_tile = [&](int nb, int stage) {
    const int key0 = nb * kBN;
    int64_t koff[IPW], voff[IPW];
#pragma unroll
    for (int j = 0; j < IPW; ++j) {
      int key = key0 + dma_key[j];
      key = key < k_len ? key : k_len - 1;
      const int64_t page = pg_id[j];
      const int slot = key - pg_idx[j] * page_size;
      koff[j] = (page * p.k_page_stride + (int64_t)slot * p.k_row_stride) * (int64_t)sizeof(T) + dma_coff[j];
      voff[j] = (page * p.v_page_stride + (int64_t)slot * p.v_row_stride) * (int64_t)sizeof(T) + dma_coff[j];
    }
    char* kdst = lds + stage * STAGEB + wave * IPW * 1024;
    char* vdst = kdst + OPB;
#pragma unroll
    for (int j = 0; j < IPW; ++j) {
      __builtin_amdgcn_global_load_lds(FG_GLBP(kbase + koff[j]), FG_LDSP(kdst + j * 1024), 16, 0, 0);
      __builtin_amdgcn_global_load_lds(FG_GLBP(vbase + voff[j]), FG_LDSP(vdst + j * 1024), 16, 0, 0);
    }
  };

  // ---- fragment addressing (fixed per lane) ---------------------------------------------------------
  // K fragment: row sigma(ql) of key sub-tile kt, chunk ks*2 + half  ->  ((ks*2) ^ kx) * 16 with kx = half ^ swz
  const int k_row = sigma(ql);
  const int k_lane = k_row * RB;
  const int kx = half ^ swz<CPR>(k_row);
  // V^T fragment via transposing reads: source lane s = lane%16 addresses key (s/4) of a group of 4 and the
  // 8-byte piece (s%4) of the 32 bytes that hold d0 .. d0+15, d0 = dt*32 + 16*((lane/16)%2)
  const int vs = lane & 15;
  const int v_key0 = half * 8 + (vs >> 2);        // + t4*16 (+4 for the second read)
  const int v_cc = 2 * ((lane >> 4) & 1) + ((vs & 3) >> 1);
  const int v_byte = (vs & 1) * 8;
  const int vx0 = v_cc ^ swz<CPR>(v_key0), vx1 = v_cc ^ swz<CPR>(v_key0 + 4);
  const int v_lane0 = v_key0 * RB + v_byte, v_lane1 = (v_key0 + 4) * RB + v_byte;

  const bool wave_rows_ok = row0 < q_len;
  const int wave_row_last = (row0 + kRW - 1 < q_len ? row0 + kRW - 1 : q_len - 1);
  const int qrow = row0 + ql;

  // Prologue: NST-1 tiles in flight.  In the loop, tile nb has landed once at most NST-2 newer steps
  // (2*IPW DMA instructions each, plus IPW page-id loads before them when those are global loads)
  // are outstanding.
  // vmcnt events per step: 2*IPW DMA, plus IPW page-id loads when those come from global memory
  constexpr int PER_TILE = LP ? 2 * IPW : 3 * IPW;
#pragma unroll
  for (int s0 = 0; s0 < NST - 1; ++s0) {
    if (n_min + s0 < n_max) {
      fetch_pages(n_min + s0);
      issue_tile(n_min + s0, s0);
    }
  }
  for (int nb = n_min; nb < n_max; ++nb) {
    const int stage = (nb - n_min) % NST;
    const int key0 = nb * kBN;
    if (NST > 2 && nb + NST - 2 < n_max) {
      FG_WAIT_VM((NST - 2) * PER_TILE);
    } else {
      FG_WAIT_VM(0);                 // this wave's share of tile nb has landed
    }
    __builtin_amdgcn_s_barrier();    // ... everybody's has, and nobody still reads the stage refilled next
    if (nb + NST - 1 < n_max) {
      fetch_pages(nb + NST - 1);
      issue_tile(nb + NST - 1, (nb - n_min + NST - 1) % NST);
    }

    if (!wave_rows_ok) continue;
    if (a.has_right && key0 > wave_row_last + shift + a.right_off_w) continue;
    if (a.has_left && key0 + kBN - 1 < row0 + shift - a.left_off_w) continue;

    const uint32_t ks_base = lds_off(lds) + stage * STAGEB + k_lane;
    const uint32_t vs_base = lds_off(lds) + stage * STAGEB + OPB;

    // ---- S^T = K . Q^T : K fragments in groups of GS reads, one group ahead of the MFMAs ---------------
    constexpr int GS = KS < 8 ? KS : 8;        // reads per group
    constexpr int NGK = 2 * KS / GS;           // groups over both key sub-tiles
    f32x16 s_acc[2];
#pragma unroll
    for (int kt = 0; kt < 2; ++kt)
#pragma unroll
      for (int e = 0; e < 16; ++e) s_acc[kt][e] = 0.f;
    {
      u32x4 kf[2][8];
      auto issue_k = [&](int g, u32x4 (&dst)[8]) {
#pragma unroll
        for (int r = 0; r < GS; ++r) {
          const int idx = g * GS + r, kt = idx / KS, ks = idx % KS;
          dst[r] = lds_read_b128(ks_base + kt * 32 * RB + (((ks * 2) ^ kx) * 16));
        }
      };
      issue_k(0, kf[0]);
#pragma unroll
      for (int g = 0; g < NGK; ++g) {
        lds_wait_all(kf[g & 1]);
        if (g + 1 < NGK) issue_k(g + 1, kf[(g + 1) & 1]);
#pragma unroll
        for (int r = 0; r < GS; ++r) {
          const int idx = g * GS + r, kt = idx / KS, ks = idx % KS;
          s_acc[kt] = AttnMfma<T>::mma(__builtin_bit_cast(Frag, kf[g & 1][r]), qf[ks], s_acc[kt]);
        }
      }
    }

    // ---- base-2 logits, masks, running max -----------------------------------------------------------
    const bool need_mask = (key0 + kBN > k_len) || (a.has_right && key0 + kBN - 1 > row0 + shift + a.right_off_w) ||
                           (a.has_left && key0 < wave_row_last + shift - a.left_off_w);
    const bool plain = !softcap && p.alibi_slopes == nullptr;
    float tmax = -INFINITY;
    if (plain && !need_mask) {
      // interior tile: raw scores; scale folded into the exponent below
#pragma unroll
      for (int kt = 0; kt < 2; ++kt)
#pragma unroll
        for (int e = 0; e < 16; ++e) tmax = fmaxf(tmax, s_acc[kt][e]);
      tmax *= a.scale_log2;  // scale > 0, so max commutes with it
    } else {
      const int col_hi = a.has_right ? (qrow + shift + a.right_off_w < k_len - 1 ? qrow + shift + a.right_off_w : k_len - 1)
                                     : k_len - 1;
      const int col_lo = a.has_left ? qrow + shift - a.left_off_w : 0;
#pragma unroll
      for (int kt = 0; kt < 2; ++kt)
#pragma unroll
        for (int e = 0; e < 16; ++e) {
          const int col = key0 + kt * 32 + (e >> 3) * 16 + half * 8 + (e & 7);
          float t = s_acc[kt][e];
          if (softcap) t = a.cap_out_log2 * tanhf(t * a.cap_in);
          else t = t * a.scale_log2;
          if (p.alibi_slopes != nullptr) {
            if (p.is_causal) t += slope * (float)(col - k_len + 1);
            else t -= slope * fabsf((float)(col - shift - qrow));
          }
          if (col > col_hi || col < col_lo) t = -INFINITY;
          s_acc[kt][e] = t;
          tmax = fmaxf(tmax, t);
        }
    }
    tmax = xhalf_max(tmax);
    // The reference maximum of a row moves only when the new maximum exceeds it by more than 2^8:
    // any reference gives the same result as long as p and the running sum use the same one, and
    // p <= 256 is harmless in bf16/fp16.  After the first steps almost no step has to rescale.
    const bool moved = tmax > m_run + 8.0f;
    const float m_new = moved ? tmax : m_run;
    const float m_use = m_new == -INFINITY ? 0.f : m_new;
    const float alpha = moved ? __builtin_amdgcn_exp2f(m_run - m_use) : 1.0f;
    float psum = 0.f;
    Frag pf[4];
    const float sc = (plain && !need_mask) ? a.scale_log2 : 1.0f;
#pragma unroll
    for (int kt = 0; kt < 2; ++kt)
#pragma unroll
      for (int t2 = 0; t2 < 2; ++t2) {
        T tmp[8];
#pragma unroll
        for (int e = 0; e < 8; ++e) {
          const float pv = __builtin_amdgcn_exp2f(fmaf(s_acc[kt][t2 * 8 + e], sc, -m_use));
          psum += pv;
          tmp[e] = (T)pv;
        }
        pf[kt * 2 + t2] = *reinterpret_cast<Frag*>(tmp);
      }
    psum = xhalf_sum(psum);
    l_run = l_run * alpha + psum;
    m_run = m_new;

    // ---- O^T = O^T * alpha + V^T . P^T  (rescale skipped while no reference maximum of this wave moved) ---
    if (__builtin_amdgcn_ballot_w64(moved) != 0) {
#pragma unroll
      for (int dt = 0; dt < DT; ++dt)
#pragma unroll
        for (int e = 0; e < 16; ++e) o_acc[dt][e] *= alpha;
    }
    {
      // V^T fragments: per d sub-tile 8 transposing reads (4 key chunks x 2 halves), one sub-tile ahead
      u32x2 vf[2][8];
      auto issue_v = [&](int dt, u32x2 (&dst)[8]) {
        const int o0 = ((dt * 4) ^ vx0) * 16, o1 = ((dt * 4) ^ vx1) * 16;
#pragma unroll
        for (int t4 = 0; t4 < 4; ++t4) {
          dst[2 * t4] = lds_read_tr_b64(vs_base + v_lane0 + t4 * 16 * RB + o0);
          dst[2 * t4 + 1] = lds_read_tr_b64(vs_base + v_lane1 + t4 * 16 * RB + o1);
        }
      };
      issue_v(0, vf[0]);
#pragma unroll
      for (int dt = 0; dt < DT; ++dt) {
        lds_wait_all(vf[dt & 1]);
        if (dt + 1 < DT) issue_v(dt + 1, vf[(dt + 1) & 1]);
#pragma unroll
        for (int t4 = 0; t4 < 4; ++t4) {
          const u32x4 both = {vf[dt & 1][2 * t4][0], vf[dt & 1][2 * t4][1], vf[dt & 1][2 * t4 + 1][0], vf[dt & 1][2 * t4 + 1][1]};
          o_acc[dt] = AttnMfma<T>::mma(__builtin_bit_cast(Frag, both), pf[t4], o_acc[dt]);
        }
      }
    }
  }

  // ---- epilogue -------------------------------------------------------------------------------------
  if (qrow >= q_len) return;
  const bool empty = l_run == 0.f || l_run != l_run;
  const float inv = empty ? 1.f : 1.f / l_run;
  if (p.lse != nullptr && half == 0) {
    p.lse[(int64_t)head * p.total_q + q_bos + qrow] = empty ? INFINITY : m_run * 0.6931471805599453f + logf(l_run);
  }
  T* op = (T*)p.out + (int64_t)(q_bos + qrow) * p.o_row_stride + (int64_t)head * p.o_head_stride;
#pragma unroll
  for (int dt = 0; dt < DT; ++dt)
#pragma unroll
    for (int g = 0; g < 4; ++g) {
      const int d = dt * 32 + g * 8 + half * 4;
      if (d < D) {
        Pack<T, 4> o;
#pragma unroll
        for (int e = 0; e < 4; ++e) o.v[e] = (T)(o_acc[dt][g * 4 + e] * inv);
        st_pack<T, 4>(op + d, o);
      }
    }
}

template <typename T, int D, int RB, int NW, int NST, bool LP>
int launch_async_lp(const AttnArgs& a, dim3 grid, hipStream_t st) {
  constexpr int STAGE_BYTES = NST * 2 * kBN * RB;
  constexpr int MAX_LDS = STAGE_BYTES + kPageTabMaxBytes;
  static hipError_t attr_err =
      hipFuncSetAttribute(reinterpret_cast<const void*>(attn_varlen_async_kernel<T, D, RB, NW, NST, LP>),
                          hipFuncAttributeMaxDynamicSharedMemorySize, MAX_LDS);
  if (attr_err != hipSuccess) {
    fg_set_error("flash_attn_varlen_fwd: cannot reserve %d bytes of LDS: %s", MAX_LDS, hipGetErrorString(attr_err));
    return FG_ERR_LAUNCH;
  }
  const int lds_bytes = STAGE_BYTES + (LP ? a.page_tab_entries * 4 : 0);
  hipLaunchKernelGGL((attn_varlen_async_kernel<T, D, RB, NW, NST, LP>), grid, dim3(NW * 64), lds_bytes, st, a);
  return fg_check_launch("flash_attn_varlen_fwd");
}
template <typename T, int D, int RB, int NW, int NST>
int launch_async(const AttnArgs& a, dim3 grid, hipStream_t st) {
  if (a.page_tab_entries > 0) return launch_async_lp<T, D, RB, NW, NST, true>(a, grid, st);
  return launch_async_lp<T, D, RB, NW, NST, false>(a, grid, st);
}

#include "attn_pipe.h"
#include "attn_decode.h"

template <typename T>
int attn_dispatch(const AttnArgs& a, dim3 grid, hipStream_t st) {
  const int D = a.p.D;
  if (a.use_fast) return D == 64 ? launch_pipe<T, 64>(a, grid, st) : launch_pipe<T, 128>(a, grid, st);
  if (a.use_async) {
    if (a.nw == 8) {
      switch (D) {
        case 64: return a.nst == 3 ? launch_async<T, 64, 128, 8, 3>(a, grid, st) : launch_async<T, 64, 128, 8, 2>(a, grid, st);
        case 96: return a.nst == 3 ? launch_async<T, 96, 256, 8, 3>(a, grid, st) : launch_async<T, 96, 256, 8, 2>(a, grid, st);
        case 128: return a.nst == 3 ? launch_async<T, 128, 256, 8, 3>(a, grid, st) : launch_async<T, 128, 256, 8, 2>(a, grid, st);
        default: break;
      }
    } else {
      switch (D) {
        // head dims that are a multiple of 16 but fill their LDS rows only partly: the padding chunks are loaded
        // with finite data and the output columns computed from them are never stored
        case 32: return launch_async<T, 32, 128, 4, 2>(a, grid, st);
        case 48: return launch_async<T, 48, 128, 4, 2>(a, grid, st);
        case 80: return launch_async<T, 80, 256, 4, 2>(a, grid, st);
        case 112: return launch_async<T, 112, 256, 4, 2>(a, grid, st);
        case 64: return launch_async<T, 64, 128, 4, 2>(a, grid, st);
        case 96: return launch_async<T, 96, 256, 4, 2>(a, grid, st);
        case 128: return launch_async<T, 128, 256, 4, 2>(a, grid, st);
        case 192: return launch_async<T, 192, 512, 4, 2>(a, grid, st);
        case 256: return launch_async<T, 256, 512, 4, 2>(a, grid, st);
        default: break;
      }
    }
  }
  if (D <= 64) hipLaunchKernelGGL((attn_varlen_kernel<T, 64>), grid, dim3(256), 0, st, a);
  else if (D <= 128) hipLaunchKernelGGL((attn_varlen_kernel<T, 128>), grid, dim3(256), 0, st, a);
  else if (D <= 192) hipLaunchKernelGGL((attn_varlen_kernel<T, 192>), grid, dim3(256), 0, st, a);
  else hipLaunchKernelGGL((attn_varlen_kernel<T, 256>), grid, dim3(256), 0, st, a);
  return fg_check_launch("flash_attn_varlen_fwd");
}

}  // namespace

namespace {
int decode_num_cu() {
  int dev = 0, n = 0;
  if (hipGetDevice(&dev) != hipSuccess) dev = 0;
  if (hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || n <= 0) n = 256;
  return n;
}
// Decides whether the single-token kernel takes these parameters and, if so, how the key ranges are cut.
// Without a large enough workspace the ranges are not split beyond what the kernel itself requires.
// `mixed`: the batch may also hold sequences with more than one query token (they are skipped by the kernel).
bool decode_setup(const FgFlashParams& p, DecodeArgs* d, bool mixed = false) {
  if ((p.max_seqlen_q != 1 && !mixed) || !(p.D == 64 || p.D == 128) || p.alibi_slopes != nullptr || p.softcap > 0.f) return false;
  if (p.window_left >= 0 && p.window_left < p.max_seqlen_k) return false;
  if (p.Hk <= 0 || p.Hq % p.Hk != 0 || p.Hq / p.Hk > 32) return false;
  int shift = -1;
  for (int sft = 0; sft < 31; ++sft)
    if ((1 << sft) == p.page_size) shift = sft;
  if (shift < 4) return false;
  if (const char* force = fg_options().attn_kernel; force[0] != 0) {
    if (force[0] != 'd') return false;
  }
  int splits = 1, tps = 4;
  decode_plan(p, shift, decode_num_cu(), &splits, &tps);
  if (splits > 1 && (p.workspace == nullptr || (size_t)p.workspace_bytes < decode_workspace_bytes(p, splits) ||
                     !fg_aligned(p.workspace, 16))) {
    // unsplit, if one range can hold the longest sequence
    const int64_t tiles = fg_cdiv(p.max_seqlen_k > 0 ? p.max_seqlen_k : 1, kDecTile);
    if (tiles * kDecTile > 4096) return false;
    splits = 1;
    tps = (int)((tiles + 3) / 4 * 4);
  }
  d->p = p;
  d->scale_log2 = p.softmax_scale * 1.4426950408889634f;
  d->page_shift = shift;
  d->group = p.Hq / p.Hk;
  d->splits = splits;
  d->tiles_per_split = tps;
  d->min_tiles = 16;
  if (fg_options().decode_min_tiles > 0) d->min_tiles = fg_options().decode_min_tiles;
  d->part_o = splits > 1 ? (float*)p.workspace : nullptr;
  d->part_ml = splits > 1 ? (float*)p.workspace + (size_t)splits * p.batch * p.Hq * p.D : nullptr;
  return true;
}
// A batch of at least four sequences with max_seqlen_q > 1 is treated as mixed: the single-token kernel takes the
// sequences with one query token (it streams K/V 2-3 times faster than the prefill kernels do for one row, and
// splits long sequences), the prefill kernel skips them.  Both read the lengths on the device; a ragged batch without
// such sequences pays two launches of workgroups that leave at once (a uniform batch is recognised on the host).
bool mixed_batch(const FgFlashParams& p) {
  if (p.max_seqlen_q <= 1 || p.batch < 4) return false;
  if (fg_options().attn_mixed >= 0) return fg_options().attn_mixed != 0;
  // every sequence as long as the longest: none has a single query token
  if ((int64_t)p.total_q >= (int64_t)p.batch * p.max_seqlen_q) return false;
  return true;
}
}  // namespace

extern "C" size_t fg_flash_attn_workspace_bytes(const FgFlashParams* pp, int device) {
  if (pp == nullptr) return 0;
  FgFlashParams p = *pp;
  if (p.batch <= 0 || p.total_q <= 0) return 0;
  // ask as if an unlimited workspace were offered
  static char dummy_ws[16] __attribute__((aligned(16)));
  p.workspace = dummy_ws;
  p.workspace_bytes = INT64_MAX;
  (void)device;
  DecodeArgs d;
  if (decode_setup(p, &d, mixed_batch(p))) return decode_workspace_bytes(p, d.splits);
  return 0;
}

extern "C" int fg_flash_attn_varlen_fwd(const FgFlashParams* pp, void* stream) {
  FG_REQUIRE(pp != nullptr, FG_ERR_INVALID, "flash_attn_varlen_fwd: null params");
  const FgFlashParams& p = *pp;
  FG_REQUIRE(p.dtype == FG_F16 || p.dtype == FG_BF16, FG_ERR_INVALID,
             "flash_attn_varlen_fwd: only fp16 and bf16 are supported (dtype %d)", p.dtype);
  FG_REQUIRE(p.batch >= 0 && p.total_q >= 0, FG_ERR_INVALID, "flash_attn_varlen_fwd: negative size");
  if (p.batch == 0 || p.total_q == 0) return FG_OK;
  FG_REQUIRE(p.q && p.k_cache && p.v_cache && p.out && p.cu_seqlens_q && p.seqused_k && p.block_table, FG_ERR_INVALID,
             "flash_attn_varlen_fwd: null pointer (q, k, v, out, cu_seqlens_q, seqused_k and block_table are required)");
  FG_REQUIRE(p.D > 0 && p.D <= 256 && p.D % 8 == 0, FG_ERR_INVALID,
             "flash_attn_varlen_fwd: head dim %d must be a multiple of 8 and at most 256", p.D);
  FG_REQUIRE(p.Hq > 0 && p.Hk > 0 && p.Hq % p.Hk == 0, FG_ERR_INVALID,
             "flash_attn_varlen_fwd: %d query heads are not a multiple of %d kv heads", p.Hq, p.Hk);
  FG_REQUIRE(p.page_size > 0, FG_ERR_INVALID, "flash_attn_varlen_fwd: page size must be positive");
  FG_REQUIRE(p.max_seqlen_q > 0, FG_ERR_INVALID, "flash_attn_varlen_fwd: max_seqlen_q must be positive");
  auto al = [](const void* q, int64_t s1, int64_t s2) { return fg_aligned(q, 16) && s1 % 8 == 0 && s2 % 8 == 0; };
  FG_REQUIRE(al(p.q, p.q_row_stride, p.q_head_stride) && al(p.k_cache, p.k_row_stride, p.k_head_stride) &&
                 al(p.v_cache, p.v_row_stride, p.v_head_stride) && p.k_page_stride % 8 == 0 && p.v_page_stride % 8 == 0,
             FG_ERR_UNSUPPORTED, "flash_attn_varlen_fwd: q/k/v rows must be 16-byte aligned");
  FG_REQUIRE(fg_aligned(p.out, 8) && p.o_row_stride % 4 == 0 && p.o_head_stride % 4 == 0, FG_ERR_UNSUPPORTED,
             "flash_attn_varlen_fwd: out rows must be 8-byte aligned");
  FG_REQUIRE(p.batch < 65536 && p.Hq < 65536, FG_ERR_UNSUPPORTED, "flash_attn_varlen_fwd: batch/heads exceed the grid");

  hipStream_t st = (hipStream_t)stream;
  bool skip_single = false;
  {
    DecodeArgs d;
    const bool mixed = mixed_batch(p);
    if (decode_setup(p, &d, mixed)) {
      int rc;
      if (p.dtype == FG_F16) rc = p.D == 64 ? launch_decode<f16_t, 64>(d, st) : launch_decode<f16_t, 128>(d, st);
      else rc = p.D == 64 ? launch_decode<bf16_t, 64>(d, st) : launch_decode<bf16_t, 128>(d, st);
      if (!mixed || rc != FG_OK) return rc;
      skip_single = true;  // the prefill kernel below handles every other sequence
    }
  }
  AttnArgs a;
  a.p = p;
  a.skip_single = skip_single ? 1 : 0;
  const int ratio = p.Hq / p.Hk;
  a.hpb = ratio % 4 == 0 ? 4 : (ratio % 2 == 0 ? 2 : 1);
  a.page_shift = -1;
  for (int sft = 0; sft < 31; ++sft)
    if ((1 << sft) == p.page_size) a.page_shift = sft;
  // Kernel variant.  Head dims 32/48/64/80/96/112/128/192/256 take the asynchronous-tile kernel with 4 waves and
  // two LDS stages (measured fastest; the 8-wave variants stay selectable for head dims 64, 96 and 128);
  // everything else the register-staged kernel.
  // FG_ATTN_KERNEL = "fast" | "fn" | "sync" | "w4s2" | "w8s2" | "w8s3" overrides (debugging and measurement aid).
  a.use_async = (p.D == 32 || p.D == 48 || p.D == 64 || p.D == 80 || p.D == 96 || p.D == 112 || p.D == 128 || p.D == 192 ||
                 p.D == 256) ? 1 : 0;
  a.nw = 4;
  a.nst = 2;
  // The lean kernel needs the 16 key rows a wave moves per tile inside one page.
  // (and computes tile addresses with 32-bit byte strides)
  auto fits31 = [](int64_t elems) { return elems >= 0 && elems < ((int64_t)1 << 30); };
  a.use_fast = (p.D == 128 || p.D == 64) && a.page_shift >= 4 && p.alibi_slopes == nullptr && !(p.softcap > 0.f) &&
               fits31(p.k_page_stride) && fits31(p.v_page_stride) && fits31(p.k_row_stride * p.page_size) &&
               fits31(p.v_row_stride * p.page_size);
  a.xcd_remap = 1;
  if (const char* force = fg_options().attn_kernel; force[0] != 0) {
    a.use_fast = a.use_fast && force[0] == 'f';
    if (force[0] == 'f' && force[1] == 'n') a.xcd_remap = 0;  // "fn...": the lean kernel in plain grid order
    if (force[0] == 's') a.use_async = 0;
    if (force[0] == 'w' && (p.D == 64 || p.D == 96 || p.D == 128)) {
      a.nw = force[1] == '8' ? 8 : 4;
      a.nst = (force[2] == 's' && force[3] == '3' && a.nw == 8) ? 3 : 2;
    }
  }
  {
    // LDS copy of the block-table slice: sized for the longest sequence, capped at kPageTabMaxBytes
    const int64_t need = fg_cdiv(p.max_seqlen_k > 0 ? p.max_seqlen_k : 1, p.page_size) + 1;
    a.page_tab_entries = need * 4 <= kPageTabMaxBytes ? (int)((need + 3) / 4 * 4) : 0;
  }
  const int waves = a.use_async ? a.nw : 4;
  a.rows_per_block = waves * 32 / a.hpb;
  // Mask bounds (bottom-right aligned): keys col with col > row + shift + right or col < row + shift - left are
  // masked.  causal forces right = 0; a one-sided window leaves the other side open.
  int wl = p.window_left, wr = p.window_right;
  if (p.is_causal) wr = 0;
  a.has_right = wr >= 0;
  a.has_left = wl >= 0;
  a.right_off_w = wr >= 0 ? wr : 0;
  a.left_off_w = wl >= 0 ? wl : 0;
  const float log2e = 1.4426950408889634f;
  a.scale_log2 = p.softmax_scale * log2e;
  a.cap_in = p.softcap > 0.f ? p.softmax_scale / p.softcap : 0.f;
  a.cap_out_log2 = p.softcap * log2e;
  dim3 grid((unsigned)fg_cdiv(p.max_seqlen_q, a.rows_per_block), (unsigned)p.batch, (unsigned)(p.Hq / a.hpb));
  if (p.dtype == FG_F16) return attn_dispatch<f16_t>(a, grid, st);
  return attn_dispatch<bf16_t>(a, grid, st);
}
