// Tiled MFMA GEMM for gfx950: C[M,N] = alpha * A[M,K].B[K,N] + beta * bias, fp32 accumulate.
//
// Workgroup = 256 threads = 4 waves in a 2x2 grid over a BM x BN output tile; a wave owns a
// (BM/2) x (BN/2) sub-tile as TM x TN MFMA 32x32 accumulators (v_mfma_f32_32x32x16_{bf16,f16},
// v_mfma_f32_32x32x2_f32 for true-fp32 inputs).  The K loop advances 128 bytes of K per step
// (BK = 64 half-precision elements or 32 floats).
//
// LDS holds both operands "K-major": row r of the A tile (an output row) or of the B tile (an
// output column) is BK consecutive K elements = 128 bytes, at a pitch of 144 bytes.  The 16-byte
// pad makes the 16 rows touched by a quarter-wave of a ds_read_b128 fall into disjoint banks, and
// does the same for the transposing stores below.  Two such stages are double-buffered, so one
// barrier per K step suffices: while the MFMAs consume stage s, the global loads of stage s^1 are
// in flight in registers and are written to LDS just before the barrier.
//
// Global -> LDS goes through registers, in one of three per-operand modes:
//   LOAD_K   the operand is K-contiguous in memory (A row-major, or B = W.t()): 16-byte loads
//            along K, stored as they are.
//   LOAD_MN  the operand is contiguous along its M/N index (A column-major, B row-major): each
//            thread loads an 8(k) x 8(mn) block as eight 16-byte rows, transposes it in registers
//            with v_perm_b32 and stores eight 16-byte K-runs.  16-bit types only.
//   LOAD_KU / LOAD_MNU  the same two layouts without the alignment and divisibility conditions (a row stride or
//            K that is not a multiple of 8 elements, a base that is only element-aligned): the 16-byte loads are
//            declared element-aligned, and a group that straddles the end of K or of the rows is assembled
//            element by element, zeros past the end.  LOAD_MNU also exists for 32-bit elements (4 x 4 blocks).
//   LOAD_GEN any strides, any alignment, full bounds checks: element-wise.
// The vector modes never read out of bounds: row indices are clamped to the last valid row (the
// duplicate rows are never stored) and 16-byte groups that lie past K are replaced by zeros.
#pragma once
#include "fg_common.h"

namespace fgk {

enum { LOAD_K = 0, LOAD_MN = 1, LOAD_GEN = 2, LOAD_KU = 3, LOAD_MNU = 4 };

constexpr int kRowBytes = 128;   // K bytes per tile row per stage
constexpr int kPitch = 144;      // LDS pitch of a tile row
constexpr int kThreads = 256;
// Stream-K workspace layout shared by every kernel that uses it: a fixed table of ticket counters
// (indexed by the first workgroup that contributes to a split tile, so kMaxWorkers entries are
// enough), then the fp32 partial tiles.  Only tickets ever live in the table, and every kernel
// returns them to zero, so kernels with different partial-tile sizes can share one buffer.
constexpr int kMaxWorkers = 1024;
constexpr size_t kTicketOffset = 256;
constexpr size_t kPartialOffset = kTicketOffset + kMaxWorkers * sizeof(unsigned);

struct GemmArgs {
  const void* A;
  const void* B;
  const void* bias;
  void* C;
  int64_t M, N, K;
  int64_t sam, sak, sbk, sbn, sim, sin, scm, scn;
  float alpha, beta;
  int tiles_m, tiles_n;
  int tile_base;        // first tile id of a data-parallel launch (tiles below it belong to stream-K)
  int k_ragged;         // direct-to-LDS kernels, K not a multiple of 64: valid k of the last K step (a multiple of 8), else 0
  const void* zeros;    // ... and 4 KB of zeros in device memory, the source of that step's chunks past K
  // stream-K (unused by the data-parallel launch)
  float* partials;      // [workers][2][BM*BN] fp32
  unsigned* tickets;    // [kMaxWorkers], zero between launches
  int sk_tiles;         // tiles shared between workers
  int iters_per_tile;   // K steps per tile
  int sk_workers;       // persistent workgroups
  int64_t sk_per, sk_rem;  // K steps per worker, and how many workers take one more
};

template <typename T> struct Mfma;
template <> struct Mfma<bf16_t> {
  typedef bf16x8 Frag;
  static constexpr int KSTEP = 16, KPL = 8;
  static __device__ __forceinline__ f32x16 mma(Frag a, Frag b, f32x16 c) {
    return __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, c, 0, 0, 0);
  }
};
template <> struct Mfma<f16_t> {
  typedef f16x8 Frag;
  static constexpr int KSTEP = 16, KPL = 8;
  static __device__ __forceinline__ f32x16 mma(Frag a, Frag b, f32x16 c) {
    return __builtin_amdgcn_mfma_f32_32x32x16_f16(a, b, c, 0, 0, 0);
  }
};
template <> struct Mfma<float> {
  typedef float Frag;
  static constexpr int KSTEP = 2, KPL = 1;
  static __device__ __forceinline__ f32x16 mma(Frag a, Frag b, f32x16 c) {
    return __builtin_amdgcn_mfma_f32_32x32x2f32(a, b, c, 0, 0, 0);
  }
};

// ---------------------------------------------------------------------------------------------
// global -> register -> LDS staging of one operand tile (ROWS rows x 128 bytes of K)
// ---------------------------------------------------------------------------------------------
template <typename T, int ROWS, int MODE> struct Stager;

template <typename T, int ROWS> struct Stager<T, ROWS, LOAD_K> {
  static constexpr int EPC = 16 / sizeof(T);              // elements per 16-byte chunk
  static constexpr int N = (ROWS * 8 + kThreads - 1) / kThreads;  // chunks per thread
  u32x4 r[N];
  // element (row, k) lives at base[row * s_row + k]
  __device__ __forceinline__ void fetch(const T* base, int64_t s_row, int64_t /*s_k*/, int row0, int rows_total,
                                        int k0, int K, int tid) {
#pragma unroll
    for (int i = 0; i < N; ++i) {
      const int idx = i * kThreads + tid;
      const int row = idx >> 3, c = idx & 7;
      if (ROWS * 8 % kThreads != 0 && idx >= ROWS * 8) continue;
      int gr = row0 + row;
      gr = gr < rows_total ? gr : rows_total - 1;
      const int k = k0 + c * EPC;
      if (k < K) r[i] = *reinterpret_cast<const u32x4*>(base + (int64_t)gr * s_row + k);
      else r[i] = u32x4{0u, 0u, 0u, 0u};
    }
  }
  __device__ __forceinline__ void store(char* lds, int tid) {
#pragma unroll
    for (int i = 0; i < N; ++i) {
      const int idx = i * kThreads + tid;
      if (ROWS * 8 % kThreads != 0 && idx >= ROWS * 8) continue;
      *reinterpret_cast<u32x4*>(lds + (idx >> 3) * kPitch + (idx & 7) * 16) = r[i];
    }
  }
};

template <typename T, int ROWS> struct Stager<T, ROWS, LOAD_MN> {
  static_assert(sizeof(T) == 2, "the transposing stager handles 16-bit elements");
  static constexpr int N = (ROWS + kThreads - 1) / kThreads;  // 8x8 blocks per thread
  u32x4 r[N][8];
  // element (row, k) lives at base[k * s_k + row]
  __device__ __forceinline__ void fetch(const T* base, int64_t /*s_row*/, int64_t s_k, int row0, int rows_total,
                                        int k0, int K, int tid) {
#pragma unroll
    for (int i = 0; i < N; ++i) {
      const int blk = i * kThreads + tid;
      if (ROWS % kThreads != 0 && blk >= ROWS) continue;
      const int kb = blk & 7, rb = blk >> 3;
      int gr = row0 + rb * 8;
      gr = gr + 8 <= rows_total ? gr : rows_total - 8;
#pragma unroll
      for (int j = 0; j < 8; ++j) {
        const int k = k0 + kb * 8 + j;
        if (k < K) r[i][j] = *reinterpret_cast<const u32x4*>(base + (int64_t)k * s_k + gr);
        else r[i][j] = u32x4{0u, 0u, 0u, 0u};
      }
    }
  }
  __device__ __forceinline__ void store(char* lds, int tid) {
#pragma unroll
    for (int i = 0; i < N; ++i) {
      const int blk = i * kThreads + tid;
      if (ROWS % kThreads != 0 && blk >= ROWS) continue;
      const int kb = blk & 7, rb = blk >> 3;
#pragma unroll
      for (int rr = 0; rr < 8; ++rr) {
        // K-run of row rr: dword d = { k = 2d (low half), k = 2d + 1 (high half) }
        const unsigned sel = (rr & 1) ? 0x07060302u : 0x05040100u;
        u32x4 o;
#pragma unroll
        for (int d = 0; d < 4; ++d) o[d] = __builtin_amdgcn_perm(r[i][2 * d + 1][rr >> 1], r[i][2 * d][rr >> 1], sel);
        *reinterpret_cast<u32x4*>(lds + (rb * 8 + rr) * kPitch + kb * 16) = o;
      }
    }
  }
};

// 16 bytes from an address that is only aligned to the element type.
template <typename T> __device__ __forceinline__ u32x4 load16_elem_aligned(const T* p) {
  u32x4 v;
  __builtin_memcpy(&v, p, 16);
  return v;
}

template <typename T, int ROWS> struct Stager<T, ROWS, LOAD_KU> {
  static constexpr int EPC = 16 / sizeof(T);
  static constexpr int N = (ROWS * 8 + kThreads - 1) / kThreads;
  u32x4 r[N];
  // element (row, k) lives at base[row * s_row + k]
  __device__ __forceinline__ void fetch(const T* base, int64_t s_row, int64_t /*s_k*/, int row0, int rows_total,
                                        int k0, int K, int tid) {
#pragma unroll
    for (int i = 0; i < N; ++i) {
      const int idx = i * kThreads + tid;
      const int row = idx >> 3, c = idx & 7;
      if (ROWS * 8 % kThreads != 0 && idx >= ROWS * 8) continue;
      int gr = row0 + row;
      gr = gr < rows_total ? gr : rows_total - 1;
      const int k = k0 + c * EPC;
      const T* p = base + (int64_t)gr * s_row + k;
      if (k + EPC <= K) {
        r[i] = load16_elem_aligned(p);
      } else {
        T e[EPC];
#pragma unroll
        for (int j = 0; j < EPC; ++j) e[j] = (k + j < K) ? p[j] : (T)0.0f;
        u32x4 v;
        __builtin_memcpy(&v, e, 16);
        r[i] = v;
      }
    }
  }
  __device__ __forceinline__ void store(char* lds, int tid) {
#pragma unroll
    for (int i = 0; i < N; ++i) {
      const int idx = i * kThreads + tid;
      if (ROWS * 8 % kThreads != 0 && idx >= ROWS * 8) continue;
      *reinterpret_cast<u32x4*>(lds + (idx >> 3) * kPitch + (idx & 7) * 16) = r[i];
    }
  }
};

template <typename T, int ROWS> struct Stager<T, ROWS, LOAD_MNU> {
  static_assert(sizeof(T) == 2, "16-bit elements; the 32-bit specialization follows");
  static constexpr int N = (ROWS + kThreads - 1) / kThreads;  // 8x8 blocks per thread
  u32x4 r[N][8];
  // element (row, k) lives at base[k * s_k + row]
  __device__ __forceinline__ void fetch(const T* base, int64_t /*s_row*/, int64_t s_k, int row0, int rows_total,
                                        int k0, int K, int tid) {
#pragma unroll
    for (int i = 0; i < N; ++i) {
      const int blk = i * kThreads + tid;
      if (ROWS % kThreads != 0 && blk >= ROWS) continue;
      const int kb = blk & 7, rb = blk >> 3;
      const int gr = row0 + rb * 8;
#pragma unroll
      for (int j = 0; j < 8; ++j) {
        const int k = k0 + kb * 8 + j;
        const T* p = base + (int64_t)k * s_k + gr;
        if (k < K && gr + 8 <= rows_total) {
          r[i][j] = load16_elem_aligned(p);
        } else {
          T e[8];
#pragma unroll
          for (int rr = 0; rr < 8; ++rr) e[rr] = (k < K && gr + rr < rows_total) ? p[rr] : (T)0.0f;
          u32x4 v;
          __builtin_memcpy(&v, e, 16);
          r[i][j] = v;
        }
      }
    }
  }
  __device__ __forceinline__ void store(char* lds, int tid) {
#pragma unroll
    for (int i = 0; i < N; ++i) {
      const int blk = i * kThreads + tid;
      if (ROWS % kThreads != 0 && blk >= ROWS) continue;
      const int kb = blk & 7, rb = blk >> 3;
#pragma unroll
      for (int rr = 0; rr < 8; ++rr) {
        const unsigned sel = (rr & 1) ? 0x07060302u : 0x05040100u;
        u32x4 o;
#pragma unroll
        for (int d = 0; d < 4; ++d) o[d] = __builtin_amdgcn_perm(r[i][2 * d + 1][rr >> 1], r[i][2 * d][rr >> 1], sel);
        *reinterpret_cast<u32x4*>(lds + (rb * 8 + rr) * kPitch + kb * 16) = o;
      }
    }
  }
};

// 32-bit elements: a thread takes a 4(k) x 4(mn) block as four 16-byte rows; its transpose is a renaming of registers.
template <int ROWS> struct Stager<float, ROWS, LOAD_MNU> {
  static constexpr int N = (ROWS * 2 + kThreads - 1) / kThreads;  // blocks per thread: 8 k-chunks x ROWS/4 row groups
  u32x4 r[N][4];
  // element (row, k) lives at base[k * s_k + row]
  __device__ __forceinline__ void fetch(const float* base, int64_t /*s_row*/, int64_t s_k, int row0, int rows_total,
                                        int k0, int K, int tid) {
#pragma unroll
    for (int i = 0; i < N; ++i) {
      const int blk = i * kThreads + tid;
      if (ROWS * 2 % kThreads != 0 && blk >= ROWS * 2) continue;
      const int kb = blk & 7, rb = blk >> 3;
      const int gr = row0 + rb * 4;
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        const int k = k0 + kb * 4 + j;
        const float* p = base + (int64_t)k * s_k + gr;
        if (k < K && gr + 4 <= rows_total) {
          r[i][j] = load16_elem_aligned(p);
        } else {
          u32x4 v;
#pragma unroll
          for (int rr = 0; rr < 4; ++rr) v[rr] = (k < K && gr + rr < rows_total) ? __builtin_bit_cast(uint32_t, p[rr]) : 0u;
          r[i][j] = v;
        }
      }
    }
  }
  __device__ __forceinline__ void store(char* lds, int tid) {
#pragma unroll
    for (int i = 0; i < N; ++i) {
      const int blk = i * kThreads + tid;
      if (ROWS * 2 % kThreads != 0 && blk >= ROWS * 2) continue;
      const int kb = blk & 7, rb = blk >> 3;
#pragma unroll
      for (int rr = 0; rr < 4; ++rr)
        *reinterpret_cast<u32x4*>(lds + (rb * 4 + rr) * kPitch + kb * 16) =
            u32x4{r[i][0][rr], r[i][1][rr], r[i][2][rr], r[i][3][rr]};
    }
  }
};

template <typename T, int ROWS> struct Stager<T, ROWS, LOAD_GEN> {
  static constexpr int BK = kRowBytes / sizeof(T);
  static constexpr int N = ROWS * BK / kThreads;  // elements per thread
  T r[N];
  bool k_fast;
  __device__ __forceinline__ void fetch(const T* base, int64_t s_row, int64_t s_k, int row0, int rows_total, int k0,
                                        int K, int tid) {
    k_fast = (s_k == 1);
#pragma unroll
    for (int i = 0; i < N; ++i) {
      const int idx = i * kThreads + tid;
      const int row = k_fast ? idx / BK : idx % ROWS;
      const int k = k_fast ? idx % BK : idx / ROWS;
      const bool ok = (row0 + row < rows_total) && (k0 + k < K);
      r[i] = ok ? base[(int64_t)(row0 + row) * s_row + (int64_t)(k0 + k) * s_k] : (T)0.0f;
    }
  }
  __device__ __forceinline__ void store(char* lds, int tid) {
#pragma unroll
    for (int i = 0; i < N; ++i) {
      const int idx = i * kThreads + tid;
      const int row = k_fast ? idx / BK : idx % ROWS;
      const int k = k_fast ? idx % BK : idx / ROWS;
      *reinterpret_cast<T*>(lds + row * kPitch + k * (int)sizeof(T)) = r[i];
    }
  }
};

// ---------------------------------------------------------------------------------------------
// tile id -> (tile_m, tile_n), a bijection on [0, tiles_m * tiles_n).  Workgroups are dispatched
// round-robin over the 8 XCDs (XCD = id mod 8), each with its own L2 and 32 CUs, and in id order
// within an XCD.
//
// Regular grids (tiles_m a multiple of 8, tiles_n of 4): the grid is cut into sub-blocks of 8 x 4
// tiles, one per XCD and round, so the 32 tiles an XCD works on at any time share 8 A panels and
// 4 B panels in its L2.  The 8 sub-blocks of a round are neighbours, 2 x 4 of them = 16 x 16 tiles,
// and rounds walk strips of 16 tile rows back and forth: a round needs as few distinct rows of A
// and columns of B as 256 tiles can (the memory-side cache holds them while the 8 XCDs fetch
// them one after the other), and consecutive rounds share their A rows, or their B columns at the
// turn of a strip.  A last partial round deals its sub-blocks to the XCDs in equal contiguous parts.
//
// Other grids: ids congruent mod 8 are made consecutive, then walked in column-major groups of
// 8 tile rows.
// ---------------------------------------------------------------------------------------------
__host__ __device__ __forceinline__ void tile_coords(int id, int tiles_m, int tiles_n, int& tm, int& tn, int strip_rows = 2) {
  constexpr int XCDS = 8, SUB_M = 8, SUB_N = 4, PER = SUB_M * SUB_N;
  if (tiles_m % SUB_M == 0 && tiles_n % SUB_N == 0) {
    const int sm_count = tiles_m / SUB_M, sn_count = tiles_n / SUB_N, nsub = sm_count * sn_count;
    const int x = id % XCDS, turn = id / XCDS;
    const int full = nsub / XCDS;  // rounds in which every XCD has a sub-block of its own
    int q, s;
    if (turn < full * PER) {
      q = (turn / PER) * XCDS + x;
      s = turn % PER;
    } else {
      const int rem = nsub - full * XCDS;  // 1..7 sub-blocks, PER * rem / 8 turns per XCD
      const int u = x * (PER / XCDS * rem) + (turn - full * PER);
      q = full * XCDS + u / PER;
      s = u % PER;
    }
    const int strip = q / (strip_rows * sn_count);
    const int left = sm_count - strip_rows * strip;
    const int rows = left < strip_rows ? left : strip_rows;
    const int r = q - strip * strip_rows * sn_count;
    int sn = r / rows;
    if (strip & 1) sn = sn_count - 1 - sn;
    tm = (strip * strip_rows + r % rows) * SUB_M + s % SUB_M;
    tn = sn * SUB_N + s / SUB_M;
    return;
  }
  constexpr int GROUP_M = 8;
  const int total = tiles_m * tiles_n;
  const int per_xcd = total / XCDS;
  int t = id;
  if (id < per_xcd * XCDS) t = (id % XCDS) * per_xcd + id / XCDS;  // the ragged tail keeps its id
  const int group = GROUP_M * tiles_n;
  const int g = t / group;
  const int first_m = g * GROUP_M;
  const int gsz = (tiles_m - first_m) < GROUP_M ? (tiles_m - first_m) : GROUP_M;
  const int in_g = t - g * group;
  tm = first_m + in_g % gsz;
  tn = in_g / gsz;
}

template <typename T, int BM, int BN, int AMODE, int BMODE> struct TileCompute {
  static constexpr int BK = kRowBytes / sizeof(T);
  static constexpr int WTM = BM / 2, WTN = BN / 2;
  static constexpr int TM = WTM / 32, TN = WTN / 32;
  static constexpr int A_STAGE = BM * kPitch, B_STAGE = BN * kPitch;
  static constexpr int LDS_BYTES = 2 * (A_STAGE + B_STAGE);
  typedef typename Mfma<T>::Frag Frag;

  // acc += A[tile rows, k-range] . B[k-range, tile cols] for K steps [it0, it1)
  static __device__ __forceinline__ void run(const GemmArgs& g, char* lds, int tm, int tn, int it0, int it1,
                                             f32x16 (&acc)[TM][TN]) {
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int wm = wave >> 1, wn = wave & 1;
    const T* A = (const T*)g.A;
    const T* B = (const T*)g.B;
    const int M = (int)g.M, N = (int)g.N, K = (int)g.K;
    char* As = lds;
    char* Bs = lds + 2 * A_STAGE;
    Stager<T, BM, AMODE> sa;
    Stager<T, BN, BMODE> sb;
    const int row0 = tm * BM, col0 = tn * BN;

    sa.fetch(A, g.sam, g.sak, row0, M, it0 * BK, K, tid);
    sb.fetch(B, g.sbn, g.sbk, col0, N, it0 * BK, K, tid);
    sa.store(As, tid);
    sb.store(Bs, tid);
    __syncthreads();

    const int frag_row = lane & 31;
    const int frag_k = (lane >> 5) * Mfma<T>::KPL * (int)sizeof(T);
    for (int it = it0; it < it1; ++it) {
      const int cur = (it - it0) & 1;
      const bool more = it + 1 < it1;
      if (more) {
        sa.fetch(A, g.sam, g.sak, row0, M, (it + 1) * BK, K, tid);
        sb.fetch(B, g.sbn, g.sbk, col0, N, (it + 1) * BK, K, tid);
      }
      const char* a_base = As + cur * A_STAGE + (wm * WTM + frag_row) * kPitch + frag_k;
      const char* b_base = Bs + cur * B_STAGE + (wn * WTN + frag_row) * kPitch + frag_k;
      // Fragments are double-buffered in registers and the scheduler is asked (iglp_opt) to
      // interleave the LDS reads of step ks+1 with the MFMAs of step ks; left alone it would sink
      // every read next to its first use and expose the LDS latency four times per K step.
      constexpr int KSTEPS = BK / Mfma<T>::KSTEP;
      if constexpr (sizeof(T) == 2) __builtin_amdgcn_iglp_opt(1);
      Frag fa[2][TM], fb[2][TN];
#pragma unroll
      for (int i = 0; i < TM; ++i) fa[0][i] = *reinterpret_cast<const Frag*>(a_base + i * 32 * kPitch);
#pragma unroll
      for (int j = 0; j < TN; ++j) fb[0][j] = *reinterpret_cast<const Frag*>(b_base + j * 32 * kPitch);
#pragma unroll
      for (int ks = 0; ks < KSTEPS; ++ks) {
        const int cb = ks & 1, nb = cb ^ 1;
        if (ks + 1 < KSTEPS) {
          const int koff = (ks + 1) * Mfma<T>::KSTEP * (int)sizeof(T);
#pragma unroll
          for (int i = 0; i < TM; ++i) fa[nb][i] = *reinterpret_cast<const Frag*>(a_base + i * 32 * kPitch + koff);
#pragma unroll
          for (int j = 0; j < TN; ++j) fb[nb][j] = *reinterpret_cast<const Frag*>(b_base + j * 32 * kPitch + koff);
        }
#pragma unroll
        for (int i = 0; i < TM; ++i)
#pragma unroll
          for (int j = 0; j < TN; ++j) acc[i][j] = Mfma<T>::mma(fa[cb][i], fb[cb][j], acc[i][j]);
      }
      if (more) {
        sa.store(As + (cur ^ 1) * A_STAGE, tid);
        sb.store(Bs + (cur ^ 1) * B_STAGE, tid);
      }
      __syncthreads();
    }
  }

  // Accumulator element e of sub-tile (i, j) of this lane sits at
  //   row = i*32 + (e/4)*8 + (lane/32)*4 + e%4,  col = j*32 + lane%32   (within the wave tile).
  template <typename F>
  static __device__ __forceinline__ void for_each_acc(f32x16 (&acc)[TM][TN], F f) {
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int wm = wave >> 1, wn = wave & 1;
#pragma unroll
    for (int i = 0; i < TM; ++i)
#pragma unroll
      for (int j = 0; j < TN; ++j)
#pragma unroll
        for (int e = 0; e < 16; ++e) {
          const int r = wm * WTM + i * 32 + (e >> 2) * 8 + (lane >> 5) * 4 + (e & 3);
          const int c = wn * WTN + j * 32 + (lane & 31);
          f(r, c, acc[i][j][e]);
        }
  }

  static __device__ __forceinline__ void epilogue(const GemmArgs& g, int tm, int tn, f32x16 (&acc)[TM][TN]) {
    T* C = (T*)g.C;
    const T* bias = (const T*)g.bias;
    const int row0 = tm * BM, col0 = tn * BN;
    const float alpha = g.alpha, beta = g.beta;
    const bool scale = alpha != 1.0f;
    for_each_acc(acc, [&](int r, int c, float v) {
      const int64_t m = row0 + r, n = col0 + c;
      if (m < g.M && n < g.N) {
        if (bias != nullptr) v = v * alpha + (float)bias[m * g.sim + n * g.sin] * beta;
        else if (scale) v = v * alpha;
        C[m * g.scm + n * g.scn] = (T)v;
      }
    });
  }
};

template <typename T, int BM, int BN, int AMODE, int BMODE>
__global__ __launch_bounds__(kThreads) void gemm_dp_kernel(GemmArgs g) {
  typedef TileCompute<T, BM, BN, AMODE, BMODE> TC;
  extern __shared__ __attribute__((aligned(16))) char lds[];
  int tm, tn;
  tile_coords(blockIdx.x + g.tile_base, g.tiles_m, g.tiles_n, tm, tn);
  f32x16 acc[TC::TM][TC::TN];
#pragma unroll
  for (int i = 0; i < TC::TM; ++i)
#pragma unroll
    for (int j = 0; j < TC::TN; ++j)
#pragma unroll
      for (int e = 0; e < 16; ++e) acc[i][j][e] = 0.f;
  TC::run(g, lds, tm, tn, 0, g.iters_per_tile, acc);
  TC::epilogue(g, tm, tn, acc);
}

// ---------------------------------------------------------------------------------------------
// stream-K over the same tile: `sk_workers` persistent workgroups share the K steps of tiles
// [0, sk_tiles) in equal contiguous ranges (tile-major).  A range is walked segment by segment
// (the part inside one tile).  Segments that span a tile's whole K are finished directly.  A tile
// split across workgroups is finished by the contributor that arrives last: each writes its fp32
// partial tile to its own workspace slot with device-coherent stores and draws a ticket from the
// tile's counter (device-scope atomic add); the holder of the last ticket adds all slots in
// workgroup order (bit-reproducible whoever finishes), runs the epilogue and resets the counter.
// No workgroup ever waits for another.
// ---------------------------------------------------------------------------------------------
__device__ __host__ __forceinline__ int64_t sk_begin(int64_t per, int64_t rem, int64_t w) {
  return w * per + (w < rem ? w : rem);
}
__device__ __forceinline__ int sk_worker_of(int64_t per, int64_t rem, int64_t u) {
  const int64_t big = rem * (per + 1);
  return (int)(u < big ? u / (per + 1) : rem + (u - big) / per);
}

template <typename T, int BM, int BN, int AMODE, int BMODE>
__global__ __launch_bounds__(kThreads) void gemm_streamk_kernel(GemmArgs g) {
  typedef TileCompute<T, BM, BN, AMODE, BMODE> TC;
  extern __shared__ __attribute__((aligned(16))) char lds[];
  __shared__ unsigned ticket_s;
  const int w = blockIdx.x, tid = threadIdx.x;
  const int64_t u_begin = sk_begin(g.sk_per, g.sk_rem, w);
  const int64_t u_end = sk_begin(g.sk_per, g.sk_rem, w + 1);
  int64_t u = u_begin;
  while (u < u_end) {
    const int tile = (int)(u / g.iters_per_tile);
    const int64_t tile_begin = (int64_t)tile * g.iters_per_tile;
    const int64_t tile_end = tile_begin + g.iters_per_tile;
    const int it0 = (int)(u - tile_begin);
    const int it1 = (int)((u_end < tile_end ? u_end : tile_end) - tile_begin);
    int tm, tn;
    tile_coords(tile, g.tiles_m, g.tiles_n, tm, tn);
    f32x16 acc[TC::TM][TC::TN];
#pragma unroll
    for (int i = 0; i < TC::TM; ++i)
#pragma unroll
      for (int j = 0; j < TC::TN; ++j)
#pragma unroll
        for (int e = 0; e < 16; ++e) acc[i][j][e] = 0.f;
    TC::run(g, lds, tm, tn, it0, it1, acc);
    bool finish = (it0 == 0 && it1 == g.iters_per_tile);
    if (!finish) {
      // slot 0 of a workgroup: the tile it starts in; slot 1: a tile it enters from the left
      float* slot = g.partials + ((int64_t)w * 2 + (u_begin < tile_begin ? 1 : 0)) * (BM * BN);
#pragma unroll
      for (int i = 0; i < TC::TM; ++i)
#pragma unroll
        for (int j = 0; j < TC::TN; ++j)
#pragma unroll
          for (int e = 0; e < 16; ++e)
            __hip_atomic_store(slot + ((i * TC::TN + j) * 16 + e) * kThreads + tid, acc[i][j][e], __ATOMIC_RELAXED,
                               __HIP_MEMORY_SCOPE_AGENT);
      // device-coherent stores need no cache write-back to be visible; waiting for their completion
      // before the ticket is enough, and far cheaper than flushing L2
      __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup");
      fg_wait_vmem_done();
      __syncthreads();  // every thread's slice of the partial tile is out
      const int w_first = sk_worker_of(g.sk_per, g.sk_rem, tile_begin);
      const int w_last = sk_worker_of(g.sk_per, g.sk_rem, tile_end - 1);
      if (tid == 0)
        ticket_s = __hip_atomic_fetch_add(g.tickets + w_first, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      __syncthreads();
      if (ticket_s == (unsigned)(w_last - w_first)) {
        finish = true;  // the loads below are device-coherent: they bypass the non-coherent caches
#pragma unroll
        for (int i = 0; i < TC::TM; ++i)
#pragma unroll
          for (int j = 0; j < TC::TN; ++j)
#pragma unroll
            for (int e = 0; e < 16; ++e) acc[i][j][e] = 0.f;
        for (int w2 = w_first; w2 <= w_last; ++w2) {
          const float* src =
              g.partials + ((int64_t)w2 * 2 + (sk_begin(g.sk_per, g.sk_rem, w2) < tile_begin ? 1 : 0)) * (BM * BN);
#pragma unroll
          for (int i = 0; i < TC::TM; ++i)
#pragma unroll
            for (int j = 0; j < TC::TN; ++j)
#pragma unroll
              for (int e = 0; e < 16; ++e)
                acc[i][j][e] += __hip_atomic_load(src + ((i * TC::TN + j) * 16 + e) * kThreads + tid, __ATOMIC_RELAXED,
                                                  __HIP_MEMORY_SCOPE_AGENT);
        }
        if (tid == 0) __hip_atomic_store(g.tickets + w_first, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      }
    }
    if (finish) TC::epilogue(g, tm, tn, acc);
    u = tile_begin + it1;
  }
}

}  // namespace fgk
