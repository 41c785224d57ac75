// Direct-to-LDS MFMA GEMM for gfx950, 16-bit inputs: C[M,N] = alpha * A[M,K].B[K,N] + beta * bias.
//
// The kernel for aligned 16-bit problems.  A BM x BN output tile per workgroup (256x256, 256x128 or
// 128x128, chosen on the host by how well the tile count fills the machine), 4 waves in a 2x2 grid,
// each wave a (BM/2) x (BN/2) sub-tile held as MFMA 16x16 accumulators (256 accumulator registers per
// lane for the largest tile).  The description below uses the 256x256 numbers.
//
// Data movement.  Each K step covers 64 elements = one full 128-byte cache line per tile row.  The
// operand tiles go from global memory straight into LDS with global_load_lds_dwordx4: no staging
// registers, no LDS store instructions.  One such instruction writes 64 lanes x 16 bytes to 1 KB of
// consecutive LDS, but every lane chooses its own global address, so the 16-byte chunks are laid
// out swizzled: what the fragment reads below need to be free of bank conflicts without any row
// padding.  LDS holds two stages (2 x 64 KB).
//
//   A (K contiguous), and B when it is K contiguous (B = W^T, "NT"):
//     stage layout [row][128 B]; chunk c of row r sits at position c ^ ((r >> 1) & 7).  A fragment
//     (16 rows x 32 k: 8 consecutive k of one row per lane) is one ds_read_b128; the 16 rows a
//     quarter-wave reads fall into 16 different 16-byte bank groups.
//   B when it is N contiguous (row-major [K,N], "NN"):
//     stage layout [k][512 B] (the 256 columns of the tile); chunk c of row k sits at position
//     c ^ (((k & 3) << 2) | (((k >> 3) & 1) << 1)).  The fragment is produced by two
//     ds_read_b64_tr_b16, which transpose 4 k-rows x 4 column groups among 16 lanes while reading.
//
// Schedule.  The matrix instruction is v_mfma_f32_16x16x32: a wave's 128 x 128 tile is 8 x 8 sub-tiles and
// a K step two k halves of 64 MFMAs.  The K step is cut into four quarters of 32 MFMAs, (k half, half of
// the A sub-tiles): a quarter issues its MFMAs while the fragments of the next quarter are read (4 A
// fragments, and the 8 B fragments of the next k half behind every second quarter), at most one LDS read
// or DMA per MFMA.  Quarter 3 already reads the first fragments of the next stage, so the MFMA pipe does
// not drain at a stage boundary.  One barrier per K step, after quarter 2: by then this wave has issued
// and completed every read of the current stage (the stage may be refilled) and every DMA it issued
// for the next stage has landed (vmcnt(0)).  The refill for stage kb+2 is issued right behind that
// barrier, spread over quarter 3 and quarter 0 of the next step, which leaves it two to three quarters
// to land.  The compiler's own scheduling is pinned with sched_barrier
// after every MFMA group; it keeps no counters for the DMA writes, hence the explicit waits.
//
// The MFMA operands are swapped (B fragment first), so a lane's accumulator registers hold 4
// consecutive output columns of one output row; after packing to 16 bits, v_permlane16_swap between
// two neighbouring sub-tiles gives every lane 8 consecutive columns and the tile is written with
// 16-byte stores.
//
// Preconditions (checked on the host): 16-bit type; A K-contiguous; B K- or N-contiguous; K a
// multiple of 64 (a multiple of 8 above 64 for the data-parallel 256x256 and 128x128 kernels, which then copy the
// missing chunks of the last K step from a buffer of zeros); N a multiple of 8; operand base pointers and row strides multiples of 16 bytes;
// C with unit column stride and 16-byte aligned rows; a bias with unit column stride and 8-byte
// aligned rows.  M and N are otherwise arbitrary: tile rows past the edge are clamped to the last
// valid row (or 8-column chunk) on load and never stored.  Everything else runs on the
// register-staged kernel.
#pragma once
#include "gemm_tile.h"

namespace fgk {

constexpr int kDmaRowB = 128;   // bytes of K per stage per A row
constexpr int kDmaBK = 64;
// Quarter steps of a K step that issue copies: 2 (quarter 3 and quarter 0, half of the copies each), or 3 (quarters
// 3, 0 and 1).  3 on the 256x256 tile with two stages was measured 2-6 % faster on large products (same instruction
// stream as built here, apart from register names) with the products checked, and its schedule holds for every K
// length in the host model of this loop (tests/test_gemm_schedule_model.py), but it has not been through the parity
// suite: the value comes from FG_V_DMA_COPY_RUNS (variants.h, default 2).  kDmaCopyRunsEveryTile extends 3 to
// every tile and to the stream-K kernel: never measured, off.
constexpr int kDmaCopyRuns = FG_V_DMA_COPY_RUNS;
constexpr bool kDmaCopyRunsEveryTile = false;
// with three quarters: the copies of a step issued in quarter 3 and in quarter 0 (the rest go to quarter 1), by the
// number of copies per wave and step
constexpr int dma_split_q3(int ndma, bool b_kc) { return ndma == 16 ? (b_kc ? 6 : 8) : ndma == 14 ? 5 : ndma == 12 ? 4 : 3; }
constexpr int dma_split_q0(int ndma) { return ndma == 16 ? 5 : ndma == 14 ? 5 : ndma == 12 ? 4 : 3; }
constexpr int dma_lds_bytes(int bm, int bn, int stages = 2) { return stages * (bm + bn) * kDmaRowB; }  // stages of (A tile + B tile)
constexpr int cmin(int a, int b) { return a < b ? a : b; }
constexpr int cmax(int a, int b) { return a > b ? a : b; }

#define FGK_LDSP(p) ((__attribute__((address_space(3))) void*)(p))
#define FGK_GLBP(p) ((const __attribute__((address_space(1))) void*)(p))
#define FGK_WAIT_VM(N) __builtin_amdgcn_s_waitcnt(((N) & 0xF) | (7 << 4) | (0xF << 8) | (((N) >> 4) << 14))
#define FGK_WAIT_LGKM0() __builtin_amdgcn_s_waitcnt(0xC07F) /* vmcnt 63, expcnt 7, lgkmcnt 0 */

template <int I> struct IntC { static constexpr int value = I; };
template <int B, int E, typename F> __device__ __forceinline__ void static_for(F&& f) {
  if constexpr (B < E) {
    f(IntC<B>{});
    static_for<B + 1, E>(f);
  }
}

template <int OFF> __device__ __forceinline__ u32x2 lds_read_tr16_b64(uint32_t addr) {
  u32x2 v;
  asm volatile("ds_read_b64_tr_b16 %0, %1 offset:%2" : "=v"(v) : "v"(addr), "i"(OFF));
  return v;
}
// Waits for every outstanding LDS read; tied to the registers the inline-asm reads wrote so that
// nothing consuming them can be placed ahead of the wait.
template <int N> __device__ __forceinline__ void lds_wait_tied(u32x4 (&r)[N]) {
  static_assert(N == 2 || N == 3 || N == 4 || N == 8, "fragments per set");
  if constexpr (N == 2) asm volatile("s_waitcnt lgkmcnt(0)" : "+v"(r[0]), "+v"(r[1]));
  if constexpr (N == 3) asm volatile("s_waitcnt lgkmcnt(0)" : "+v"(r[0]), "+v"(r[1]), "+v"(r[2]));
  if constexpr (N >= 4) asm volatile("s_waitcnt lgkmcnt(0)" : "+v"(r[0]), "+v"(r[1]), "+v"(r[2]), "+v"(r[3]));
  if constexpr (N == 8) asm volatile("" : "+v"(r[4]), "+v"(r[5]), "+v"(r[6]), "+v"(r[7]));
}
// rows of 16 lanes: X.row1 <-> Y.row0 and X.row3 <-> Y.row2, for two register pairs at once
__device__ __forceinline__ void swap_rows16x2(unsigned& x0, unsigned& y0, unsigned& x1, unsigned& y1) {
  asm volatile("s_nop 1\n\tv_permlane16_swap_b32 %0, %1\n\tv_permlane16_swap_b32 %2, %3\n\ts_nop 1"
               : "+v"(x0), "+v"(y0), "+v"(x1), "+v"(y1));
}

// The matrix instruction of these kernels: 16x16 outputs over 32 k.  Under the part's power limit it sustains
// ~14 % more than the 32x32x16 shape on the same data (2.0 against 1.78 PFLOP/s in a loop of nothing else): it
// touches its accumulators half as often per flop.
// The instruction is written as asm with the accumulator tied to itself in the AGPR file: a wave's 64 accumulator
// tiles fill that file exactly, and left to the register allocator some of them travel between the two files
// inside the loop (a v_accvgpr_read waits for the matrix pipe to drain: ~100 cycles each).  The compiler does not
// see a matrix instruction here, so the code that reads accumulators afterwards waits for the pipe itself
// (mfma_drain).
template <typename T> struct MfmaK32;
template <> struct MfmaK32<bf16_t> {
  typedef bf16x8 Frag;
  static __device__ __forceinline__ void mma(Frag a, Frag b, f32x4& c) {
    asm volatile("v_mfma_f32_16x16x32_bf16 %0, %1, %2, %0" : "+a"(c) : "v"(a), "v"(b));
  }
};
template <> struct MfmaK32<f16_t> {
  typedef f16x8 Frag;
  static __device__ __forceinline__ void mma(Frag a, Frag b, f32x4& c) {
    asm volatile("v_mfma_f32_16x16x32_f16 %0, %1, %2, %0" : "+a"(c) : "v"(a), "v"(b));
  }
};
// Waits out the matrix pipe, then passes every accumulator through an empty asm: volatile asm statements keep
// their order, so no read of an accumulator can be scheduled ahead of the wait.
template <int TM, int TN> __device__ __forceinline__ void mfma_drain(f32x4 (&acc)[TM][TN]) {
  asm volatile("s_nop 15\n\ts_nop 15" ::: "memory");
#pragma unroll
  for (int i = 0; i < TM; ++i)
#pragma unroll
    for (int j = 0; j < TN; ++j) asm volatile("" : "+a"(acc[i][j]));
}

// Epilogue of one tile (the host guarantees: C rows 16-byte aligned with unit column stride, N a multiple
// of 8, bias -- if any -- with unit column stride and 8-byte aligned rows).  acc is in the layout the
// main loop leaves: operands swapped, so lane (r = lane % 16, g = lane / 16) of sub-tile (i, j) owns output
// row 16 i + r and the 4 consecutive columns 16 j + 4 g ...
template <typename T, int BM, int BN>
__device__ __forceinline__ void dma_tile_epilogue(const GemmArgs& g, int tm, int tn, f32x4 (&acc)[BM / 32][BN / 32]) {
  constexpr int WTM = BM / 2, WTN = BN / 2, TM = WTM / 16, TN = WTN / 16;
  static_assert(TN % 2 == 0, "sub-tiles are stored in pairs");
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int wm = wave >> 1, wn = wave & 1;
  const int row0 = tm * BM, col0 = tn * BN;
  const int M = (int)g.M, N = (int)g.N;
  T* C = (T*)g.C;
  const T* bias = (const T*)g.bias;
  const float alpha = g.alpha, beta = g.beta;
  const bool scale = alpha != 1.0f;
  const int lr = lane & 15, lg = lane >> 4;
  // a bias row broadcast over M (the addmm of a linear layer) is the same for every output row: fetched once per
  // lane and sub-tile column instead of once per output element group
  typedef T T4 __attribute__((ext_vector_type(4)));
  const bool bcast = bias != nullptr && g.sim == 0;
  T4 brow[TN];
#pragma unroll
  for (int j = 0; j < TN; ++j) {
    const int c = col0 + wn * WTN + j * 16 + lg * 4;
    brow[j] = T4{(T)0.f, (T)0.f, (T)0.f, (T)0.f};
    if (bcast && c < N) brow[j] = *reinterpret_cast<const T4*>(bias + c);
  }
#pragma unroll
  for (int i = 0; i < TM; ++i) {
    const int64_t r = row0 + wm * WTM + i * 16 + lr;
#pragma unroll
    for (int jp = 0; jp < TN / 2; ++jp) {
      unsigned pk[2][2];
#pragma unroll
      for (int jj = 0; jj < 2; ++jj) {
        const int j = 2 * jp + jj;
        const int c = col0 + wn * WTN + j * 16 + lg * 4;
        float v[4];
#pragma unroll
        for (int e = 0; e < 4; ++e) v[e] = acc[i][j][e];
#if FG_V_ADDMM_BCAST_BRANCH
        if (bcast) {
          // (variant, variants.h: a branch of its own: merged with the per-element case below, the wait for that
          // case's load lands behind the join and this case, which loads nothing, waits there for every store still
          // in flight)
          const T4 t = brow[j];
#pragma unroll
          for (int e = 0; e < 4; ++e) v[e] = v[e] * alpha + (float)t[e] * beta;
        } else if (bias != nullptr) {
          T4 t = T4{(T)0.f, (T)0.f, (T)0.f, (T)0.f};
          if (r < M && c < N) t = *reinterpret_cast<const T4*>(bias + r * g.sim + c);
#pragma unroll
          for (int e = 0; e < 4; ++e) v[e] = v[e] * alpha + (float)t[e] * beta;
        } else if (scale) {
#else
        if (bias != nullptr) {
          T4 t = brow[j];
          if (!bcast && r < M && c < N) t = *reinterpret_cast<const T4*>(bias + r * g.sim + c);
#pragma unroll
          for (int e = 0; e < 4; ++e) v[e] = v[e] * alpha + (float)t[e] * beta;
        } else if (scale) {
#endif
#pragma unroll
          for (int e = 0; e < 4; ++e) v[e] *= alpha;
        }
#pragma unroll
        for (int d = 0; d < 2; ++d) {
          typedef T T2 __attribute__((ext_vector_type(2)));
          const T2 t = {(T)v[2 * d], (T)v[2 * d + 1]};
          pk[jj][d] = __builtin_bit_cast(unsigned, t);
        }
      }
      // sub-tiles 2jp (X) and 2jp+1 (Y): after X.odd rows <-> Y.even rows of 16 lanes, an even lane group g owns
      // columns 4g .. 4g+7 of sub-tile 2jp and an odd one columns 4(g-1) .. 4(g-1)+7 of sub-tile 2jp+1
      unsigned x0 = pk[0][0], x1 = pk[0][1], y0 = pk[1][0], y1 = pk[1][1];
      swap_rows16x2(x0, y0, x1, y1);
      const int c = col0 + wn * WTN + (2 * jp + (lg & 1)) * 16 + (lg & 2) * 4;
      if (r < M && c < N) *reinterpret_cast<u32x4*>(C + r * g.scm + c) = u32x4{x0, x1, y0, y1};
      // (keeps the scheduler from fetching every accumulator up front: 256 registers at once spill)
      __builtin_amdgcn_sched_barrier(0);
    }
  }
}

// Main loop over the K steps [kb0, kb0 + nk) of tile (tm, tn); `finish` receives the accumulators.
// NS = number of LDS stages: K step kb lives in stage kb % NS and is requested NS - 1 steps ahead.
// RAGGED: K is a multiple of 8 but not of 64; nk counts the partial last K step, whose 16-byte chunks past K are
// copied from a buffer of zeros instead (both operands, so whatever follows the rows in memory never enters a sum).
template <typename T, bool B_KC, int BM, int BN, int NS, bool RAGGED = false, typename F>
__device__ __forceinline__ void dma_tile_mainloop(const GemmArgs& g, char* lds, int tm, int tn, int kb0, int nk, F&& finish) {
  static_assert(sizeof(T) == 2, "16-bit element types");
  typedef typename MfmaK32<T>::Frag Frag;
  constexpr int WTM = BM / 2, WTN = BN / 2;        // wave tile
  constexpr int TM = WTM / 16, TN = WTN / 16;      // 16x16 sub-tiles per wave
  constexpr int HM = TM / 2;                       // A sub-tiles of one quarter step
  constexpr int A_OPB = BM * kDmaRowB;             // A tile, one stage
  constexpr int B_OPB = BN * kDmaRowB;             // B tile, one stage (64 k-rows of BN*2 bytes when N-contiguous)
  constexpr int STAGEB = A_OPB + B_OPB;
  constexpr int NA = BM / 32, NB = BN / 32;        // DMA instructions per wave, operand and stage
  constexpr int NDMA = NA + NB;
  // The copies of one K step, by the quarter step that issues them: C3 in quarter 3 of the step NS steps earlier
  // (whose stage has just been read for the last time), C0 and C1 in quarters 0 and 1 of the step after that one.
  // The barrier of a K step puts the four waves back in step, so they reach these quarters together, and a copy
  // holds the CU's address path for 16 cycles: the more quarters share the copies, the less the waves queue.
  constexpr bool THREE_RUNS = kDmaCopyRuns == 3 && !RAGGED && (kDmaCopyRunsEveryTile || (BM == 256 && BN == 256 && NS == 2));
  constexpr int C3 = THREE_RUNS ? dma_split_q3(NDMA, B_KC) : NDMA / 2;
  constexpr int C0 = THREE_RUNS ? dma_split_q0(NDMA) : NDMA - C3;
  constexpr int C1 = NDMA - C3 - C0;
  constexpr int HALF = C3;
  static_assert(C0 > 0 && C1 >= 0, "copy split");
  constexpr int NMF = HM * TN;                     // MFMAs per quarter step
  constexpr int RBB = BN * 2;                      // N-contiguous B: bytes per k-row of the tile
  constexpr int CPRB = RBB / 16, RPI = 1024 / RBB; // ... chunks per k-row, k-rows per DMA instruction
  static_assert(TM % 2 == 0 && TN <= 8 && TN >= 2, "wave tile");
  static_assert(NS >= 2 && NS <= 4 && NDMA * (NS - 1) + HALF <= 63, "outstanding DMAs must fit the vmcnt counter");
  auto stage_off = [](int kb) { return (NS == 2 ? (kb & 1) : NS == 4 ? (kb & 3) : kb % NS) * STAGEB; };
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int wm = wave >> 1, wn = wave & 1;
  const int row0 = tm * BM, col0 = tn * BN;
  const int M = (int)g.M, N = (int)g.N;
  const int64_t b_step = B_KC ? (int64_t)kDmaRowB : g.sbk * (int64_t)(kDmaBK * 2);  // bytes per K step

  // ---- DMA source addresses: a scalar base per operand and K step plus a 32-bit byte offset per lane and
  // instruction, so that the loop spends no vector instruction on addresses.  Wave w issues NA (NB) instructions
  // per stage for A (B); instruction j lands at operand base + (w*NA + j) * 1024, split into a part that goes
  // through M0 ((j/4)*4096) and an instruction immediate ((j%4)*1024).  The hardware adds the immediate to the
  // global address as well, so it is taken out of the lane offset; the scalar bases sit 3072 bytes low to keep
  // every lane offset non-negative.  (The host admits only operands whose tile-local offsets fit 32 bits.)
  uint32_t a_off[NA], b_off[NB];
#pragma unroll
  for (int j = 0; j < NA; ++j) {
    const int r = (wave * NA + j) * 8 + (lane >> 3);
    const int c = (lane & 7) ^ ((r >> 1) & 7);
    int ra = row0 + r;
    ra = (ra < M ? ra : M - 1) - row0;
    a_off[j] = (uint32_t)(((int64_t)ra * g.sam + c * 8) * 2) + 3072u - (uint32_t)((j & 3) * 1024);
  }
  const char* a_base = (const char*)g.A + ((int64_t)row0 * g.sam) * 2 + (int64_t)kb0 * kDmaRowB - 3072;
  const char* b_base;
#pragma unroll
  for (int j = 0; j < NB; ++j) {
    if constexpr (B_KC) {
      const int r = (wave * NB + j) * 8 + (lane >> 3);
      const int c = (lane & 7) ^ ((r >> 1) & 7);
      int rb = col0 + r;
      rb = (rb < N ? rb : N - 1) - col0;
      b_off[j] = (uint32_t)(((int64_t)rb * g.sbn + c * 8) * 2) + 3072u - (uint32_t)((j & 3) * 1024);
    } else {
      const int k = (wave * NB + j) * RPI + lane / CPRB;
      const int c = (lane % CPRB) ^ (((k & 3) << 2) | (((k >> 3) & 1) << 1));
      int cb = col0 + c * 8;
      cb = (cb + 8 <= N ? cb : N - 8) - col0;
      b_off[j] = (uint32_t)(((int64_t)k * g.sbk + cb) * 2) + 3072u - (uint32_t)((j & 3) * 1024);
    }
  }
  if constexpr (B_KC) b_base = (const char*)g.B + ((int64_t)col0 * g.sbn) * 2 + kb0 * b_step - 3072;
  else b_base = (const char*)g.B + (int64_t)col0 * 2 + kb0 * b_step - 3072;
  const int wave_s = __builtin_amdgcn_readfirstlane(wave);
  char* const dma_a = lds + wave_s * (NA * 1024);
  char* const dma_b = lds + A_OPB + wave_s * (NB * 1024);
  // operand bases of K step kk, forced into scalar registers
  auto uniform_ptr = [](const char* q) {
    const uint64_t v = (uint64_t)(uintptr_t)q;
    const uint32_t lo = __builtin_amdgcn_readfirstlane((uint32_t)v), hi = __builtin_amdgcn_readfirstlane((uint32_t)(v >> 32));
    return (const char*)(uintptr_t)(((uint64_t)hi << 32) | lo);
  };
  // A scalar register written by a vector instruction (v_readfirstlane) may be read by a memory instruction only
  // five wait states later.  The compiler keeps that distance for the loads it emits itself, but it cannot see
  // that the asm of issue() is such a load.  So the tile's two bases are made scalar once, here, with the wait
  // states behind them; what bases_of() derives from them is scalar arithmetic on scalar registers, which has no
  // such rule.  (The tile's row and column come from integer divisions, which run on the vector unit: without
  // this, how far a v_readfirstlane lands ahead of the first copy is up to the instruction scheduler.)
  // Variant FG_V_DMA_SCALAR_BASES (variants.h).  Off, the tested code: bases_of() makes the bases scalar per K step, and
  // the build's scan of the device assembly (isa_check.py) is what establishes that no copy follows a
  // v_readfirstlane too closely.
#if FG_V_DMA_SCALAR_BASES
  a_base = uniform_ptr(a_base);
  b_base = uniform_ptr(b_base);
  asm volatile("s_nop 4" : "+s"(a_base), "+s"(b_base));
#else
  static_assert(!kDmaCopyRunsEveryTile, "the three-quarter split on every tile needs FG_V_DMA_SCALAR_BASES");
#endif
  struct KBase { const char* a; const char* b; bool last; };
  auto bases_of = [&](int kk) {
    return KBase{uniform_ptr(a_base + (int64_t)kk * kDmaRowB), uniform_ptr(b_base + (int64_t)kk * b_step), RAGGED && kk == nk - 1};
  };
  // `first_c`: the instruction opens a run of consecutive issue() calls (M0 holds nothing known)
  auto issue = [&](int stage_bytes, const KBase& kbase, auto jc, auto first_c) {
    constexpr int j = decltype(jc)::value;  // 0..NDMA-1: the A instructions, then the B instructions
    constexpr bool IS_A = j < NA;
    constexpr int jj = IS_A ? j : j - NA;
    char* l = (IS_A ? dma_a : dma_b) + stage_bytes + (jj >> 2) * 4096;
    // Written as asm: scalar base + 32-bit lane offset + immediate, LDS address in M0 (set here, with the wait
    // state the hardware wants between a scalar write of M0 and an LDS-direct load; nothing else in these kernels
    // uses M0).  Through the builtin the compiler either goes back to 64-bit lane addresses (a quarter-rate
    // vector add per instruction) or needs a register copy and a wait state per instruction, and every
    // instruction issued here is a slot the wave's next MFMA waits for.
    if constexpr (decltype(first_c)::value != 0 || (jj & 3) == 0) {
      const uint32_t m0v = (uint32_t)(uintptr_t)FGK_LDSP(l);
      asm volatile("s_mov_b32 m0, %0\n\ts_nop 0" : : "s"(m0v) : "memory", "m0");
    }
    const uint32_t off = IS_A ? a_off[IS_A ? jj : 0] : b_off[IS_A ? 0 : jj];
    if constexpr (RAGGED) {
      if (kbase.last) {
        // the partial K step: per-lane 64-bit addresses, lanes whose chunk lies past K read zeros
        bool valid;
        if constexpr (IS_A || B_KC) {
          const int r = (wave * (IS_A ? NA : NB) + jj) * 8 + (lane >> 3);
          valid = (((lane & 7) ^ ((r >> 1) & 7)) * 8) < g.k_ragged;
        } else {
          valid = (wave * NB + jj) * RPI + lane / CPRB < g.k_ragged;
        }
        const char* gp = valid ? (IS_A ? kbase.a : kbase.b) + (uint64_t)off : (const char*)g.zeros;
        asm volatile("global_load_lds_dwordx4 %0, off offset:%1" : : "v"(gp), "n"((jj & 3) * 1024) : "memory");
        return;
      }
    }
    asm volatile("global_load_lds_dwordx4 %0, %1 offset:%2" : : "v"(off), "s"(IS_A ? kbase.a : kbase.b), "n"((jj & 3) * 1024) : "memory");
  };

  // ---- fragment addresses.  A fragment is 16 rows x 32 k: lane (r = lane % 16, g = lane / 16) holds the 8 k
  // 32 ks + 8 g ... of row r, i.e. chunk 4 ks + g of the row's 128 bytes.
  const int fr = lane & 15, fg = lane >> 4;
  const int q = fr >> 1;  // sub-tile rows start at multiples of 16, so (row >> 1) & 7 depends on fr only
  const int a_lane = (wm * WTM + fr) * kDmaRowB;
  int pos[2];
#pragma unroll
  for (int ks = 0; ks < 2; ++ks) pos[ks] = ((4 * ks + fg) ^ q) * 16;
  int b_lane = 0;      // K-contiguous B: like A
  uint32_t b_tr[TN];   // N-contiguous B: per sub-tile j, the lane's address within a stage
#pragma unroll
  for (int j = 0; j < TN; ++j) b_tr[j] = 0;
  if constexpr (B_KC) {
    b_lane = A_OPB + (wn * WTN + fr) * kDmaRowB;
  } else {
    // the transposing read hands lane t of every 16-lane row the 4 k of column t that the row's lanes addressed as
    // 4 k-rows x 4 column quads: lane -> k-row 8 g + m (+ 32 ks, + 4 for the second read), columns 4 (lane & 3) ...
    // of sub-tile j
    const int m = (lane & 15) >> 2, b1 = (lane & 3) >> 1;
    const int krow = 8 * fg + m;
    const int sw = (m << 2) | ((fg & 1) << 1);
#pragma unroll
    for (int j = 0; j < TN; ++j) {
      const int chunk = (wn * (WTN / 8) + j * 2 + b1) ^ sw;
      b_tr[j] = (uint32_t)(uintptr_t)(__attribute__((address_space(3))) char*)lds + A_OPB + krow * RBB + chunk * 16 +
                (lane & 1) * 8;
    }
  }

  f32x4 acc[TM][TN];
#pragma unroll
  for (int i = 0; i < TM; ++i)
#pragma unroll
    for (int j = 0; j < TN; ++j) acc[i][j] = f32x4{0.f, 0.f, 0.f, 0.f};

  // A fragments of sub-tiles 0 .. HM-1 (set 0) and HM .. TM-1 (set 1); B fragments of the k half 0 and 1
  Frag fa[2][HM];
  u32x4 fb[2][TN];
  // Per-stage lane addresses, kept in registers: a stage sits up to 3 x 64 KB into LDS, more than the offset field of
  // an LDS instruction holds, and the compiler would otherwise add the stage offset once per read.
  const uint32_t lds0 = (uint32_t)(uintptr_t)(__attribute__((address_space(3))) char*)lds;
  uint32_t a_st[NS][2], b_st[NS][2], b_tr_st[NS][B_KC ? 1 : TN];
#pragma unroll
  for (int st = 0; st < NS; ++st) {
#pragma unroll
    for (int ks = 0; ks < 2; ++ks) {
      a_st[st][ks] = lds0 + st * STAGEB + a_lane + pos[ks];
      b_st[st][ks] = lds0 + st * STAGEB + b_lane + pos[ks];
      asm volatile("" : "+v"(a_st[st][ks]), "+v"(b_st[st][ks]));
    }
#pragma unroll
    for (int x = 0; x < (B_KC ? 1 : TN); ++x) {
      b_tr_st[st][x] = b_tr[B_KC ? 0 : x] + st * STAGEB;
      asm volatile("" : "+v"(b_tr_st[st][x]));
    }
  }
  typedef __attribute__((address_space(3))) const char* LdsPtr;
  // `stc`: the stage as a constant (IntC<0 .. NS-1>) or IntC<-1> with its byte offset in stage_bytes
  auto read_a = [&](auto stc, int stage_bytes, auto ksc, auto hc, auto xc) {
    constexpr int ST = decltype(stc)::value, ks = decltype(ksc)::value, h = decltype(hc)::value, x = decltype(xc)::value;
    if constexpr (ST >= 0)
      fa[h][x] = *reinterpret_cast<__attribute__((address_space(3))) const Frag*>((LdsPtr)(uintptr_t)a_st[ST][ks] + (h * HM + x) * 16 * kDmaRowB);
    else
      fa[h][x] = *reinterpret_cast<const Frag*>(lds + stage_bytes + a_lane + (h * HM + x) * 16 * kDmaRowB + pos[ks]);
  };
  auto read_b = [&](auto stc, int stage_bytes, auto ksc, auto xc) {
    constexpr int ST = decltype(stc)::value, ks = decltype(ksc)::value, x = decltype(xc)::value;
    if constexpr (B_KC) {
      if constexpr (ST >= 0)
        fb[ks][x] = *reinterpret_cast<__attribute__((address_space(3))) const u32x4*>((LdsPtr)(uintptr_t)b_st[ST][ks] + x * 16 * kDmaRowB);
      else
        fb[ks][x] = *reinterpret_cast<const u32x4*>(lds + stage_bytes + b_lane + x * 16 * kDmaRowB + pos[ks]);
    } else {
      const uint32_t addr = ST >= 0 ? b_tr_st[ST >= 0 ? ST : 0][B_KC ? 0 : x] : b_tr[x] + stage_bytes;
      const u32x2 lo = lds_read_tr16_b64<(32 * ks) * RBB>(addr);
      const u32x2 hi = lds_read_tr16_b64<(32 * ks + 4) * RBB>(addr);
      fb[ks][x] = u32x4{lo[0], lo[1], hi[0], hi[1]};
    }
  };
  auto wait_reads = [&](auto ksc) {
    if constexpr (B_KC) FGK_WAIT_LGKM0();
    else lds_wait_tied(fb[decltype(ksc)::value]);
  };

  // ---- prologue: K steps 0 .. NS-2, and the head of step NS-1 (the part the last quarter of the step before
  // would issue)
  static_for<0, NS - 1>([&](auto sc) {
    constexpr int s = decltype(sc)::value;
    if (s < nk) {
      const KBase kbase = bases_of(s);
      static_for<0, NDMA>([&](auto jc) { issue(s * STAGEB, kbase, jc, IntC<(decltype(jc)::value == 0)>{}); });
    }
  });
  if (nk >= NS) {
    const KBase kbase = bases_of(NS - 1);
    static_for<0, HALF>([&](auto jc) { issue((NS - 1) * STAGEB, kbase, jc, IntC<(decltype(jc)::value == 0)>{}); });
    FGK_WAIT_VM(NDMA * (NS - 2) + HALF);  // K step 0 has landed
  } else {
    FGK_WAIT_VM(0);
  }
  __builtin_amdgcn_s_barrier();
  static_for<0, HM>([&](auto xc) { read_a(IntC<0>{}, 0, IntC<0>{}, IntC<0>{}, xc); });
  static_for<0, TN>([&](auto xc) { read_b(IntC<0>{}, 0, IntC<0>{}, xc); });
  wait_reads(IntC<0>{});
  __builtin_amdgcn_sched_barrier(0);

  // One K step = four quarter steps of HM x TN MFMAs: quarter (ks, h) multiplies the A sub-tiles of half h by all
  // B sub-tiles over the k half ks, while the fragments of the next quarter are read: the other A half, and behind
  // an h = 1 quarter also the B fragments of the next k half (quarter 3 reads them from the next stage).  The
  // memory operations of a quarter, reads first, are spread over its MFMAs.
  // REFILL_TAIL: quarters 0 and 1 issue the last C0 + C1 DMAs of K step kb+NS-1; REFILL_HEAD: quarter 3 issues the
  // first C3 DMAs of K step kb+NS (into the stage this step has just finished reading).  LATER = DMAs
  // that may still be in flight once K step kb+1 has landed: those of the K steps behind it, which retire in
  // order after it.
  // ST: the stage of K step kb when the caller knows it at compile time (the unrolled part of the loop), else -1.
  auto k_step = [&](int kb, auto st_c, auto tail_c, auto head_c, auto later_c) {
    constexpr int ST = decltype(st_c)::value;
    // LDS byte offset of the stage of K step kb + d
    auto stage_of = [&](auto dc) {
      constexpr int d = decltype(dc)::value;
      if constexpr (ST >= 0) return ((ST + d) % NS) * STAGEB;
      else return stage_off(kb + d);
    };
    constexpr bool REFILL_TAIL = decltype(tail_c)::value != 0;
    constexpr bool REFILL_HEAD = decltype(head_c)::value != 0;
    constexpr int LATER = decltype(later_c)::value;
    KBase kk_head = {nullptr, nullptr, false}, kk_tail = {nullptr, nullptr, false};
    if constexpr (REFILL_HEAD) kk_head = bases_of(kb + NS);
    if constexpr (REFILL_TAIL) kk_tail = bases_of(kb + NS - 1);
    static_for<0, 4>([&](auto qc) {
      constexpr int qt = decltype(qc)::value;
      constexpr int ks = qt >> 1, h = qt & 1;
      constexpr int nks = ((qt + 1) & 3) >> 1, nh = (qt + 1) & 1;   // the quarter the reads are for
      constexpr int NRA = HM, NRB = nh == 0 ? TN : 0, NRD = NRA + NRB;
      constexpr int ND = (qt == 0 && REFILL_TAIL) ? C0 : (qt == 1 && REFILL_TAIL) ? C1 : (qt == 3 && REFILL_HEAD) ? C3 : 0;
      constexpr int DONE = qt == 1 ? C3 + C0 : C3;  // copies of the tail's K step issued before this quarter
      constexpr int NOPS = NRD + ND, OPM = (NOPS + NMF - 1) / NMF;
      const int rstage = stage_of(IntC<(qt == 3 ? 1 : 0)>{});
      constexpr int RST = ST >= 0 ? (ST + (qt == 3 ? 1 : 0)) % NS : -1;
      static_for<0, NMF>([&](auto xc) {
        constexpr int x = decltype(xc)::value;
        constexpr int il = x / TN, j = x % TN;
        MfmaK32<T>::mma(__builtin_bit_cast(Frag, fb[ks][j]), fa[h][il], acc[h * HM + il][j]);
        static_for<0, OPM>([&](auto oc) {
          constexpr int o = x * OPM + decltype(oc)::value;
          if constexpr (o < NRA) read_a(IntC<RST>{}, rstage, IntC<nks>{}, IntC<nh>{}, IntC<(o < NRA ? o : 0)>{});
          else if constexpr (o < NRD) read_b(IntC<RST>{}, rstage, IntC<nks>{}, IntC<(o < NRD ? o - NRA : 0)>{});
          else if constexpr (o < NOPS) {
            if constexpr (qt != 3) issue(stage_of(IntC<NS - 1>{}), kk_tail, IntC<(o < NOPS ? DONE + (o - NRD) : 0)>{}, IntC<(o == NRD)>{});
            else issue(stage_of(IntC<NS>{}), kk_head, IntC<(o < NOPS ? o - NRD : 0)>{}, IntC<(o == NRD)>{});
          }
        });
        __builtin_amdgcn_sched_barrier(0);
      });
      if constexpr (qt == 2) {
        FGK_WAIT_VM(LATER);
        wait_reads(IntC<nks>{});
        __builtin_amdgcn_s_barrier();
      } else {
        wait_reads(IntC<nks>{});
      }
      __builtin_amdgcn_sched_barrier(0);
    });
  };
  // the steady state, NS steps per trip so that the stage of every step is a constant of the code
  int kb = 0;
  for (; kb + NS <= nk - NS; kb += NS)
    static_for<0, NS>([&](auto sc) { k_step(kb + decltype(sc)::value, sc, IntC<1>{}, IntC<1>{}, IntC<NDMA * (NS - 2)>{}); });
  static_for<0, NS - 1>([&](auto) {  // up to NS - 1 steady-state steps are left
    if (kb < nk - NS) {
      k_step(kb, IntC<-1>{}, IntC<1>{}, IntC<1>{}, IntC<NDMA * (NS - 2)>{});
      ++kb;
    }
  });
  // the last NS steps (fewer when nk < NS), by the number r of K steps behind them: nothing new to request
  // except the second half of the last step, and ever fewer DMAs left in flight
  static_for<0, NS - 1>([&](auto ic) {
    constexpr int r = NS - 1 - decltype(ic)::value;
    if (kb == nk - 1 - r) {
      k_step(kb, IntC<-1>{}, IntC<(r >= NS - 1 ? 1 : 0)>{}, IntC<0>{}, IntC<NDMA * cmin(NS - 2, r - 1)>{});
      ++kb;
    }
  });
  k_step(kb, IntC<-1>{}, IntC<0>{}, IntC<0>{}, IntC<0>{});
  mfma_drain(acc);

  finish(acc);
}

template <typename T, bool B_KC, int BM, int BN, int NS = 2, bool RAGGED = false>
__global__ __launch_bounds__(256, (2 * dma_lds_bytes(BM, BN, NS) <= 160 * 1024 ? 2 : 1)) void gemm_dma_kernel(GemmArgs g) {
  extern __shared__ __attribute__((aligned(16))) char lds[];
  int tm, tn;
  tile_coords(blockIdx.x + g.tile_base, g.tiles_m, g.tiles_n, tm, tn, B_KC ? 2 : 4);
  const int nk = (int)((g.K + kDmaBK - 1) / kDmaBK);
  dma_tile_mainloop<T, B_KC, BM, BN, NS, RAGGED>(
      g, lds, tm, tn, 0, nk, [&](f32x4 (&acc)[BM / 32][BN / 32]) { dma_tile_epilogue<T, BM, BN>(g, tm, tn, acc); });
}
// Stream-K over 128x128 tiles with the main loop above: the (tile, K step) units, tile-major, are dealt
// in equal contiguous ranges to the workgroups; a tile split between workgroups is finished by whichever
// of them arrives last (ticket per tile, fp32 partial tiles in the workspace, added in workgroup order so
// the result does not depend on who finishes).  Same scheme as gemm_streamk_kernel in gemm_tile.h.
template <typename T, bool B_KC, int NS>
__global__ __launch_bounds__(256, 2) void gemm_dma_streamk_kernel(GemmArgs g) {
  constexpr int BM = 128, BN = 128, TM = 4, TN = 4;  // 16x16 sub-tiles per wave
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
    __syncthreads();  // the LDS stages of the previous segment are no longer read
    dma_tile_mainloop<T, B_KC, BM, BN, NS>(g, lds, tm, tn, it0, it1 - it0, [&](f32x4 (&acc)[TM][TN]) {
      bool finish = (it0 == 0 && it1 == g.iters_per_tile);
      if (!finish) {
        // slot 0 of a workgroup: the tile it starts in; slot 1: a tile it enters from the left
        float* slot = g.partials + ((int64_t)w * 2 + (u_begin < tile_begin ? 1 : 0)) * (BM * BN);
#pragma unroll
        for (int i = 0; i < TM; ++i)
#pragma unroll
          for (int j = 0; j < TN; ++j)
#pragma unroll
            for (int e = 0; e < 4; ++e)
              __hip_atomic_store(slot + ((i * TN + j) * 4 + e) * 256 + tid, acc[i][j][e], __ATOMIC_RELAXED,
                                 __HIP_MEMORY_SCOPE_AGENT);
        // device-coherent stores: every one of them has completed before the ticket publishes them
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup");
        fg_wait_vmem_done();
        __syncthreads();
        const int w_first = sk_worker_of(g.sk_per, g.sk_rem, tile_begin);
        const int w_last = sk_worker_of(g.sk_per, g.sk_rem, tile_end - 1);
        if (tid == 0)
          ticket_s = __hip_atomic_fetch_add(g.tickets + w_first, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        __syncthreads();
        if (ticket_s == (unsigned)(w_last - w_first)) {
          finish = true;
#pragma unroll
          for (int i = 0; i < TM; ++i)
#pragma unroll
            for (int j = 0; j < TN; ++j)
#pragma unroll
              for (int e = 0; e < 4; ++e) acc[i][j][e] = 0.f;
          auto slot_of = [&](int w2) {
            return g.partials + ((int64_t)w2 * 2 + (sk_begin(g.sk_per, g.sk_rem, w2) < tile_begin ? 1 : 0)) * (BM * BN) + tid;
          };
          // contributors in workgroup order, two at a time: both partial tiles are requested before either is added,
          // so a pair costs one trip to memory
          int w2 = w_first;
          for (; w2 < w_last; w2 += 2) {
            const float* s0 = slot_of(w2);
            const float* s1 = slot_of(w2 + 1);
            float t0[TM * TN * 4], t1[TM * TN * 4];
#pragma unroll
            for (int x = 0; x < TM * TN * 4; ++x) t0[x] = __hip_atomic_load(s0 + x * 256, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
#pragma unroll
            for (int x = 0; x < TM * TN * 4; ++x) t1[x] = __hip_atomic_load(s1 + x * 256, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
#pragma unroll
            for (int i = 0; i < TM; ++i)
#pragma unroll
              for (int j = 0; j < TN; ++j)
#pragma unroll
                for (int e = 0; e < 4; ++e) acc[i][j][e] = (acc[i][j][e] + t0[(i * TN + j) * 4 + e]) + t1[(i * TN + j) * 4 + e];
          }
          if (w2 == w_last) {
            const float* s0 = slot_of(w2);
#pragma unroll
            for (int i = 0; i < TM; ++i)
#pragma unroll
              for (int j = 0; j < TN; ++j)
#pragma unroll
                for (int e = 0; e < 4; ++e)
                  acc[i][j][e] += __hip_atomic_load(s0 + ((i * TN + j) * 4 + e) * 256, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
          }
          if (tid == 0) __hip_atomic_store(g.tickets + w_first, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        }
      }
      if (finish) dma_tile_epilogue<T, BM, BN>(g, tm, tn, acc);
    });
    u = tile_begin + it1;
  }
}

}  // namespace fgk
