// Skinny GEMM (M <= 16) with a stream-K schedule for gfx950.
//
// With so few rows the product is a bandwidth-bound stream of B (arithmetic intensity ~ M flop per
// byte), so the schedule's only job is to keep every CU streaming an equal share of B.  The output
// is cut into tiles of 16 rows x 128 columns and K into steps of 32; the (tile, k-step) units, in
// tile-major order, are dealt in equal contiguous ranges to one persistent workgroup per CU
// (stream-K).  A workgroup walks its range segment by segment (a segment = its units inside one
// tile); its 8 waves split the segment's k-steps, accumulate in registers with
// v_mfma_f32_16x16x32_{bf16,f16}, and add their accumulators up through LDS.
//
// A segment that covers its tile's whole K range is finished on the spot.  A tile split between
// workgroups is finished by whichever of them arrives LAST: every contributor writes its fp32
// partial tile to its own slot of the workspace (device-coherent stores), then takes a ticket from
// the tile's counter (one device-scope atomic add).  The contributor that draws the last ticket
// reads all slots of the tile in workgroup order, adds them in that fixed order (so the result is
// bit-reproducible whoever finishes), applies the epilogue, stores C and resets the counter.
// Nobody ever waits for anybody, so there is nothing to deadlock or time out.
//
// B feeds the MFMA "A" operand (rows = output columns), the activations feed the "B" operand, so
// the accumulators hold C^T: lane (m = lane%16, g = lane/16) owns column slots 4g..4g+3.
//   B row-major (N contiguous): a lane loads an 8(k) x 8(n) block as eight 16-byte rows and
//     transposes it in registers (v_perm_b32); MFMA c of 8 then covers columns n0 + 8*slot + c.
//   B = W^T (K contiguous): a lane loads 16 bytes = 8 k of one column directly; MFMA c covers
//     columns n0 + 16*c + slot.
#include <atomic>
#include <stdlib.h>
#include <mutex>
#include "gemm_dma.h"

namespace fgk {

namespace {

constexpr int kTileN = 128, kStepK = 32, kWaves = 8, kBlock = kWaves * 64;
constexpr int kTileElems = 16 * kTileN;  // fp32 partial tile
constexpr int kEPT = kTileElems / kBlock;  // tile elements per thread in the block-wide phases
typedef float f32x4v __attribute__((ext_vector_type(4)));

template <typename T> struct Mfma16;
template <> struct Mfma16<bf16_t> {
  typedef bf16x8 Frag;
  static __device__ __forceinline__ f32x4v mma(Frag a, Frag b, f32x4v c) {
    return __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, b, c, 0, 0, 0);
  }
};
template <> struct Mfma16<f16_t> {
  typedef f16x8 Frag;
  static __device__ __forceinline__ f32x4v mma(Frag a, Frag b, f32x4v c) {
    return __builtin_amdgcn_mfma_f32_16x16x32_f16(a, b, c, 0, 0, 0);
  }
};

struct SkinnyArgs {
  GemmArgs g;
  int tiles_n, ksteps;  // output tiles along N, k-steps per tile
  int64_t per, rem;     // units per workgroup, and how many workgroups take one more
  int workers;
  float* partials;      // [workers][2][kTileElems]
  unsigned* tickets;    // [kMaxWorkers], zero between launches
};

__device__ __host__ __forceinline__ int64_t range_begin(int64_t per, int64_t rem, int64_t w) {
  return w * per + (w < rem ? w : rem);
}
// workgroup that owns unit u
__device__ __forceinline__ int worker_of(int64_t per, int64_t rem, int64_t u) {
  const int64_t big = rem * (per + 1);
  return (int)(u < big ? u / (per + 1) : rem + (u - big) / per);
}

// Device-coherent accesses to the partial tiles: they must be seen by CUs behind another L2.
__device__ __forceinline__ void st_coherent(float* p, float v) {
  __hip_atomic_store(p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
__device__ __forceinline__ float ld_coherent(const float* p) {
  return __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

template <typename T, bool B_ROWMAJOR>
__global__ __launch_bounds__(kBlock) void gemm_skinny_kernel(SkinnyArgs a) {
  typedef typename Mfma16<T>::Frag Frag;
  __shared__ float red[kWaves][kTileElems];  // accumulators of every wave, element-major [c][i][lane]
  __shared__ unsigned ticket_s;
  const GemmArgs& g = a.g;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int m = lane & 15, grp = lane >> 4;
  const int w = blockIdx.x;
  const int M = (int)g.M, N = (int)g.N, K = (int)g.K;
  const T* A = (const T*)g.A;
  const T* B = (const T*)g.B;

  const int64_t u_begin = range_begin(a.per, a.rem, w);
  const int64_t u_end = range_begin(a.per, a.rem, w + 1);
  int64_t u = u_begin;
  while (u < u_end) {
    const int tile = (int)(u / a.ksteps);
    const int64_t tile_begin = (int64_t)tile * a.ksteps;
    const int64_t tile_end = tile_begin + a.ksteps;
    const int ks0 = (int)(u - tile_begin);
    const int ks1 = (int)((u_end < tile_end ? u_end : tile_end) - tile_begin);
    const int n0 = tile * kTileN;

    // ---- this wave's share of the segment's k-steps --------------------------------------------
    const int nsteps = ks1 - ks0;
    const int share = (nsteps + kWaves - 1) / kWaves;
    const int my0 = ks0 + wave * share;
    const int my1 = (my0 + share < ks1) ? my0 + share : ks1;

    f32x4v acc[8];
#pragma unroll
    for (int c = 0; c < 8; ++c) acc[c] = f32x4v{0.f, 0.f, 0.f, 0.f};

    // a ring of kDepth k-steps in flight per wave: a wave's share is only a handful of steps, so the
    // depth of the ring decides how quickly the stream of B reaches full bandwidth
    constexpr int kDepth = 4;
    u32x4 bv[kDepth][8];
    u32x4 av[kDepth];
    auto load_step = [&](int ks, u32x4 (&bd)[8], u32x4& ad) {
      const int k0 = ks * kStepK;
      const int ka = k0 + grp * 8;
      ad = u32x4{0u, 0u, 0u, 0u};
      if (m < M && ka < K) ad = *reinterpret_cast<const u32x4*>(A + (int64_t)m * g.sam + ka);
      if constexpr (B_ROWMAJOR) {
        const int n = n0 + m * 8;  // m doubles as the column-slot index of this lane
#pragma unroll
        for (int j = 0; j < 8; ++j) {
          const int k = k0 + grp * 8 + j;
          bd[j] = u32x4{0u, 0u, 0u, 0u};
          if (k < K && n < N)
            bd[j] = __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(B + (int64_t)k * g.sbk + n));
        }
      } else {
#pragma unroll
        for (int c = 0; c < 8; ++c) {
          const int n = n0 + 16 * c + m;
          bd[c] = u32x4{0u, 0u, 0u, 0u};
          if (ka < K && n < N)
            bd[c] = __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(B + (int64_t)n * g.sbn + ka));
        }
      }
    };
    auto compute = [&](u32x4 (&bd)[8], u32x4& ad) {
      const Frag af = __builtin_bit_cast(Frag, ad);
#pragma unroll
      for (int c = 0; c < 8; ++c) {
        u32x4 o;
        if constexpr (B_ROWMAJOR) {
          // column c of the 8x8 block as a K-run: dword d = { k = 2d (low half), k = 2d+1 (high half) }
          const unsigned sel = (c & 1) ? 0x07060302u : 0x05040100u;
#pragma unroll
          for (int d = 0; d < 4; ++d) o[d] = __builtin_amdgcn_perm(bd[2 * d + 1][c >> 1], bd[2 * d][c >> 1], sel);
        } else {
          o = bd[c];
        }
        acc[c] = Mfma16<T>::mma(__builtin_bit_cast(Frag, o), af, acc[c]);
      }
    };
    const int nmine = my1 - my0;
#pragma unroll
    for (int p = 0; p < kDepth - 1; ++p)
      if (p < nmine) load_step(my0 + p, bv[p], av[p]);
    for (int i = 0; i < nmine; i += kDepth) {
#pragma unroll
      for (int p = 0; p < kDepth; ++p) {
        if (i + p < nmine) {
          if (i + p + kDepth - 1 < nmine)
            load_step(my0 + i + p + kDepth - 1, bv[(p + kDepth - 1) % kDepth], av[(p + kDepth - 1) % kDepth]);
          compute(bv[p], av[p]);
        }
      }
    }

    // ---- add the 8 waves' accumulators through LDS; thread t ends up with elements t + kBlock*j --
    __syncthreads();  // red[] of the previous segment is no longer read
#pragma unroll
    for (int c = 0; c < 8; ++c)
#pragma unroll
      for (int i = 0; i < 4; ++i) red[wave][(c * 4 + i) * 64 + lane] = acc[c][i];
    __syncthreads();
    float sum[kEPT];
#pragma unroll
    for (int j = 0; j < kEPT; ++j) {
      float s = 0.f;
#pragma unroll
      for (int v = 0; v < kWaves; ++v) s += red[v][tid + kBlock * j];
      sum[j] = s;
    }

    bool finish = (ks0 == 0 && ks1 == a.ksteps);  // the whole tile was ours
    if (!finish) {
      // slot 0 of a workgroup: the segment it starts in; slot 1: a tile it enters from the left
      float* slot = a.partials + ((int64_t)w * 2 + (u_begin < tile_begin ? 1 : 0)) * kTileElems;
#pragma unroll
      for (int j = 0; j < kEPT; ++j) st_coherent(slot + tid + kBlock * j, sum[j]);
      // The partial tile is written with device-coherent (write-through) stores, so no cache
      // write-back is needed to publish it: it is enough that every store has completed before the
      // ticket is drawn.  A device-scope release/acquire pair here would flush and invalidate the
      // whole L2 and costs more than the rest of the kernel.
      __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup");
      fg_wait_vmem_done();
      __syncthreads();  // every thread's slice of the partial tile is out
      const int w_first = worker_of(a.per, a.rem, tile_begin);
      const int w_last = worker_of(a.per, a.rem, tile_end - 1);
      if (tid == 0)
        ticket_s = __hip_atomic_fetch_add(a.tickets + w_first, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      __syncthreads();
      if (ticket_s == (unsigned)(w_last - w_first)) {
        finish = true;  // the loads below bypass the non-coherent caches (device-coherent loads)
#pragma unroll
        for (int j = 0; j < kEPT; ++j) sum[j] = 0.f;
        // contributors in groups of kGroup: all loads of a group are issued before the first add, so a
        // group costs one memory round trip; the adds keep workgroup order
        constexpr int kGroup = 8;
        for (int wb = w_first; wb <= w_last; wb += kGroup) {
          float part[kGroup][kEPT];
#pragma unroll
          for (int q = 0; q < kGroup; ++q) {
            const int w2 = wb + q <= w_last ? wb + q : w_last;
            const float* src =
                a.partials + ((int64_t)w2 * 2 + (range_begin(a.per, a.rem, w2) < tile_begin ? 1 : 0)) * kTileElems;
#pragma unroll
            for (int j = 0; j < kEPT; ++j) part[q][j] = ld_coherent(src + tid + kBlock * j);
          }
#pragma unroll
          for (int q = 0; q < kGroup; ++q)
            if (wb + q <= w_last) {
#pragma unroll
              for (int j = 0; j < kEPT; ++j) sum[j] += part[q][j];
            }
        }
        if (tid == 0) __hip_atomic_store(a.tickets + w_first, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      }
    }
    if (finish) {
      T* C = (T*)g.C;
      const T* bias = (const T*)g.bias;
#pragma unroll
      for (int j = 0; j < kEPT; ++j) {
        const int e = tid + kBlock * j;           // element (c, i, lane) of the tile
        const int el = e & 63, ci = e >> 6;
        const int em = el & 15, eg = el >> 4;
        const int c = ci >> 2, i = ci & 3;
        const int n = n0 + (B_ROWMAJOR ? 8 * (4 * eg + i) + c : 16 * c + 4 * eg + i);
        if (em < M && n < N) {
          float v = sum[j];
          if (bias != nullptr) v = v * g.alpha + (float)bias[(int64_t)em * g.sim + (int64_t)n * g.sin] * g.beta;
          else if (g.alpha != 1.0f) v = v * g.alpha;
          C[(int64_t)em * g.scm + (int64_t)n * g.scn] = (T)v;
        }
      }
    }
    u = tile_begin + ks1;
  }
}

// ---- K-contiguous B (B = W^T with W [N, K]: the layout of a linear layer's weight) -------------
//
// Read straight into MFMA fragments, this layout gives every load instruction 16 rows x 64 bytes: half
// cache lines, and only as many bytes in flight as registers can hold.  Here the rows go to LDS by
// asynchronous copies (global_load_lds) instead, 8 rows x 128 bytes per instruction, into a private
// ring of slots per wave, issued ring-1 steps ahead of their use; fragments are read back
// from LDS (the 16-byte pieces of a row are permuted by the row number on the way in, so that the
// sixteen lanes of a fragment read hit different banks).  The output tile is 16 rows x 16 columns:
// with that few columns a workgroup's range usually covers whole tiles (N = 4096 gives exactly one
// tile per CU of a 256-CU part) and there is nothing to fix up between workgroups; split tiles use
// the same ticket scheme as above.  Requires K % 64 == 0.
// Wide outputs (N >= 8192) take 32-column tiles on a ring of 4 slots instead: the same bytes in flight, but
// every A fragment (which all workgroups fetch from L2 at the same time) feeds two column blocks, and a
// workgroup restarts its pipeline half as often.
#if FG_V_SKINNY_ASM_A
// Variant FG_V_SKINNY_ASM_A (variants.h).  The A fragments of gemm_skinny_kc_kernel are loaded into a ring of
// registers RING - 1 steps ahead of their use, so a register written in one trip of the main loop is read in the next.
// The compiler places the waits for the loads it emits, and across the loop's back edge it waits for EVERY operation
// in flight (s_waitcnt vmcnt(0) in front of the first use of a trip): once per RING steps the wave has nothing on
// its way.  Here the loads are written as asm, which the compiler does not count, and the wait that makes a slot's
// registers valid is the counted one the copies into LDS already use.  The wait names the slot's registers as
// operands, so no use of them can be scheduled in front of it; the build's scan of the device assembly
// (isa_check.py, scan_vmem_loads) follows the VM counter through the loop and fails on any instruction that touches
// a register whose load may still be outstanding.
__device__ __forceinline__ void kc_load_a(u32x4& dst, const char* p) {
  asm volatile("global_load_dwordx4 %0, %1, off" : "=v"(dst) : "v"(p) : "memory");
}
template <int N, int NAL> __device__ __forceinline__ void kc_wait_vm_pin(u32x4 (&r)[NAL]) {
  static_assert(NAL == 2 || NAL == 4 || NAL == 8, "two loads per 16-row block");
  if constexpr (NAL == 2) {
    asm volatile("s_waitcnt vmcnt(%2)" : "+v"(r[0]), "+v"(r[1]) : "n"(N) : "memory");
  } else if constexpr (NAL == 4) {
    asm volatile("s_waitcnt vmcnt(%4)" : "+v"(r[0]), "+v"(r[1]), "+v"(r[2]), "+v"(r[3]) : "n"(N) : "memory");
  } else {
    asm volatile("s_waitcnt vmcnt(%8)"
                 : "+v"(r[0]), "+v"(r[1]), "+v"(r[2]), "+v"(r[3]), "+v"(r[4]), "+v"(r[5]), "+v"(r[6]), "+v"(r[7])
                 : "n"(N) : "memory");
  }
}
#endif

constexpr int kcStepK = 64;
constexpr int kcLdsBytes = kWaves * 8 * 16 * kcStepK * 2;  // 128 KB: 8 slots of 16 rows, or 4 slots of 32 rows, per wave

// MB = 16-row blocks of A (1, 2 or 4: up to 64 rows).  Every B fragment read from LDS feeds MB MFMAs.  With MB > 1
// the cross-wave reduction buffer would not fit next to the ring, so it lives in the ring itself: after the last
// step of a segment every wave's copies have landed, each wave writes its accumulators into its own ring region,
// and a barrier at the start of the next segment keeps that segment's copies from overwriting sums still being read.
template <typename T, int TN, int RING, bool A_LINES, int MB>
__global__ __launch_bounds__(kBlock) void gemm_skinny_kc_kernel(SkinnyArgs a) {
  typedef typename Mfma16<T>::Frag Frag;
  constexpr int SLOTB = TN * kcStepK * 2;      // bytes of one ring slot
  constexpr int NCB = TN / 16;                 // 16-column blocks per tile
  constexpr int NDMA = TN / 8;                 // copy instructions per step (8 rows x 128 bytes each)
  constexpr int NAL = 2 * MB;                  // A loads per step
  constexpr int OPS = NDMA + NAL;              // memory operations per step
  constexpr int TILE_ELEMS = 16 * MB * TN;
  constexpr int EPT = (TILE_ELEMS + kBlock - 1) / kBlock;  // tile elements per thread in the block-wide phases
  constexpr int WAVE_RING = RING * SLOTB;
  static_assert(kWaves * WAVE_RING <= kcLdsBytes, "ring exceeds the LDS budget");
  static_assert(OPS * (RING - 1) < 64, "wait count exceeds the counter");
  static_assert(MB == 1 || A_LINES, "several row blocks are fetched in whole lines");
  static_assert(TILE_ELEMS * 4 <= WAVE_RING, "a wave's accumulators fit its own ring region");
  static_assert(TILE_ELEMS % kBlock == 0 || TILE_ELEMS < kBlock, "whole elements per thread");
  static_assert(TILE_ELEMS <= kTileElems, "partial tiles fit the workspace slots");
  extern __shared__ __attribute__((aligned(16))) char lds[];
  __shared__ unsigned ticket_s;
  const GemmArgs& g = a.g;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int m = lane & 15, grp = lane >> 4;
  const int w = blockIdx.x;
  const int M = (int)g.M, N = (int)g.N;
  const char* A = (const char*)g.A;
  const char* B = (const char*)g.B;
  char* const ring = lds + __builtin_amdgcn_readfirstlane(wave) * WAVE_RING;
  float* const red_mine = reinterpret_cast<float*>(ring);  // this wave's slice of the reduction buffer
  // fragment of MFMA h of column block c: row 16c + m of the slot, 16-byte piece 4h + grp, stored at position
  // piece ^ (row & 7); (16c + m) & 7 == m & 7, so the block only adds c * 2048 bytes
  int rd[2];
#pragma unroll
  for (int h = 0; h < 2; ++h) rd[h] = m * 128 + (((4 * h + grp) ^ (m & 7)) << 4);

  const int64_t u_begin = range_begin(a.per, a.rem, w);
  const int64_t u_end = range_begin(a.per, a.rem, w + 1);
  int64_t u = u_begin;
  while (u < u_end) {
    const int tile = (int)(u / a.ksteps);
    const int64_t tile_begin = (int64_t)tile * a.ksteps;
    const int64_t tile_end = tile_begin + a.ksteps;
    const int ks0 = (int)(u - tile_begin);
    const int ks1 = (int)((u_end < tile_end ? u_end : tile_end) - tile_begin);
    const int n0 = tile * TN;

    const int nsteps = ks1 - ks0;
    const int share = (nsteps + kWaves - 1) / kWaves;
    const int my0 = ks0 + wave * share;
    const int my1 = (my0 + share < ks1) ? my0 + share : ks1;
    const int nmine = my1 - my0;

    __syncthreads();  // the sums of the previous segment (kept in the ring) are no longer read

    f32x4v acc[MB][NCB];
#pragma unroll
    for (int rb = 0; rb < MB; ++rb)
#pragma unroll
      for (int c = 0; c < NCB; ++c) acc[rb][c] = f32x4v{0.f, 0.f, 0.f, 0.f};
    if (nmine > 0) {
      // copy instruction i of a step: slot rows 8i + lane/8, the lane's piece chosen so that it lands permuted
      const char* bsrc[NDMA];
#pragma unroll
      for (int i = 0; i < NDMA; ++i) {
        const int r = 8 * i + (lane >> 3);
        const int c = (lane & 7) ^ (r & 7);
        int n = n0 + r;
        n = n < N ? n : N - 1;
        bsrc[i] = B + ((int64_t)n * g.sbn + c * 8) * 2 - i * 1024;  // the instruction offset moves both addresses
      }
      // A_LINES (more than 8 rows): A is fetched in whole cache lines, load j of a step covering rows 8j .. 8j+7
      // with eight lanes per row (a load in fragment order touches 16 half lines; measured 4 us of a 30 us call).
      // The fragment of MFMA h of row block rb, piece 4h + grp of row 16rb + m, then sits in load 2rb + m / 8 of
      // lane (m % 8) * 8 + 4h + grp and is fetched from there with ds_bpermute when the step is computed.  With few
      // rows the lanes of a fragment load share their lines anyway and the loads go straight to fragment order
      // (load h = MFMA h).  Rows beyond M are computed on a copy of the last row and never stored.
      const char* asrc[NAL];
#pragma unroll
      for (int j = 0; j < NAL; ++j) {
        int fr = A_LINES ? 8 * j + (lane >> 3) : m;
        fr = fr < M ? fr : M - 1;
        asrc[j] = A + ((int64_t)fr * g.sam + (A_LINES ? (lane & 7) : 4 * j + grp) * 8) * 2;
      }
      int perm[2];
#pragma unroll
      for (int h = 0; h < 2; ++h) perm[h] = ((m & 7) * 8 + 4 * h + grp) * 4;
      const bool upper = m >= 8;
      u32x4 af[RING][NAL];
      // Every workgroup would otherwise walk K in the same order at the same time, all of them asking L2 for the
      // same lines of A (and, with power-of-two row lengths, the same memory channels for B): each wave starts its
      // share at its own offset and wraps around.  The order is a function of (workgroup, wave), so results stay
      // bit-identical from run to run.
      const int rot = (int)(((unsigned)w * 13u + (unsigned)wave * 5u) % (unsigned)nmine);
      // Every step issues the same memory operations, so the count to wait for is a constant; steps past the
      // end of the share re-read the last one (served by the caches) and are not computed.
      auto issue = [&](int step, auto pc) {
        constexpr int p = decltype(pc)::value;
        const int sidx = step < nmine ? step : nmine - 1;
        int kidx = sidx + rot;
        kidx = kidx >= nmine ? kidx - nmine : kidx;
        const int64_t koff = (int64_t)(my0 + kidx) * (kcStepK * 2);
        char* slot = ring + p * SLOTB;
        static_for<0, NDMA>([&](auto ic) {
          constexpr int i = decltype(ic)::value;
          __builtin_amdgcn_global_load_lds(FGK_GLBP(bsrc[i] + koff), FGK_LDSP(slot), 16, i * 1024, 0);
        });
#if FG_V_SKINNY_ASM_A
        if constexpr (A_LINES) {
#pragma unroll
          for (int j = 0; j < NAL; ++j) kc_load_a(af[p][j], asrc[j] + koff);
        } else
#endif
        {
#pragma unroll
          for (int j = 0; j < NAL; ++j) af[p][j] = *reinterpret_cast<const u32x4*>(asrc[j] + koff);
        }
      };
      auto compute = [&](auto pc) {
        constexpr int p = decltype(pc)::value;
        const char* slot = ring + p * SLOTB;
        u32x4 fa[MB][2];
        if constexpr (A_LINES) {
#pragma unroll
          for (int rb = 0; rb < MB; ++rb)
#pragma unroll
            for (int h = 0; h < 2; ++h)
#pragma unroll
              for (int d = 0; d < 4; ++d) {
                const int lo = __builtin_amdgcn_ds_bpermute(perm[h], (int)af[p][2 * rb][d]);
                const int hi = __builtin_amdgcn_ds_bpermute(perm[h], (int)af[p][2 * rb + 1][d]);
                fa[rb][h][d] = (uint32_t)(upper ? hi : lo);
              }
        } else {
          fa[0][0] = af[p][0];
          fa[0][1] = af[p][1];
        }
#pragma unroll
        for (int c = 0; c < NCB; ++c) {
#pragma unroll
          for (int h = 0; h < 2; ++h) {
            const Frag bf = *reinterpret_cast<const Frag*>(slot + c * 2048 + rd[h]);
#pragma unroll
            for (int rb = 0; rb < MB; ++rb)
              acc[rb][c] = Mfma16<T>::mma(bf, __builtin_bit_cast(Frag, fa[rb][h]), acc[rb][c]);
          }
        }
      };
      static_for<0, RING - 1>([&](auto pc) {
        issue(decltype(pc)::value, pc);
        __builtin_amdgcn_sched_barrier(0);
      });
      // whole rounds of the ring: issue, wait for the step issued RING-1 steps ago, compute -- no branches,
      // so the number of operations in flight at every wait is known
      int i = 0;
      for (; i + RING <= nmine; i += RING) {
        static_for<0, RING>([&](auto pc) {
          constexpr int p = decltype(pc)::value;
          issue(i + p + RING - 1, IntC<(p + RING - 1) % RING>{});
#if FG_V_SKINNY_ASM_A
          if constexpr (A_LINES) kc_wait_vm_pin<OPS * (RING - 1)>(af[p]);
          else
#endif
            FGK_WAIT_VM(OPS * (RING - 1));
          compute(pc);
          __builtin_amdgcn_sched_barrier(0);
        });
      }
      // the rest (fewer than RING steps) is already on its way
      FGK_WAIT_VM(0);
      const int rest = nmine - i;
      static_for<0, RING - 1>([&](auto pc) {
#if FG_V_SKINNY_ASM_A
        if constexpr (A_LINES) kc_wait_vm_pin<0>(af[decltype(pc)::value]);  // (names the registers: no use moves above it)
#endif
        if (decltype(pc)::value < rest) compute(pc);
      });
    }

    // ---- add the 8 waves' accumulators through LDS (the wave's own ring region: all its copies have landed
    // and its fragment reads are done); thread t ends up with elements t + kBlock * j ---------------------------
#pragma unroll
    for (int rb = 0; rb < MB; ++rb)
#pragma unroll
      for (int c = 0; c < NCB; ++c)
#pragma unroll
        for (int i = 0; i < 4; ++i) red_mine[((rb * NCB + c) * 4 + i) * 64 + lane] = acc[rb][c][i];
    __syncthreads();
    float sum[EPT];
#pragma unroll
    for (int j = 0; j < EPT; ++j) {
      const int e = tid + kBlock * j;
      float sacc = 0.f;
      if (e < TILE_ELEMS) {
#pragma unroll
        for (int v = 0; v < kWaves; ++v) sacc += reinterpret_cast<const float*>(lds + v * WAVE_RING)[e];
      }
      sum[j] = sacc;
    }

    bool finish = (ks0 == 0 && ks1 == a.ksteps);
    if (!finish) {
      float* slot = a.partials + ((int64_t)w * 2 + (u_begin < tile_begin ? 1 : 0)) * TILE_ELEMS;
#pragma unroll
      for (int j = 0; j < EPT; ++j)
        if (tid + kBlock * j < TILE_ELEMS) st_coherent(slot + tid + kBlock * j, sum[j]);
      __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup");
      fg_wait_vmem_done();
      __syncthreads();
      const int w_first = worker_of(a.per, a.rem, tile_begin);
      const int w_last = worker_of(a.per, a.rem, tile_end - 1);
      if (tid == 0)
        ticket_s = __hip_atomic_fetch_add(a.tickets + w_first, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      __syncthreads();
      if (ticket_s == (unsigned)(w_last - w_first)) {
        finish = true;
#pragma unroll
        for (int j = 0; j < EPT; ++j) sum[j] = 0.f;
        for (int w2 = w_first; w2 <= w_last; ++w2) {
          const float* src =
              a.partials + ((int64_t)w2 * 2 + (range_begin(a.per, a.rem, w2) < tile_begin ? 1 : 0)) * TILE_ELEMS;
#pragma unroll
          for (int j = 0; j < EPT; ++j)
            if (tid + kBlock * j < TILE_ELEMS) sum[j] += ld_coherent(src + tid + kBlock * j);
        }
        if (tid == 0) __hip_atomic_store(a.tickets + w_first, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      }
    }
    if (finish) {
      T* C = (T*)g.C;
      const T* bias = (const T*)g.bias;
#pragma unroll
      for (int j = 0; j < EPT; ++j) {
        // element e = ((rb * NCB + cb) * 4 + i) * 64 + el of the accumulators: row 16rb + (el & 15),
        // column 16cb + 4 * (el >> 4) + i
        const int e = tid + kBlock * j;
        const int el = e & 63, i = (e >> 6) & 3, blk = e >> 8;
        const int cb = blk % NCB, rb = blk / NCB;
        const int em = 16 * rb + (el & 15), eg = el >> 4;
        const int n = n0 + 16 * cb + 4 * eg + i;
        if (e < TILE_ELEMS && em < M && n < N) {
          float v = sum[j];
          if (bias != nullptr) v = v * g.alpha + (float)bias[(int64_t)em * g.sim + (int64_t)n * g.sin] * g.beta;
          else if (g.alpha != 1.0f) v = v * g.alpha;
          C[(int64_t)em * g.scm + (int64_t)n * g.scn] = (T)v;
        }
      }
    }
    u = tile_begin + ks1;
  }
}

template <typename T, int TN, int RING, bool A_LINES, int MB>
int launch_kc_t(const SkinnyArgs& a, hipStream_t st) {
  static std::once_flag once;
  static hipError_t attr_err = hipSuccess;
  auto kern = gemm_skinny_kc_kernel<T, TN, RING, A_LINES, MB>;
  std::call_once(once, [&] {
    attr_err = hipFuncSetAttribute(reinterpret_cast<const void*>(kern), hipFuncAttributeMaxDynamicSharedMemorySize, kcLdsBytes);
  });
  if (attr_err != hipSuccess) {
    fg_set_error("gemm(stream-K, skinny): cannot reserve %d bytes of LDS: %s", kcLdsBytes, hipGetErrorString(attr_err));
    return FG_ERR_LAUNCH;
  }
  hipLaunchKernelGGL(kern, dim3((unsigned)a.workers), dim3(kBlock), kcLdsBytes, st, a);
  return fg_check_launch("gemm(stream-K, skinny)");
}

// Up to 16 rows: 16-column tiles on 8 slots, or 32-column tiles on 4 slots (wide outputs).  17..32 rows: the same
// with two row blocks.  33..64 rows: four row blocks, always on 32-column tiles (10 memory operations per step on an
// 8-slot ring would overrun the wait counter, and the A fragments of four row blocks want two column blocks to feed).
template <typename T>
int launch_kc(const SkinnyArgs& a, int tile, hipStream_t st) {
  const int64_t M = a.g.M;
  if (M > 32) return launch_kc_t<T, 32, 4, true, 4>(a, st);
  if (tile == 32) {
    if (M > 16) return launch_kc_t<T, 32, 4, true, 2>(a, st);
    return M > 8 ? launch_kc_t<T, 32, 4, true, 1>(a, st) : launch_kc_t<T, 32, 4, false, 1>(a, st);
  }
  if (M > 16) return launch_kc_t<T, 16, 8, true, 2>(a, st);
  return M > 8 ? launch_kc_t<T, 16, 8, true, 1>(a, st) : launch_kc_t<T, 16, 8, false, 1>(a, st);
}

}  // namespace

// 0: not a case for this kernel; 1: B row-major (N contiguous); 2: B = W^T (K contiguous)
int skinny_supported(const GemmArgs& g, int dtype, int amode, int bmode) {
  if (dtype != FG_F16 && dtype != FG_BF16) return 0;
  if (g.M > 64 || amode != LOAD_K) return 0;
  if (g.K < 1024) return 0;  // worth it only when K is deep enough to give every CU several k-steps
  // 17..64 rows: only the kernel that stages a K-contiguous B through LDS has the row blocks for them.  Every
  // column tile re-reads its rows of A from L2, M / 32 bytes per byte of B, so it pays where the 128x128 tile
  // kernels cannot fill the machine (narrow outputs) and, up to 32 rows, for outputs of moderate width; measured
  // against those kernels on 4096..32000 columns with K = 4096..14336.
  if (g.M > 16) {
    if (bmode != LOAD_K || g.K % kcStepK != 0 || fg_options().skinny_no_lds) return 0;
    const bool pays = g.N <= 8192 || (g.M <= 32 && g.N <= 24576);
    return pays || fg_options().skinny_rows64 ? 2 : 0;
  }
  if (bmode == LOAD_K) return 2;
  if (bmode == LOAD_MN) return 1;
  return 0;
}

size_t skinny_workspace_bytes(int64_t M, int64_t N, int64_t K, int num_cu) {
  if (M > 64 || K < 1024) return 0;
  return kPartialOffset + (size_t)num_cu * 2 * kTileElems * sizeof(float);
}

int skinny_launch(const GemmArgs& g, int dtype, int b_kind, void* workspace, size_t workspace_bytes, int num_cu,
                  hipStream_t st) {
  FG_REQUIRE(workspace_bytes >= skinny_workspace_bytes(g.M, g.N, g.K, num_cu), FG_ERR_WORKSPACE,
             "gemm(stream-K): workspace too small");
  FG_REQUIRE(fg_aligned(workspace, 256), FG_ERR_WORKSPACE, "gemm(stream-K): workspace must be 256-byte aligned");
  SkinnyArgs a;
  a.g = g;
  // K-contiguous B with K a multiple of 64: the kernel that stages B through LDS, on 16-column tiles
  const bool kc = b_kind == 2 && g.K % kcStepK == 0 && !fg_options().skinny_no_lds;
  // 32-column tiles once they still give every CU a tile of its own (measurement aid: FG_SKINNY_TILE=16|32)
  int kc_tile = g.N >= 32 * (int64_t)num_cu ? 32 : 16;
  if (fg_options().skinny_tile != 0) kc_tile = fg_options().skinny_tile;
  if (g.M > 32) kc_tile = 32;
  a.tiles_n = (int)fg_cdiv(g.N, kc ? kc_tile : kTileN);
  a.ksteps = (int)fg_cdiv(g.K, kc ? kcStepK : kStepK);
  const int64_t units = (int64_t)a.tiles_n * a.ksteps;
  if (num_cu > kMaxWorkers) num_cu = kMaxWorkers;
  a.workers = (int)(units < num_cu ? units : num_cu);
  a.per = units / a.workers;
  a.rem = units % a.workers;
  char* ws = (char*)workspace;
  a.tickets = (unsigned*)(ws + kTicketOffset);
  a.partials = (float*)(ws + kPartialOffset);
  if (kc) return dtype == FG_BF16 ? launch_kc<bf16_t>(a, kc_tile, st) : launch_kc<f16_t>(a, kc_tile, st);
  FG_REQUIRE(g.M <= 16, FG_ERR_UNSUPPORTED, "gemm(stream-K, skinny): more than 16 rows need the LDS-staged kernel");
  dim3 grid((unsigned)a.workers), block(kBlock);
  if (dtype == FG_BF16) {
    if (b_kind == 1) hipLaunchKernelGGL((gemm_skinny_kernel<bf16_t, true>), grid, block, 0, st, a);
    else hipLaunchKernelGGL((gemm_skinny_kernel<bf16_t, false>), grid, block, 0, st, a);
  } else {
    if (b_kind == 1) hipLaunchKernelGGL((gemm_skinny_kernel<f16_t, true>), grid, block, 0, st, a);
    else hipLaunchKernelGGL((gemm_skinny_kernel<f16_t, false>), grid, block, 0, st, a);
  }
  return fg_check_launch("gemm(stream-K, skinny)");
}

}  // namespace fgk

// ---------------------------------------------------------------------------------------------
// fg_gemm_skinny_static: the skinny stream-K GEMM for callers that cannot allocate device memory
// (code under HIP graph capture, serving loops, harnesses that forbid hipMalloc).  Same kernels
// as above; the partial tiles and ticket counters live in a file-scope device array instead of a
// caller-provided workspace.  Every GPU holds its own copy of the array until the process ends;
// all calls on a GPU share it, so calls that overlap on one GPU (two streams) race.
// ---------------------------------------------------------------------------------------------
namespace fgk {
int pick_mode(const void* base, int64_t rows, int64_t K, int64_t s_row, int64_t s_k, int elem_bytes);  // gemm.hip
int num_cus(int device);                                                                                // gemm.hip
}

namespace {
constexpr int kStaticMaxCu = 256;  // MI355X; a device with more CUs is turned away
constexpr size_t kStaticScratchBytes = fgk::kPartialOffset + (size_t)kStaticMaxCu * 2 * 16 * 128 * sizeof(float);
}  // namespace

static __device__ __align__(256) unsigned char scratch[kStaticScratchBytes];  // 4 198 656 bytes

namespace {
__global__ void clear_tickets_kernel(unsigned* tickets, int n) {
  const int i = blockIdx.x * blockDim.x + threadIdx.x;
  if (i < n) tickets[i] = 0u;
}

// Device address of this GPU's copy of `scratch`, looked up once per device with that device current.
// In host code the array's name is only a handle for this lookup, never an address to hand to a kernel.
// The lookup is not a stream operation and may load the code object: it must not happen while `st` is being
// captured, so a first call on a device that arrives under capture is refused (fg_device_info on that device, or
// any eager call of the entry point, makes the lookup beforehand).
std::mutex g_static_mu;
unsigned char* g_static_ptr[64] = {nullptr};

int static_scratch(unsigned char** out, hipStream_t st, bool launching = true) {
  int dev = 0;
  hipError_t e = hipGetDevice(&dev);
  if (e != hipSuccess || dev < 0 || dev >= 64) {
    fg_set_error("gemm_skinny_static: cannot identify the current device: %s", hipGetErrorString(e));
    return FG_ERR_INVALID;
  }
  std::lock_guard<std::mutex> lk(g_static_mu);
  if (g_static_ptr[dev] == nullptr) {
    hipStreamCaptureStatus cap = hipStreamCaptureStatusNone;
    if (launching && hipStreamIsCapturing(st, &cap) != hipSuccess) (void)hipGetLastError();
    if (cap != hipStreamCaptureStatusNone) {
      fg_set_error("gemm_skinny_static: the first call on device %d came under stream capture; call fg_device_info(%d, "
                   "...) or this entry point once outside capture first", dev, dev);
      return FG_ERR_UNSUPPORTED;
    }
    void* p = nullptr;
    e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
    if (e != hipSuccess || p == nullptr) {
      (void)hipGetLastError();
      fg_set_error("gemm_skinny_static: hipGetSymbolAddress failed on device %d: %s", dev, hipGetErrorString(e));
      return FG_ERR_LAUNCH;
    }
    g_static_ptr[dev] = (unsigned char*)p;
  }
  *out = g_static_ptr[dev];
  return FG_OK;
}
}  // namespace

// Called by fg_device_info (abi.cpp): looks the address up for `device` ahead of the first call, so that the first
// fg_gemm_skinny_static on that device may come under stream capture.  Failure is not an error of fg_device_info;
// the entry point reports it when it is called.
void fg_static_scratch_prime(int device) {
  int cur = 0;
  if (hipGetDevice(&cur) != hipSuccess) { (void)hipGetLastError(); return; }
  if (device < 0) device = cur;
  if (device >= 64) return;
  {
    std::lock_guard<std::mutex> lk(g_static_mu);
    if (g_static_ptr[device] != nullptr) return;
  }
  if (device != cur && hipSetDevice(device) != hipSuccess) { (void)hipGetLastError(); return; }
  unsigned char* p = nullptr;
  (void)static_scratch(&p, nullptr, /*launching=*/false);
  if (device != cur) (void)hipSetDevice(cur);
}

extern "C" int fg_gemm_skinny_static(const void* A, const void* B, const void* bias, void* C, int64_t M, int64_t N,
                                     int64_t K, int64_t sam, int64_t sak, int64_t sbk, int64_t sbn, int64_t sim,
                                     int64_t sin_, int64_t scm, int64_t scn, float alpha, float beta, int ab_dtype,
                                     int c_dtype, int bias_dtype, void* stream) {
  using namespace fgk;
  FG_REQUIRE(M >= 0 && N >= 0 && K >= 0, FG_ERR_INVALID, "gemm_skinny_static: negative size");
  FG_REQUIRE(ab_dtype == FG_F16 || ab_dtype == FG_BF16, FG_ERR_UNSUPPORTED,
             "gemm_skinny_static: 16-bit inputs only (dtype %d)", ab_dtype);
  FG_REQUIRE(c_dtype == ab_dtype && (bias == nullptr || bias_dtype == ab_dtype), FG_ERR_UNSUPPORTED,
             "gemm_skinny_static: output and bias must have the input dtype");
  if (M == 0 || N == 0) return FG_OK;
  FG_REQUIRE(M <= 64, FG_ERR_UNSUPPORTED,
             "gemm_skinny_static: %lld rows exceed the maximum of 64 the static scratch buffer is sized for; use fg_gemm",
             (long long)M);
  FG_REQUIRE(A && B && C, FG_ERR_INVALID, "gemm_skinny_static: null pointer");
  FG_REQUIRE(N < ((int64_t)1 << 31) && K < ((int64_t)1 << 31), FG_ERR_UNSUPPORTED, "gemm_skinny_static: extent exceeds 2^31");
  GemmArgs g = {};
  g.A = A; g.B = B; g.bias = bias; g.C = C;
  g.M = M; g.N = N; g.K = K;
  g.sam = sam; g.sak = sak; g.sbk = sbk; g.sbn = sbn; g.sim = sim; g.sin = sin_; g.scm = scm; g.scn = scn;
  g.alpha = alpha; g.beta = beta;
  const int amode = pick_mode(A, M, K, sam, sak, 2);
  const int bmode = pick_mode(B, N, K, sbn, sbk, 2);
  const int kind = skinny_supported(g, ab_dtype, amode, bmode);
  FG_REQUIRE(kind != 0, FG_ERR_UNSUPPORTED,
             "gemm_skinny_static: not a problem of the skinny stream-K kernels (K >= 1024, 16-byte aligned A with unit "
             "K stride, B row-major or K-contiguous; 17..64 rows only with a K-contiguous B); use fg_gemm");
  const int cu = num_cus(-1);
  const size_t need = skinny_workspace_bytes(M, N, K, cu);
  FG_REQUIRE(need <= kStaticScratchBytes, FG_ERR_UNSUPPORTED,
             "gemm_skinny_static: this device (%d CUs) needs %zu bytes of scratch, the static buffer holds %zu", cu, need,
             kStaticScratchBytes);
  unsigned char* ws = nullptr;
  hipStream_t st = (hipStream_t)stream;
  const int rc = static_scratch(&ws, st);
  if (rc != FG_OK) return rc;
  // The array keeps what the last call left.  The ticket counters must read zero when the kernel starts: cleared
  // by a small kernel (a memset node would not be safe to record into a caller's graph).
  hipLaunchKernelGGL(clear_tickets_kernel, dim3(kMaxWorkers / 256), dim3(256), 0, st, (unsigned*)(ws + kTicketOffset),
                     kMaxWorkers);
  const int rc_clear = fg_check_launch("gemm_skinny_static(clear tickets)");
  if (rc_clear != FG_OK) return rc_clear;
  return skinny_launch(g, ab_dtype, kind, ws, kStaticScratchBytes, cu, st);
}

