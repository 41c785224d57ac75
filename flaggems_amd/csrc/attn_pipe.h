// Paged varlen attention forward, the lean kernel for the common case: head dim 64 or 128, page size a power of
// two >= 16, no ALiBi, no soft-cap.  Same work split (4 waves x 32 query rows, a GQA group's heads per
// workgroup), MFMA formulation (S^T = K.Q^T, O^T = V^T.P^T, MFMA 32x32x16) and swizzled LDS tiles filled by
// global_load_lds as attn_varlen_async_kernel; what differs is that nothing address-like is recomputed per
// tile on the vector ALU, and the order of work inside a wave:
//   * A wave moves 16 consecutive key rows of every tile, which lie in one page.  So the page id and the row base
//     are wave-uniform: the ids of 128 tiles sit in two registers (a lane each) and become a 64-bit scalar base;
//     each lane adds a 32-bit offset fixed for the whole kernel.  The window of 128 ids is re-read when a
//     sequence runs past it.  The last, partial tile of a sequence clamps keys per lane and looks its pages up
//     per lane; that path runs once per sequence.
//   * Stage, sub-tile and k-step offsets of every fragment read are instruction immediates on top of lane-constant
//     registers.
//
// Measured on gfx950, one wave issues a plain vector instruction every ~5 cycles and an exponential every ~9,
// and it cannot issue anything while it waits for a matrix result; a vector instruction placed between two
// MFMAs of the same wave that do not need its result costs nothing while the matrix pipe is busy (32 cycles per
// MFMA).  Running QK^T, softmax and PV of a tile one after the other leaves the matrix pipe idle through ~1200
// cycles of softmax per tile and wave, and two waves per SIMD do not mesh well enough to fill the gap.  So the
// work is cut into half tiles of 32 keys (one 32x32 score block per wave), and the softmax of half tile h is
// split in two, each part in the shadow of the MFMAs of a neighbour:
//
//   phase A of step h:  S(h+1) = K(h+1).Q^T   D/16 MFMAs  ||  P(h) = exp2(S(h)*scale - m), row sums
//   phase B of step h:  O     += V(h)^T.P(h)  D/16 MFMAs  ||  running max over S(h+1)
//   end of step h:      new reference m, and the (rare) rescale of O and the row sum.
//
// S is double-buffered in registers (16 + 16).  Fragment reads from LDS run up to four MFMAs ahead of their
// use through a small register ring, with counted waits (the loop holds no other LDS or scalar-memory
// instruction, so the LDS counter is exact).  One barrier per step.  Tiles of 64 keys still move as a whole:
// at the top of step 2t (first half of tile t) V(t-1) is no longer read and V(t+1) is requested into its
// slot; at the top of step 2t+1, K(t) is no longer read (its second half was scored in step 2t) and K(t+2)
// is requested.  Two K and two V slots: 64 KB for head dim 128, two workgroups per CU.
//
// The vector ALU's issue port is as scarce as the matrix pipe (an exponential holds it ~8 cycles,
// any other vector instruction 4, an MFMA 8): so the per-score work is one exponential, an addition, half a
// convert and half a three-way maximum, and nothing else (measured: two exponentials and three to four plain
// instructions fit behind one MFMA of the same wave; v_dot2 instructions do not, they queue behind the MFMA).  The softmax scale is folded into Q
// once (Q * scale * log2(e), rounded to the input type: an error of ~2^-9 per element of Q that averages to
// ~1e-3 in a base-2 score, well below the rounding of P itself), and the row's reference m is subtracted by
// the matrix pipe: one extra MFMA per step multiplies a fragment of ones with a fragment holding -m split in
// three 16-bit pieces, so the accumulator leaves the pipe as S*scale - m.  The reference moves only when a
// lane finds a score more than 2^8 above it (a lane-local test, no exchange on the common path); then the
// waiting scores, O and the row sum are shifted once.
//
// Every wave runs every step of its workgroup in the same form: half tiles that lie wholly outside a wave's
// mask bounds are scored and masked to -inf like the partly masked ones (P = 0 adds nothing to O) instead of
// being branched around.  Variants of the step body that merge again cost this compiler a second copy of the
// accumulators (80 registers of moves per step); the waves that would skip are not the ones the workgroup
// waits for.  The loop body is two tiles = four steps, so that ring slots and buffers are instruction immediates.
//
// RBW = query row blocks of 32 per wave.  Only RBW = 1 is built (two workgroups per CU).  With RBW = 2 every K or
// V fragment read from LDS feeds two MFMAs and the per-step costs are shared by twice the work, but the ~370
// registers mean one wave per SIMD, and this compiler then keeps the score accumulators in the AGPR half of the
// register file and moves every score to a VGPR before the vector ALU can touch it: measured 2.4 to 3.5 times
// slower, so it is not instantiated.
// This header is included by attn_varlen.hip inside its unnamed namespace.

template <int OFF> __device__ __forceinline__ u32x4 lds_read_b128_imm(uint32_t addr) {
  u32x4 v;
  asm volatile("ds_read_b128 %0, %1 offset:%2" : "=v"(v) : "v"(addr), "i"(OFF));
  return v;
}
template <int OFF> __device__ __forceinline__ u32x2 lds_read_tr_b64_imm(uint32_t addr) {
  u32x2 v;
  asm volatile("ds_read_b64_tr_b16 %0, %1 offset:%2" : "=v"(v) : "v"(addr), "i"(OFF));
  return v;
}
template <int I> struct AInt { static constexpr int value = I; };
template <int B, int E, typename F> __device__ __forceinline__ void a_static_for(F&& f) {
  if constexpr (B < E) {
    f(AInt<B>{});
    a_static_for<B + 1, E>(f);
  }
}

template <int N, typename V>
__device__ __forceinline__ void lds_wait_n(V& r) {
  asm volatile("s_waitcnt lgkmcnt(%1)" : "+v"(r) : "i"(N));
}
template <int N, typename V>
__device__ __forceinline__ void lds_wait_n2(V& r0, V& r1) {
  asm volatile("s_waitcnt lgkmcnt(%2)" : "+v"(r0), "+v"(r1) : "i"(N));
}

template <typename T, int D, int RBW>
__global__ __launch_bounds__(256, (RBW == 1 ? 2 : 1)) void attn_varlen_pipe_kernel(AttnArgs a) {
  typedef typename AttnMfma<T>::Frag Frag;
  constexpr int RB = 2 * D;            // bytes per key row in LDS
  constexpr int CPR = RB / 16;         // 16-byte chunks per row
  constexpr int KS = D / 16;           // MFMA k-steps over the head dim = fragment reads of phase A
  constexpr int DT = D / 32;           // 32-row output sub-tiles over the head dim
  constexpr int NPV = 2 * DT;          // fragment reads of phase B
  constexpr int OPB = kBN * RB;        // one operand tile
  constexpr int KPI = 1024 / RB;       // key rows per DMA instruction
  constexpr int IPW = kBN / KPI / 4;   // DMA instructions per wave, operand and tile
  constexpr int RING = KS < 4 ? KS : 4;  // fragment reads run this many slots ahead
  constexpr int kHB = kBN / 2;         // keys per half tile
  constexpr int WROWS = kRW * RBW;     // query rows per wave
  static_assert(KS == NPV && KS >= RING, "both phases read the same number of fragments");
  extern __shared__ __attribute__((aligned(16))) char lds[];  // K slot 0, K slot 1, V slot 0, V slot 1

  const FgFlashParams& p = a.p;
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int half = lane >> 5, ql = lane & 31;
  // Workgroups go to the 8 XCDs round-robin by their linear id, and every XCD has its own L2.  The id is therefore
  // re-read as (XCD, turn) and XCD k works through the k-th eighth of the (head group, sequence, row block) order:
  // all row blocks of a sequence and KV head run on one XCD, next to each other in time, so that its K and V are
  // fetched into one L2 instead of eight.  Within a sequence, long (late) row blocks first; the order is rotated
  // per (sequence, head group) so that sequences of one row block do not all start in the same turn.
  int bx = blockIdx.x, b = blockIdx.y, hgroup = blockIdx.z;
  if (a.xcd_remap) {
    const unsigned total = gridDim.x * gridDim.y * gridDim.z;
    const unsigned lin = blockIdx.x + gridDim.x * (blockIdx.y + gridDim.y * blockIdx.z);
    const unsigned per = total / 8;
    if (lin < per * 8) {  // (a ragged tail keeps its place)
      const unsigned idx = (lin % 8) * per + lin / 8;
      bx = (int)(idx % gridDim.x);
      b = (int)((idx / gridDim.x) % gridDim.y);
      hgroup = (int)(idx / (gridDim.x * gridDim.y));
    }
  }
  const int m_block = (int)((gridDim.x - 1 - bx + (unsigned)(b * 5 + hgroup * 3)) % gridDim.x);

  const int q_bos = p.cu_seqlens_q[b];
  const int q_len = p.cu_seqlens_q[b + 1] - q_bos;
  const int k_len = p.seqused_k[b];
  const int block_row0 = m_block * a.rows_per_block;
  if (block_row0 >= q_len || (a.skip_single && q_len == 1)) return;

  const int waves_per_head = 4 / a.hpb;
  const int head = hgroup * a.hpb + wave / waves_per_head;
  const int row0 = block_row0 + (wave % waves_per_head) * WROWS;
  const int kv_head = head / (p.Hq / p.Hk);

  // ---- key tiles of the workgroup: [n_min, n_max) ----------------------------------------------------------
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
  const int T_ = n_max > n_min ? n_max - n_min : 0;  // tiles of the workgroup
  const int key_base = n_min * kBN;

  // ---- Q fragments, scaled: scores leave the MFMA in base-2 units -------------------------------------------
  Frag qf[RBW][KS];
#pragma unroll
  for (int rb = 0; rb < RBW; ++rb) {
    const int qrow = row0 + rb * kRW + ql;
    const bool row_ok = qrow < q_len;
    const T* qp = (const T*)p.q + (int64_t)(q_bos + (row_ok ? qrow : 0)) * p.q_row_stride + (int64_t)head * p.q_head_stride;
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) {
      u32x4 v = {0u, 0u, 0u, 0u};
      if (row_ok) v = *reinterpret_cast<const u32x4*>(qp + ks * 16 + half * 8);
      Frag f = __builtin_bit_cast(Frag, v);
#pragma unroll
      for (int e = 0; e < 8; ++e) f[e] = (T)((float)f[e] * a.scale_log2);
      qf[rb][ks] = f;
    }
  }
  // the reference m enters the scores through the matrix pipe: ones_f (k-slots 0..2 of the lower half-wave) times
  // m_f (-m as three 16-bit pieces in the same slots of the lane that owns the row)
  Frag ones_f, m_f[RBW];
#pragma unroll
  for (int e = 0; e < 8; ++e) {
    ones_f[e] = (T)((half == 0 && e < 3) ? 1.0f : 0.0f);
#pragma unroll
    for (int rb = 0; rb < RBW; ++rb) m_f[rb][e] = (T)0.0f;
  }
  f32x16 o_acc[RBW][DT];
  float m_run[RBW], l_run[RBW];
#pragma unroll
  for (int rb = 0; rb < RBW; ++rb) {
#pragma unroll
    for (int dt = 0; dt < DT; ++dt)
#pragma unroll
      for (int e = 0; e < 16; ++e) o_acc[rb][dt][e] = 0.f;
    m_run[rb] = -INFINITY;
    l_run[rb] = 0.f;
  }

  // ---- DMA geometry (as in the lean kernel: one page id per wave and tile, kept in two registers) ------
  const int32_t* btab = p.block_table + (int64_t)b * p.block_table_stride;
  const char* kbase = (const char*)((const T*)p.k_cache + (int64_t)kv_head * p.k_head_stride);
  const char* vbase = (const char*)((const T*)p.v_cache + (int64_t)kv_head * p.v_head_stride);
  const int page_shift = a.page_shift, page_mask = p.page_size - 1;
  const int lane_key = lane / CPR, lane_pos = lane % CPR;
  // the lane's swizzled chunk offset in bytes for DMA instruction j is lane_c0 ^ (j * 16): instruction j moves the
  // keys (wave * IPW + j) * KPI + lane_key, and swz() of that differs from swz() of instruction 0's key by j
  const uint32_t lane_c0 = (uint32_t)((lane_pos ^ swz<CPR>(wave * IPW * KPI + lane_key)) * 16);
  const uint32_t lane_row_k = (uint32_t)(lane_key * (int)p.k_row_stride * 2);
  const uint32_t lane_row_v = (uint32_t)(lane_key * (int)p.v_row_stride * 2);
  // byte strides (the host admits the kernel only when they fit 31 bits)
  const uint32_t k_page_b = (uint32_t)p.k_page_stride * 2u, v_page_b = (uint32_t)p.v_page_stride * 2u;
  const uint32_t k_row_b = (uint32_t)p.k_row_stride * 2u, v_row_b = (uint32_t)p.v_row_stride * 2u;
  const uint32_t wave_key0 = (uint32_t)(wave * (IPW * KPI));
  const int last_page = k_len > 0 ? (k_len - 1) >> page_shift : 0;
  // page ids of this wave's rows in tiles pg_base + l (pg_cache0) and pg_base + 64 + l (pg_cache1), lane l
  int pg_cache0, pg_cache1, pg_base;
  auto load_page_window = [&](int first_tile) {
    pg_base = first_tile;
    int pg0 = ((n_min + first_tile + lane) * kBN + wave * (IPW * KPI)) >> page_shift;
    int pg1 = ((n_min + first_tile + 64 + lane) * kBN + wave * (IPW * KPI)) >> page_shift;
    pg0 = pg0 < last_page ? pg0 : last_page;
    pg1 = pg1 < last_page ? pg1 : last_page;
    pg_cache0 = btab[pg0];
    pg_cache1 = btab[pg1];
    // the ids are consumed here, so that the wait for them stays on this (rare) path: left pending, the compiler
    // would wait for every outstanding tile copy wherever the two paths meet again
    asm volatile("v_mov_b32 %0, %0\n\tv_mov_b32 %1, %1" : "+v"(pg_cache0), "+v"(pg_cache1));
  };
  load_page_window(0);
  // one operand tile (K: is_v = 0, V: is_v = 1) of key tile n_min + t into `slot` of its ring
  auto issue_op = [&](int t, int slot, auto is_v_c) {
    constexpr bool IS_V = decltype(is_v_c)::value != 0;
    const int nb = n_min + t;
    char* dst = lds + (IS_V ? 2 * OPB : 0) + slot * OPB + wave * (IPW * 1024);
    const char* base = IS_V ? vbase : kbase;
    const uint32_t page_b = IS_V ? v_page_b : k_page_b;
    const uint32_t row_b = IS_V ? v_row_b : k_row_b;
    if (nb * kBN + kBN <= k_len) {
      // Full tile: every key exists.  One scalar row base per tile, 32-bit scalar arithmetic but for the product
      // with the page id; instruction j lands 1024 bytes further in LDS through its immediate offset, which the
      // hardware adds to the global address as well, so the scalar step between instructions is the distance of
      // their rows less those 1024 bytes (never negative: KPI rows are at least 1024 bytes apart).
      // Tiles are requested in the order V(1), K(2), V(2), K(3), ...: a window that starts one tile below the
      // request that overran it still holds the V tile that follows.
      if (t - pg_base >= 128) load_page_window(t - 1);
      const uint32_t tl = (uint32_t)(t - pg_base);
      const uint32_t page = (uint32_t)__builtin_amdgcn_readlane(tl < 64 ? pg_cache0 : pg_cache1, (int)(tl & 63));
      const uint32_t slot_in_page = ((uint32_t)(nb * kBN) + wave_key0) & (uint32_t)page_mask;
      const char* rp = base + ((uint64_t)page * page_b + (uint64_t)(slot_in_page * row_b));
      const uint32_t step_b = (uint32_t)KPI * row_b - 1024u;
      // The copies are written as asm: scalar row base, 32-bit lane offset, immediate; M0 (the LDS address of the
      // wave's part of the slot) is set once per operand tile, with the wait state the hardware wants between a
      // scalar write of M0 and an LDS-direct load.  Through the builtin every copy costs a register move and a wait
      // state more, and on this part vector instructions are paid for in matrix-pipe time.
      {
        const uint32_t m0v = (uint32_t)(uintptr_t)FG_LDSP(dst);
        asm volatile("s_mov_b32 m0, %0\n\ts_nop 0" : : "s"(m0v) : "memory", "m0");
      }
      a_static_for<0, IPW>([&](auto jc) {
        constexpr int j = decltype(jc)::value;
        const uint32_t voff = (IS_V ? lane_row_v : lane_row_k) + (lane_c0 ^ (uint32_t)(j * 16));
        const char* rj = rp + (uint64_t)((uint32_t)j * step_b);
        asm volatile("global_load_lds_dwordx4 %0, %1 offset:%2" : : "v"(voff), "s"(rj), "n"(j * 1024) : "memory");
      });
    } else {
      // partial tile: keys past the end are clamped to the last one (their scores are masked)
#pragma unroll
      for (int j = 0; j < IPW; ++j) {
        int key = nb * kBN + (wave * IPW + j) * KPI + lane_key;
        key = key < k_len ? key : k_len - 1;
        const uint32_t page = (uint32_t)btab[key >> page_shift];
        const uint32_t slot_in_page = (uint32_t)key & (uint32_t)page_mask;
        uint32_t c0 = lane_c0;
        asm volatile("" : "+v"(c0));
        const char* rp = base + ((uint64_t)page * page_b + (uint64_t)(slot_in_page * row_b + (c0 ^ (uint32_t)(j * 16))));
        __builtin_amdgcn_global_load_lds(FG_GLBP(rp), FG_LDSP(dst + j * 1024), 16, 0, 0);
      }
    }
  };

  // ---- fragment addresses: lane-constant registers, everything else is an immediate ---------------------
  const uint32_t lds0 = lds_off(lds);
  const int k_row = sigma(ql);
  const int kx = half ^ swz<CPR>(k_row);
  uint32_t k_addr[KS];
#pragma unroll
  for (int ks = 0; ks < KS; ++ks) k_addr[ks] = lds0 + k_row * RB + (((ks * 2) ^ kx) * 16);
  const int vs = lane & 15;
  const int v_key0 = half * 8 + (vs >> 2);
  const int v_cc = 2 * ((lane >> 4) & 1) + ((vs & 3) >> 1);
  const int v_byte = (vs & 1) * 8;
  const int vx0 = v_cc ^ swz<CPR>(v_key0), vx1 = v_cc ^ swz<CPR>(v_key0 + 4);
  uint32_t v_addr0[DT], v_addr1[DT];
#pragma unroll
  for (int dt = 0; dt < DT; ++dt) {
    v_addr0[dt] = lds0 + 2 * OPB + v_key0 * RB + v_byte + (((dt * 4) ^ vx0) * 16);
    v_addr1[dt] = lds0 + 2 * OPB + (v_key0 + 4) * RB + v_byte + (((dt * 4) ^ vx1) * 16);
  }

  // visible keys of this lane's rows, relative to the first key of the workgroup and the lane's half: [col_lo, col_hi]
  int col_hi[RBW], col_lo[RBW];
#pragma unroll
  for (int rb = 0; rb < RBW; ++rb) {
    const int qrow = row0 + rb * kRW + ql;
    col_hi[rb] = (a.has_right ? (qrow + shift + a.right_off_w < k_len - 1 ? qrow + shift + a.right_off_w : k_len - 1)
                              : k_len - 1) - key_base - half * 8;
    col_lo[rb] = (a.has_left ? qrow + shift - a.left_off_w : 0) - key_base - half * 8;
  }

  f32x16 s_buf[RBW][2];   // S(h) in buffer h & 1
  Frag pf[RBW][2];        // P(h) as the B operand of the PV MFMAs (2 x 16 keys)
  float psum[RBW];
  float tmax_a[RBW], tmax_b[RBW];
  u32x4 kring[RING];
  u32x2 vring[RING][2];

  // fragment read for slot `i` of phase A (key sub-tile KT of K slot SK) or of phase B (the keys of sub-tile KT in
  // V slot SV)
  auto read_k = [&](auto i_c, auto sk_c, auto kt_c) {
    constexpr int i = decltype(i_c)::value, SK = decltype(sk_c)::value, KT = decltype(kt_c)::value;
    kring[i % RING] = lds_read_b128_imm<SK * OPB + KT * 32 * RB>(k_addr[i]);
  };
  auto read_v = [&](auto i_c, auto sv_c, auto kt_c) {
    constexpr int i = decltype(i_c)::value, SV = decltype(sv_c)::value, KT = decltype(kt_c)::value;
    constexpr int dt = (i / 2) % DT, t4 = KT * 2 + i % 2;
    vring[i % RING][0] = lds_read_tr_b64_imm<SV * OPB + t4 * 16 * RB>(v_addr0[dt]);
    vring[i % RING][1] = lds_read_tr_b64_imm<SV * OPB + t4 * 16 * RB>(v_addr1[dt]);
  };

  // Phase A of the step whose scores S(h) sit in buffer CUR.  QK: S(h+1) = K.Q^T - m -> buffer CUR^1, from key
  // sub-tile CUR^1 of K slot SK.  EXP: P(h) = exp2(S(h)) and its row sum; the last RING slots then start the V
  // fragment reads of the phase B that follows (V slot SV).  Per slot: one K fragment, one MFMA and one score pair
  // per row block.
  auto phase_a = [&](auto cur_c, auto sk_c, auto sv_c, auto qk_c, auto exp_c) {
    constexpr int CUR = decltype(cur_c)::value;
    constexpr bool QK = decltype(qk_c)::value != 0, EXP = decltype(exp_c)::value != 0;
    constexpr bool PRE_V = EXP;
    constexpr int NXT = CUR ^ 1;
    if constexpr (QK) {
      a_static_for<0, RING>([&](auto ic) { read_k(ic, sk_c, AInt<NXT>{}); });
#pragma unroll
      for (int rb = 0; rb < RBW; ++rb) {
#pragma unroll
        for (int e = 0; e < 16; ++e) s_buf[rb][NXT][e] = 0.f;
        s_buf[rb][NXT] = AttnMfma<T>::mma(ones_f, m_f[rb], s_buf[rb][NXT]);  // -m, while the first K fragments arrive
      }
    }
    if constexpr (EXP) {
#pragma unroll
      for (int rb = 0; rb < RBW; ++rb) psum[rb] = 0.f;
    }
    a_static_for<0, KS>([&](auto ic) {
      constexpr int i = decltype(ic)::value;
      if constexpr (QK) {
        // LDS operations younger than read i at this point: those issued in the RING - 1 slots before this one
        constexpr int y1 = (RING > 1) ? ((i + 1 < KS) ? 1 : (PRE_V ? 2 : 0)) : 0;
        constexpr int y2 = (RING > 2) ? ((i + 2 < KS) ? 1 : (PRE_V ? 2 : 0)) : 0;
        constexpr int y3 = (RING > 3) ? ((i + 3 < KS) ? 1 : (PRE_V ? 2 : 0)) : 0;
        lds_wait_n<y1 + y2 + y3>(kring[i % RING]);
      }
      a_static_for<0, RBW>([&](auto rc) {
        constexpr int rb = decltype(rc)::value;
        if constexpr (QK)
          s_buf[rb][NXT] = AttnMfma<T>::mma(__builtin_bit_cast(Frag, kring[i % RING]), qf[rb][i], s_buf[rb][NXT]);
        if constexpr (rb == RBW - 1) {
          if constexpr (QK && i + RING < KS) read_k(AInt<i + RING>{}, sk_c, AInt<NXT>{});
          else if constexpr (PRE_V && i + RING >= KS) read_v(AInt<i + RING - KS>{}, sv_c, cur_c);
        }
        if constexpr (EXP) {
          // 8 score pairs over KS slots: elements 2w, 2w+1 of half t2 -> word w of pf[t2]
          constexpr int per = 8 / KS > 0 ? 8 / KS : 1;
          a_static_for<0, per>([&](auto jc) {
            constexpr int pi = i * per + decltype(jc)::value;
            if constexpr (pi < 8) {
              constexpr int t2 = pi / 4, w = pi % 4;
              const float p0 = __builtin_amdgcn_exp2f(s_buf[rb][CUR][t2 * 8 + 2 * w]);
              const float p1 = __builtin_amdgcn_exp2f(s_buf[rb][CUR][t2 * 8 + 2 * w + 1]);
              typedef T T2 __attribute__((ext_vector_type(2)));
              const T2 pk = {(T)p0, (T)p1};
              psum[rb] += p0 + p1;  // (dot-product instructions would halve this, but they wait for the matrix pipe)
              u32x4 words = __builtin_bit_cast(u32x4, pf[rb][t2]);
              words[w] = __builtin_bit_cast(uint32_t, pk);
              pf[rb][t2] = __builtin_bit_cast(Frag, words);
            }
          });
        }
        __builtin_amdgcn_sched_barrier(0);
      });
    });
    if constexpr (EXP) {
#pragma unroll
      for (int rb = 0; rb < RBW; ++rb) l_run[rb] += xhalf_sum(psum[rb]);
    }
  };

  // Phase B.  PV: O += V(keys of sub-tile CUR of V slot SV)^T.P (the first RING fragment pairs were requested by
  // phase A).  MAX: the lane's maximum over S(h+1) in buffer CUR^1 (redone by mask_and_max where the half tile
  // needs a mask); it starts two slots into the phase, when the last scores have left the matrix pipe.
  auto phase_b = [&](auto cur_c, auto sv_c, auto max_c) {
    constexpr int CUR = decltype(cur_c)::value;
    constexpr bool MAX = decltype(max_c)::value != 0;
    constexpr int NXT = CUR ^ 1;
    if constexpr (MAX) {
#pragma unroll
      for (int rb = 0; rb < RBW; ++rb) tmax_a[rb] = tmax_b[rb] = -INFINITY;
    }
    a_static_for<0, NPV>([&](auto ic) {
      constexpr int i = decltype(ic)::value;
      constexpr int ahead = (i + RING - 1 < NPV) ? RING - 1 : (NPV - 1 - i);
      lds_wait_n2<2 * ahead>(vring[i % RING][0], vring[i % RING][1]);
      const u32x4 both = {vring[i % RING][0][0], vring[i % RING][0][1], vring[i % RING][1][0], vring[i % RING][1][1]};
      a_static_for<0, RBW>([&](auto rc) {
        constexpr int rb = decltype(rc)::value;
        o_acc[rb][i / 2] = AttnMfma<T>::mma(__builtin_bit_cast(Frag, both), pf[rb][i % 2], o_acc[rb][i / 2]);
        if constexpr (rb == RBW - 1 && i + RING < NPV) read_v(AInt<i + RING>{}, sv_c, cur_c);
        if constexpr (MAX && i >= 2) {
          // the 8 score pairs over the slots from the third on
          constexpr int per = (8 + NPV - 3) / (NPV - 2);
          a_static_for<0, per>([&](auto jc) {
            constexpr int pi = (i - 2) * per + decltype(jc)::value;
            if constexpr (pi < 8) {
              if constexpr (pi % 2 == 0)
                tmax_a[rb] = fmaxf(fmaxf(tmax_a[rb], s_buf[rb][NXT][2 * pi]), s_buf[rb][NXT][2 * pi + 1]);
              else
                tmax_b[rb] = fmaxf(fmaxf(tmax_b[rb], s_buf[rb][NXT][2 * pi]), s_buf[rb][NXT][2 * pi + 1]);
            }
          });
          if constexpr (i == NPV - 1) asm volatile("" : "+v"(tmax_a[rb]), "+v"(tmax_b[rb]));  // keeps the maxima in their slots
        }
        __builtin_amdgcn_sched_barrier(0);
      });
    });
  };

  // masks on the scores of half tile h of row block RBI (in buffer BUF), then their maximum (diagonal, window edge
  // and last tiles)
  auto mask_and_max = [&](int h, auto rb_c, auto buf_c) {
    constexpr int BUF = decltype(buf_c)::value, rb = decltype(rb_c)::value;
    // element e is key key_base + h*32 + half*8 + (e>>3)*16 + (e&7)
    const int hi_rel = col_hi[rb] - h * kHB, lo_rel = col_lo[rb] - h * kHB;
    float tm = -INFINITY;
#pragma unroll
    for (int e = 0; e < 16; ++e) {
      const int rel = (e >> 3) * 16 + (e & 7);
      float s = s_buf[rb][BUF][e];
      s = rel > hi_rel ? -INFINITY : s;
      if (a.has_left) s = rel < lo_rel ? -INFINITY : s;
      s_buf[rb][BUF][e] = s;
      tm = fmaxf(tm, s);
    }
    tmax_a[rb] = tm;
    tmax_b[rb] = -INFINITY;
  };
  // half tile h of row block rb needs the mask pass from mask_from[rb] on (diagonal, right window edge, partial
  // last tile) and below mask_below[rb] (left window edge)
  int mask_from[RBW], mask_below[RBW];
#pragma unroll
  for (int rb = 0; rb < RBW; ++rb) {
    const int r_first = row0 + rb * kRW;
    const int r_last = (r_first + kRW - 1 < q_len ? r_first + kRW - 1 : q_len - 1);
    // key0 + 32 > k_len  <=>  h > (k_len - key_base - 32) / 32 ;  key0 + 31 > bound  <=>  h > (bound - 31 - key_base) / 32
    int from = (k_len - key_base - kHB) < 0 ? 0 : (k_len - key_base - kHB) / kHB + 1;
    if (a.has_right) {
      const int bnd = r_first + shift + a.right_off_w - (kHB - 1) - key_base;
      const int f2 = bnd < 0 ? 0 : bnd / kHB + 1;
      from = from < f2 ? from : f2;
    }
    mask_from[rb] = from;
    // key0 < r_last + shift - left  <=>  h < ceil((r_last + shift - left - key_base) / 32)
    const int lb = r_last + shift - a.left_off_w - key_base;
    mask_below[rb] = a.has_left ? (lb <= 0 ? 0 : (lb + kHB - 1) / kHB) : 0;
  }
  auto needs_mask = [&](int h, int rb) { return h >= mask_from[rb] || h < mask_below[rb]; };
  // The scores in buffer BUF are relative to the reference m_run they were scored with.  Where a lane finds one
  // more than 2^8 above it (or the row has no reference yet and sees its first key), the row's reference moves to
  // the new maximum: the waiting scores, O and the row sum are shifted by the difference and -m is split anew.
  // Any reference gives the same result as long as P and the running sum use the same one.
  auto new_reference = [&](auto buf_c) {
    constexpr int BUF = decltype(buf_c)::value;
    float tl[RBW];
    bool any = false;
#pragma unroll
    for (int rb = 0; rb < RBW; ++rb) {
      tl[rb] = fmaxf(tmax_a[rb], tmax_b[rb]);
      any = any || tl[rb] > 8.0f || (m_run[rb] == -INFINITY && tl[rb] > -INFINITY);
    }
    if (__builtin_amdgcn_ballot_w64(any) == 0) return;
    a_static_for<0, RBW>([&](auto rc) {
      constexpr int rb = decltype(rc)::value;
      const bool fresh = m_run[rb] == -INFINITY;
      const float tmax = xhalf_max(tl[rb]);
      const bool moved = tmax > 8.0f || (fresh && tmax > -INFINITY);
      if (__builtin_amdgcn_ballot_w64(moved) == 0) return;
      const float delta = moved ? tmax : 0.f;
      const float alpha = __builtin_amdgcn_exp2f(-delta);
#pragma unroll
      for (int e = 0; e < 16; ++e) s_buf[rb][BUF][e] -= delta;
#pragma unroll
      for (int dt = 0; dt < DT; ++dt)
#pragma unroll
        for (int e = 0; e < 16; ++e) o_acc[rb][dt][e] *= alpha;
      l_run[rb] *= alpha;
      if (moved) m_run[rb] = (fresh ? 0.f : m_run[rb]) + delta;
      // -m_run as three pieces of the input type (their sum is exact to ~2^-24 of m), in k-slots 0..2 of the lane
      // of the lower half-wave that owns the row
      const float mm = (m_run[rb] == -INFINITY || half != 0) ? 0.f : -m_run[rb];
      const T hi = (T)mm;
      const float r1 = mm - (float)hi;
      const T mid = (T)r1;
      const T lo = (T)(r1 - (float)mid);
      m_f[rb][0] = hi;
      m_f[rb][1] = mid;
      m_f[rb][2] = lo;
    });
  };
  auto mask_where_needed = [&](int h, auto buf_c) {
    a_static_for<0, RBW>([&](auto rc) {
      if (needs_mask(h, decltype(rc)::value)) mask_and_max(h, rc, buf_c);
    });
  };

  // Step h = 2t + KT of a tile t of parity PAR: S(h) sits in buffer KT, V(t) in V slot PAR; S(h+1) comes from the
  // second half of K(t) (KT = 0: K slot PAR) or the first half of K(t+1) (KT = 1: K slot PAR^1).  LAST: the final
  // step of the workgroup, which has no S(h+1) to score.
  auto step = [&](int t, auto par_c, auto kt_c, auto last_c) {
    constexpr int PAR = decltype(par_c)::value, KT = decltype(kt_c)::value;
    constexpr bool LAST = decltype(last_c)::value != 0;
    constexpr int SK = KT == 0 ? PAR : (PAR ^ 1);
    const int h = 2 * t + KT;
    // landed: V(t) (KT = 0) or K(t+1) (KT = 1); the request behind it, K(t+1) resp. V(t+1), exists iff t+1 < T_
    if (t + 1 < T_) FG_WAIT_VM(IPW);
    else FG_WAIT_VM(0);
    __builtin_amdgcn_s_barrier();
    if constexpr (KT == 0) {
      if (t + 1 < T_) issue_op(t + 1, PAR ^ 1, AInt<1>{});  // V(t-1) is no longer read
    } else {
      if (t + 2 < T_) issue_op(t + 2, PAR, AInt<0>{});      // K(t) is no longer read
    }
    if constexpr (!LAST) {
      phase_a(kt_c, AInt<SK>{}, par_c, AInt<1>{}, AInt<1>{});
      phase_b(kt_c, par_c, AInt<1>{});
      mask_where_needed(h + 1, AInt<KT ^ 1>{});
      new_reference(AInt<KT ^ 1>{});
    } else {
      phase_a(kt_c, AInt<SK>{}, par_c, AInt<0>{}, AInt<1>{});
      phase_b(kt_c, par_c, AInt<0>{});
    }
  };

  if (T_ > 0) {
    issue_op(0, 0, AInt<0>{});
    issue_op(0, 0, AInt<1>{});
    if (1 < T_) issue_op(1, 1, AInt<0>{});
    // "step -1": K(0) has landed; S(0) is scored on its own (into buffer 0, from the first half of K slot 0)
    if (1 < T_) FG_WAIT_VM(2 * IPW);
    else FG_WAIT_VM(IPW);
    __builtin_amdgcn_s_barrier();
    phase_a(AInt<1>{}, AInt<0>{}, AInt<0>{}, AInt<1>{}, AInt<0>{});
    a_static_for<0, RBW>([&](auto rc) { mask_and_max(0, rc, AInt<0>{}); });
    new_reference(AInt<0>{});
    // every step but the last, two tiles per trip
    int t = 0;
    for (; t + 2 < T_; t += 2) {
      step(t, AInt<0>{}, AInt<0>{}, AInt<0>{});
      step(t, AInt<0>{}, AInt<1>{}, AInt<0>{});
      step(t + 1, AInt<1>{}, AInt<0>{}, AInt<0>{});
      step(t + 1, AInt<1>{}, AInt<1>{}, AInt<0>{});
    }
    if (t + 2 == T_) {
      step(t, AInt<0>{}, AInt<0>{}, AInt<0>{});
      step(t, AInt<0>{}, AInt<1>{}, AInt<0>{});
      step(t + 1, AInt<1>{}, AInt<0>{}, AInt<0>{});
      step(t + 1, AInt<1>{}, AInt<1>{}, AInt<1>{});
    } else {
      step(t, AInt<0>{}, AInt<0>{}, AInt<0>{});
      step(t, AInt<0>{}, AInt<1>{}, AInt<1>{});
    }
  }

  // ---- epilogue --------------------------------------------------------------------------------------
#pragma unroll
  for (int rb = 0; rb < RBW; ++rb) {
    const int qrow = row0 + rb * kRW + ql;
    if (qrow >= q_len) continue;
    const bool empty = l_run[rb] == 0.f || l_run[rb] != l_run[rb];
    const float inv = empty ? 1.f : 1.f / l_run[rb];
    if (p.lse != nullptr && half == 0) {
      p.lse[(int64_t)head * p.total_q + q_bos + qrow] = empty ? INFINITY : m_run[rb] * 0.6931471805599453f + logf(l_run[rb]);
    }
    T* op = (T*)p.out + (int64_t)(q_bos + qrow) * p.o_row_stride + (int64_t)head * p.o_head_stride;
#pragma unroll
    for (int dt = 0; dt < DT; ++dt)
#pragma unroll
      for (int g = 0; g < 4; ++g) {
        const int d = dt * 32 + g * 8 + half * 4;
        Pack<T, 4> o;
#pragma unroll
        for (int e = 0; e < 4; ++e) o.v[e] = (T)(o_acc[rb][dt][g * 4 + e] * inv);
        st_pack<T, 4>(op + d, o);
      }
  }
}

template <typename T, int D, int RBW>
int launch_pipe(const AttnArgs& a, dim3 grid, hipStream_t st) {
  constexpr int LDS_BYTES = 2 * 2 * kBN * 2 * D;
  static hipError_t attr_err = hipFuncSetAttribute(reinterpret_cast<const void*>(attn_varlen_pipe_kernel<T, D, RBW>),
                                                   hipFuncAttributeMaxDynamicSharedMemorySize, LDS_BYTES);
  if (attr_err != hipSuccess) {
    fg_set_error("flash_attn_varlen_fwd: cannot reserve %d bytes of LDS: %s", LDS_BYTES, hipGetErrorString(attr_err));
    return FG_ERR_LAUNCH;
  }
  hipLaunchKernelGGL((attn_varlen_pipe_kernel<T, D, RBW>), grid, dim3(256), LDS_BYTES, st, a);
  return fg_check_launch("flash_attn_varlen_fwd");
}
