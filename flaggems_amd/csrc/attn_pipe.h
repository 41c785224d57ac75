// Paged varlen attention forward, the lean kernel for the common case: head dim 64 or 128, page size a power of
// two >= 16, no ALiBi, no soft-cap.  Same work split (4 waves x 32 query rows, a GQA group's heads per workgroup)
// and swizzled LDS tiles filled by global_load_lds as attn_varlen_async_kernel; what differs:
//   * A wave moves 16 consecutive key rows of every tile, which lie in one page.  So the page id and the row base
//     are wave-uniform: the ids of 128 tiles sit in two registers (a lane each) and become a 64-bit scalar base;
//     each lane adds a 32-bit offset fixed for the whole kernel.  The window of 128 ids is re-read when a
//     sequence runs past it.  The last, partial tile of a sequence clamps keys per lane and looks its pages up
//     per lane; that path runs once per sequence.
//   * Stage, sub-tile and k-step offsets of every fragment read are instruction immediates on top of lane-constant
//     registers.
//   * The matrix instruction is MFMA 16x16x32 (below), and the work inside a wave is software-pipelined.
//
// Measured on gfx950, one wave issues a plain vector instruction every ~5 cycles and an exponential every ~9,
// and it cannot issue anything while it waits for a matrix result; a vector instruction placed between two
// MFMAs of the same wave that do not need its result costs little while the matrix pipe is busy.  Running QK^T,
// softmax and PV of a tile one after the other leaves the matrix pipe idle through the softmax, and two waves per
// SIMD do not mesh well enough to fill the gap.  So the work is cut into half tiles of 32 keys, and the softmax of
// half tile h is split in two, each part in the shadow of the MFMAs of a neighbour:
//
//   phase A of step h:  S(h+1) = K(h+1).Q^T - m   D/8 MFMAs  ||  P(h) = exp2(S(h)), row sums
//   phase B of step h:  O     += V(h)^T.P(h)      D/8 MFMAs  ||  running max over S(h+1)
//   end of step h:      new reference m, and the (rare) rescale of O and the row sum.
//
// S is double-buffered in registers (16 + 16).  Fragment reads from LDS run up to four slots ahead of their
// use through a small register ring, with counted waits (the loop holds no other LDS or scalar-memory
// instruction, so the LDS counter is exact).  One barrier per step.  Tiles of 64 keys still move as a whole:
// at the top of step 2t (first half of tile t) V(t-1) is no longer read and V(t+1) is requested into its
// slot; at the top of step 2t+1, K(t) is no longer read (its second half was scored in step 2t) and K(t+2)
// is requested.  Two K and two V slots: 64 KB for head dim 128, two workgroups per CU.
//
// The vector ALU's issue port is as scarce as the matrix pipe: the per-score work is one exponential, an addition,
// half a convert and half a three-way maximum, and nothing else (v_dot2 instructions would halve the additions but
// queue behind the MFMAs).  The softmax scale is folded into Q once (Q * scale * log2(e), rounded to the input
// type: an error of ~2^-9 per element of Q that averages to ~1e-3 in a base-2 score, well below the rounding of P
// itself).
//
// Every wave runs every step of its workgroup in the same form: half tiles that lie wholly outside a wave's
// mask bounds are scored and masked to -inf like the partly masked ones (P = 0 adds nothing to O) instead of
// being branched around.  Variants of the step body that merge again cost this compiler a second copy of the
// accumulators; the waves that would skip are not the ones the workgroup waits for.  The loop body is two tiles =
// four steps, so that ring slots and buffers are instruction immediates.
//
// The same kernel on MFMA 32x32x16 (a lane owning one query row and 16 keys of a half tile, the reference subtracted
// by a ninth MFMA of ones x -m split in three 16-bit pieces) ran 2-4 % slower: with the 16-cycle instruction the
// vector instructions of the neighbouring wave find twice as many gaps to issue into.
//
// Lane l = (g = l / 16, c = l % 16).  A wave's 32 query rows are two column tiles (QT = 0, 1) of 16; a half tile
// of 32 keys is two row tiles (KT2 = 0, 1) of 16.
//   S^T[key, q] = K . Q^T      per (KT2, QT): D/32 MFMAs.  A = K rows from LDS: lane (g, c) reads 16 bytes of the
//                              key in row slot c (8 head-dim elements 32 kk + 8 g ...), one ds_read_b128 feeding
//                              both QT.  B = Q from registers.  The accumulator of lane (g, c) holds column
//                              q = 16 QT + c and the row slots 4 g + r, r = 0..3.
//   O^T[d, q] += V^T . P^T     per (16 head-dim rows, QT): ONE MFMA over the 32 keys of the half tile.  Its k slot
//                              8 g + t belongs to lane group g: t = 0..3 are the lane's four scores of KT2 = 0,
//                              t = 4..7 those of KT2 = 1, so P^T is the exponentials of the S^T accumulators in
//                              register order and no data moves between the two products.  A = V^T: two
//                              ds_read_b64_tr_b16 (4 keys x 16 head-dim elements per group of 16 lanes each), the
//                              keys of the lane's own row slots in KT2 = 0 and 1.
// Row slot 4 x + r of a 16-key tile holds key 4 pi(x) + r, with pi chosen per LDS row length so that both kinds of
// fragment read are free of bank conflicts under the tile swizzle (checked with SQ_LDS_BANK_CONFLICT on the bare
// access patterns).  The hardware serves a ds_read_b128 sixteen lanes at a time, and not consecutive ones: lanes
// 0-3, 12-15, 20-23, 24-27 go together (and the three translates of that set by 4, 32 and 36), so a K fragment
// read puts row slots 0-3 and 12-15 of chunk g next to slots 4-11 of chunk g ^ 1; a ds_read_b64_tr_b16 serves
// lanes 0-31 together, i.e. the key quadruples of lane groups 0 and 1.  Rows of 256 bytes: pi = 0, 2, 3, 1; rows of
// 128 bytes: pi = 0, 1, 3, 2.
// The softmax reference m enters the scores as the C operand of the first MFMA of every accumulation (a register
// quadruple holding -m, exact in fp32), so the vector ALU runs exp2(s) on what the matrix pipe delivers.  A lane
// owns a quarter of the keys of its two rows: maxima are tested lane-locally (the reference moves only when a lane
// sees a score more than 2^8 above it), row sums stay per lane and are added across the four lane groups once, in
// the epilogue.
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

// sum / maximum over the four lanes c, c + 16, c + 32, c + 48 (every one of them receives the result)
__device__ __forceinline__ void xrow16_split(float v, float& a, float& b) {
  a = v;
  b = v;
  asm volatile("s_nop 1\n\tv_permlane16_swap_b32 %0, %1\n\ts_nop 1" : "+v"(a), "+v"(b));
}
__device__ __forceinline__ float xquad_sum(float v) {
  float a, b;
  xrow16_split(v, a, b);
  return xhalf_sum(a + b);
}
__device__ __forceinline__ float xquad_max(float v) {
  float a, b;
  xrow16_split(v, a, b);
  return xhalf_max(fmaxf(a, b));
}

template <typename T, int D>
__global__ __launch_bounds__(256, 2) void attn_varlen_pipe_kernel(AttnArgs a) {
  typedef typename AttnMfma<T>::Frag Frag;
  constexpr int RB = 2 * D;            // bytes per key row in LDS
  constexpr int CPR = RB / 16;         // 16-byte chunks per row
  constexpr int KK = D / 32;           // MFMA k-steps over the head dim
  constexpr int KS = 2 * KK;           // K fragment reads (= slots) of phase A: (KT2, kk)
  constexpr int NPV = D / 16;          // V fragment pairs (= slots) of phase B: 16 head-dim rows each
  constexpr int OPB = kBN * RB;        // one operand tile
  constexpr int KPI = 1024 / RB;       // key rows per DMA instruction
  constexpr int IPW = kBN / KPI / 4;   // DMA instructions per wave, operand and tile
  constexpr int RING = KS < 4 ? KS : 4;  // fragment reads run this many slots ahead
  constexpr int kHB = kBN / 2;         // keys per half tile
  constexpr int QT = 2;                // column tiles of 16 query rows per wave
  static_assert(KS == NPV && KS >= RING, "both phases read the same number of fragments");
  extern __shared__ __attribute__((aligned(16))) char lds[];  // K slot 0, K slot 1, V slot 0, V slot 1

  const FgFlashParams& p = a.p;
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int g = lane >> 4, c = lane & 15;
  // Row slots 4 x .. 4 x + 3 of a 16-key tile hold keys 4 pi(x) .. 4 pi(x) + 3 (see the header); pig = pi(g)
  auto pi_of = [](int x) { return CPR >= 16 ? ((0x1320 >> (4 * x)) & 3) : ((0x2310 >> (4 * x)) & 3); };
  const int pig = pi_of(g);
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
    if (lin < per * 8) {
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
  const int row0 = block_row0 + (wave % waves_per_head) * kRW;
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
  Frag qf[QT][KK];
#pragma unroll
  for (int qt = 0; qt < QT; ++qt) {
    const int qrow = row0 + qt * 16 + c;
    const bool row_ok = qrow < q_len;
    const T* qp = (const T*)p.q + (int64_t)(q_bos + (row_ok ? qrow : 0)) * p.q_row_stride + (int64_t)head * p.q_head_stride;
#pragma unroll
    for (int kk = 0; kk < KK; ++kk) {
      // Variant FG_V_ATTN_Q_UNCOND (variants.h; off: each load under the row check).  Unconditional: rows past the
      // end read row 0 of the sequence (qp is clamped) and are zeroed afterwards; a branch around each load makes the
      // compiler wait for one before it requests the next
      u32x4 v = {0u, 0u, 0u, 0u};
      if constexpr (FG_V_ATTN_Q_UNCOND != 0) {
        v = *reinterpret_cast<const u32x4*>(qp + kk * 32 + g * 8);
        if (!row_ok) v = u32x4{0u, 0u, 0u, 0u};
      } else {
        if (row_ok) v = *reinterpret_cast<const u32x4*>(qp + kk * 32 + g * 8);
      }
      Frag f = __builtin_bit_cast(Frag, v);
#pragma unroll
      for (int e = 0; e < 8; ++e) f[e] = (T)((float)f[e] * a.scale_log2);
      qf[qt][kk] = f;
    }
    // (with the variant) the conversions of the two column tiles are not interleaved: scheduled freely, the register
    // allocator put the reload of a spilled register in front of the first barrier, and with it a wait for every copy
    // in flight
    if constexpr (FG_V_ATTN_Q_UNCOND != 0) __builtin_amdgcn_sched_barrier(0);
  }
  f32x4 minit[QT];          // -m of the lane's row, four times: C operand of the first MFMA of a score tile
  f32x4 o_acc[QT][NPV];
  float m_run[QT], l_run[QT];
  // Variant FG_V_ATTN_ROWSUM_MFMA (variants.h): the row sums come from the matrix pipe.  One more MFMA per column
  // tile and half-tile step multiplies a fragment of ones with P^T, exactly the B operand of the PV products: every
  // element of its 16 x 16 result in column q is the sum over the 32 keys of P[key][q], so each lane holds the WHOLE
  // row sum of its column (four times), summed from the P values as rounded for the PV product.  It replaces sixteen
  // vector additions per step, on a kernel whose vector ALU is as busy as its matrix pipe.
  // Head dim 128 only: at head dim 64 the eight extra accumulator registers take the kernel from three waves per
  // SIMD to two.
  constexpr bool ROWSUM_MFMA = FG_V_ATTN_ROWSUM_MFMA != 0 && D == 128;
  f32x4 l_acc[ROWSUM_MFMA ? QT : 1];
  Frag ones;
#pragma unroll
  for (int e = 0; e < 8; ++e) ones[e] = (T)1.0f;
#pragma unroll
  for (int qt = 0; qt < QT; ++qt) {
    minit[qt] = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int dt = 0; dt < NPV; ++dt) o_acc[qt][dt] = f32x4{0.f, 0.f, 0.f, 0.f};
    m_run[qt] = -INFINITY;
    l_run[qt] = 0.f;   // the lane's share of the row sum
    if constexpr (ROWSUM_MFMA) l_acc[qt] = f32x4{0.f, 0.f, 0.f, 0.f};
  }

  // ---- DMA geometry: one page id per wave and tile, kept in two registers ------------------------------
  const int32_t* btab = p.block_table + (int64_t)b * p.block_table_stride;
  const char* kbase = (const char*)((const T*)p.k_cache + (int64_t)kv_head * p.k_head_stride);
  const char* vbase = (const char*)((const T*)p.v_cache + (int64_t)kv_head * p.v_head_stride);
  const int page_shift = a.page_shift, page_mask = p.page_size - 1;
  const int lane_key = lane / CPR, lane_pos = lane % CPR;
  const uint32_t lane_c0 = (uint32_t)((lane_pos ^ swz<CPR>(wave * IPW * KPI + lane_key)) * 16);
  const uint32_t lane_row_k = (uint32_t)(lane_key * (int)p.k_row_stride * 2);
  const uint32_t lane_row_v = (uint32_t)(lane_key * (int)p.v_row_stride * 2);
  const uint32_t k_page_b = (uint32_t)p.k_page_stride * 2u, v_page_b = (uint32_t)p.v_page_stride * 2u;
  const uint32_t k_row_b = (uint32_t)p.k_row_stride * 2u, v_row_b = (uint32_t)p.v_row_stride * 2u;
  const uint32_t wave_key0 = (uint32_t)(wave * (IPW * KPI));
  const int last_page = k_len > 0 ? (k_len - 1) >> page_shift : 0;
  int pg_cache0, pg_cache1, pg_base;
  auto load_page_window = [&](int first_tile) {
    pg_base = first_tile;
    int pg0 = ((n_min + first_tile + lane) * kBN + wave * (IPW * KPI)) >> page_shift;
    int pg1 = ((n_min + first_tile + 64 + lane) * kBN + wave * (IPW * KPI)) >> page_shift;
    pg0 = pg0 < last_page ? pg0 : last_page;
    pg1 = pg1 < last_page ? pg1 : last_page;
    pg_cache0 = btab[pg0];
    pg_cache1 = btab[pg1];
    asm volatile("v_mov_b32 %0, %0\n\tv_mov_b32 %1, %1" : "+v"(pg_cache0), "+v"(pg_cache1));
  };
  load_page_window(0);
  auto issue_op = [&](int t, int slot, auto is_v_c) {
    constexpr bool IS_V = decltype(is_v_c)::value != 0;
    const int nb = n_min + t;
    char* dst = lds + (IS_V ? 2 * OPB : 0) + slot * OPB + wave * (IPW * 1024);
    const char* base = IS_V ? vbase : kbase;
    const uint32_t page_b = IS_V ? v_page_b : k_page_b;
    const uint32_t row_b = IS_V ? v_row_b : k_row_b;
    if (nb * kBN + kBN <= k_len) {
      if (t - pg_base >= 128) load_page_window(t - 1);
      const uint32_t tl = (uint32_t)(t - pg_base);
      const uint32_t page = (uint32_t)__builtin_amdgcn_readlane(tl < 64 ? pg_cache0 : pg_cache1, (int)(tl & 63));
      const uint32_t slot_in_page = ((uint32_t)(nb * kBN) + wave_key0) & (uint32_t)page_mask;
      const char* rp = base + ((uint64_t)page * page_b + (uint64_t)(slot_in_page * row_b));
      const uint32_t step_b = (uint32_t)KPI * row_b - 1024u;
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
  // K: row slot c of a 16-key tile = key 4 pi(c / 4) + c % 4; chunk kk * 4 + g of that row
  const int k_row = 4 * pi_of(c >> 2) + (c & 3);
  uint32_t k_addr[KK];
#pragma unroll
  for (int kk = 0; kk < KK; ++kk) k_addr[kk] = lds0 + k_row * RB + (((kk * 4 + g) ^ swz<CPR>(k_row)) * 16);
  // V: the 16 lanes of group g address keys 4 pi(g) + c / 4, 32 bytes of each (16 head-dim elements), 8 bytes a lane
  const int v_key = 4 * pig + (c >> 2);
  const int v_byte = (c & 1) * 8;
  const int v_cb = (c & 3) >> 1;
  uint32_t v_addr[NPV];
#pragma unroll
  for (int dt = 0; dt < NPV; ++dt) v_addr[dt] = lds0 + 2 * OPB + v_key * RB + v_byte + (((dt * 2 + v_cb) ^ swz<CPR>(v_key)) * 16);

  // visible keys of this lane's rows, relative to the first key of the workgroup and the lane's row slots: [col_lo, col_hi]
  int col_hi[QT], col_lo[QT];
#pragma unroll
  for (int qt = 0; qt < QT; ++qt) {
    const int qrow = row0 + qt * 16 + c;
    col_hi[qt] = (a.has_right ? (qrow + shift + a.right_off_w < k_len - 1 ? qrow + shift + a.right_off_w : k_len - 1)
                              : k_len - 1) - key_base - 4 * pig;
    col_lo[qt] = (a.has_left ? qrow + shift - a.left_off_w : 0) - key_base - 4 * pig;
  }

  f32x4 s_buf[2][2][QT];   // S(h) in buffer h & 1: [buffer][KT2][QT]
  Frag pf[QT];             // P(h) as the B operand of the PV MFMAs
  float psum[QT];
  float tmax[QT];
  u32x4 kring[RING];
  u32x2 vring[RING][2];

  // fragment read for slot `i` of phase A (K slot SK, half tile KT) or of phase B (V slot SV, half tile KT)
  auto read_k = [&](auto i_c, auto sk_c, auto kt_c) {
    constexpr int i = decltype(i_c)::value, SK = decltype(sk_c)::value, KT = decltype(kt_c)::value;
    constexpr int kt2 = i % 2, kk = i / 2;
    kring[i % RING] = lds_read_b128_imm<SK * OPB + (KT * 32 + kt2 * 16) * RB>(k_addr[kk]);
  };
  auto read_v = [&](auto i_c, auto sv_c, auto kt_c) {
    constexpr int i = decltype(i_c)::value, SV = decltype(sv_c)::value, KT = decltype(kt_c)::value;
    // (callers guard with `if constexpr (i < NPV)`, but inside nested generic lambdas the compiler still instantiates
    // this body for the discarded calls; the clamp keeps those instantiations inside the array)
    constexpr int ia = i < NPV ? i : 0;
    vring[i % RING][0] = lds_read_tr_b64_imm<SV * OPB + (KT * 32) * RB>(v_addr[ia]);
    vring[i % RING][1] = lds_read_tr_b64_imm<SV * OPB + (KT * 32 + 16) * RB>(v_addr[ia]);
  };
  // score pair pi (0..7) of a half tile: elements 2 w, 2 w + 1 of tile (KT2, QT); it is word 2 KT2 + w of pf[QT]
  // Phase A of the step whose scores S(h) sit in buffer CUR.  QK: S(h+1) = K.Q^T - m -> buffer CUR^1, from half
  // CUR^1 of K slot SK.  EXP: P(h) = exp2(S(h)) and its row sum; the last RING slots then start the V fragment
  // reads of the phase B that follows (V slot SV).  Per slot: one K fragment, two MFMAs and one score pair.
  auto phase_a = [&](auto cur_c, auto sk_c, auto sv_c, auto qk_c, auto exp_c) {
    constexpr int CUR = decltype(cur_c)::value;
    constexpr bool QK = decltype(qk_c)::value != 0, EXP = decltype(exp_c)::value != 0;
    constexpr bool PRE_V = EXP;
    constexpr int NXT = CUR ^ 1;
    if constexpr (QK) {
      a_static_for<0, RING>([&](auto ic) { read_k(ic, sk_c, AInt<NXT>{}); });
    }
    if constexpr (EXP && !ROWSUM_MFMA) {
#pragma unroll
      for (int qt = 0; qt < QT; ++qt) psum[qt] = 0.f;
    }
    a_static_for<0, KS>([&](auto ic) {
      constexpr int i = decltype(ic)::value;
      constexpr int kt2 = i % 2, kk = i / 2;
      if constexpr (QK) {
        // LDS operations younger than read i at this point: those issued in the RING - 1 slots before this one
        constexpr int y1 = (RING > 1) ? ((i + 1 < KS) ? 1 : (PRE_V ? 2 : 0)) : 0;
        constexpr int y2 = (RING > 2) ? ((i + 2 < KS) ? 1 : (PRE_V ? 2 : 0)) : 0;
        constexpr int y3 = (RING > 3) ? ((i + 3 < KS) ? 1 : (PRE_V ? 2 : 0)) : 0;
        lds_wait_n<y1 + y2 + y3>(kring[i % RING]);
      }
      a_static_for<0, QT>([&](auto qc) {
        constexpr int qt = decltype(qc)::value;
        if constexpr (QK) {
          const Frag kf = __builtin_bit_cast(Frag, kring[i % RING]);
          if constexpr (kk == 0) s_buf[NXT][kt2][qt] = AttnMfma<T>::mma16(kf, qf[qt][kk], minit[qt]);
          else s_buf[NXT][kt2][qt] = AttnMfma<T>::mma16(kf, qf[qt][kk], s_buf[NXT][kt2][qt]);
        }
        if constexpr (qt == QT - 1) {
          if constexpr (QK && i + RING < KS) read_k(AInt<i + RING>{}, sk_c, AInt<NXT>{});
          else if constexpr (PRE_V && i + RING >= KS) read_v(AInt<i + RING - KS>{}, sv_c, cur_c);
        }
      });
      if constexpr (EXP) {
        constexpr int per = 8 / KS > 0 ? 8 / KS : 1;
        a_static_for<0, per>([&](auto jc) {
          constexpr int pi = i * per + decltype(jc)::value;
          if constexpr (pi < 8) {
            constexpr int qt = pi / 4, t2 = (pi % 4) / 2, w = pi % 2;
            const float p0 = __builtin_amdgcn_exp2f(s_buf[CUR][t2][qt][2 * w]);
            const float p1 = __builtin_amdgcn_exp2f(s_buf[CUR][t2][qt][2 * w + 1]);
            typedef T T2 __attribute__((ext_vector_type(2)));
            const T2 pk = {(T)p0, (T)p1};
            if constexpr (!ROWSUM_MFMA) {
              psum[qt] += p0 + p1;
              asm volatile("" : "+v"(psum[qt]));  // (keeps the addition in this slot: left free it sinks behind phase B)
            }
            u32x4 words = __builtin_bit_cast(u32x4, pf[qt]);
            words[t2 * 2 + w] = __builtin_bit_cast(uint32_t, pk);
            pf[qt] = __builtin_bit_cast(Frag, words);
          }
        });
      }
      __builtin_amdgcn_sched_barrier(0);
    });
    if constexpr (EXP && !ROWSUM_MFMA) {
#pragma unroll
      for (int qt = 0; qt < QT; ++qt) l_run[qt] += psum[qt];
    }
  };

  // Phase B.  PV: O += V(keys of half tile CUR of V slot SV)^T.P (the first RING fragment pairs were requested by
  // phase A).  MAX: the lane's maximum over S(h+1) in buffer CUR^1 (redone by mask_and_max where the half tile
  // needs a mask); it starts two slots into the phase, when the last scores have left the matrix pipe.
  auto phase_b = [&](auto cur_c, auto sv_c, auto max_c) {
    constexpr int CUR = decltype(cur_c)::value;
    constexpr bool MAX = decltype(max_c)::value != 0;
    constexpr int NXT = CUR ^ 1;
    if constexpr (MAX) {
#pragma unroll
      for (int qt = 0; qt < QT; ++qt) tmax[qt] = -INFINITY;
    }
    a_static_for<0, NPV>([&](auto ic) {
      constexpr int i = decltype(ic)::value;
      constexpr int ahead = (i + RING - 1 < NPV) ? RING - 1 : (NPV - 1 - i);
      lds_wait_n2<2 * ahead>(vring[i % RING][0], vring[i % RING][1]);
      const u32x4 both = {vring[i % RING][0][0], vring[i % RING][0][1], vring[i % RING][1][0], vring[i % RING][1][1]};
      a_static_for<0, QT>([&](auto qc) {
        constexpr int qt = decltype(qc)::value;
        o_acc[qt][i] = AttnMfma<T>::mma16(__builtin_bit_cast(Frag, both), pf[qt], o_acc[qt][i]);
        if constexpr (qt == QT - 1 && i + RING < NPV) read_v(AInt<i + RING>{}, sv_c, cur_c);
      });
      if constexpr (ROWSUM_MFMA && i < QT) {
        // slot i carries the row-sum product of column tile i: the first two slots of the phase hold no vector work
        l_acc[i < QT ? i : 0] = AttnMfma<T>::mma16(ones, pf[i < QT ? i : 0], l_acc[i < QT ? i : 0]);
      }
      if constexpr (MAX && i >= 2) {
        // the 8 score pairs over the slots from the third on
        constexpr int per = (8 + NPV - 3) / (NPV - 2);
        a_static_for<0, per>([&](auto jc) {
          constexpr int pi = (i - 2) * per + decltype(jc)::value;
          if constexpr (pi < 8) {
            constexpr int qt = pi % 2, t2 = (pi / 2) % 2, w = pi / 4;   // the two rows' chains alternate
            tmax[qt] = fmaxf(fmaxf(tmax[qt], s_buf[NXT][t2][qt][2 * w]), s_buf[NXT][t2][qt][2 * w + 1]);
          }
        });
        if constexpr (i == NPV - 1) asm volatile("" : "+v"(tmax[0]), "+v"(tmax[1]));
      }
      __builtin_amdgcn_sched_barrier(0);
    });
  };

  // masks on the scores of half tile h of column tile QT (in buffer BUF), then their maximum (diagonal, window edge
  // and last tiles)
  auto mask_and_max = [&](int h, auto qt_c, auto buf_c) {
    constexpr int BUF = decltype(buf_c)::value, qt = decltype(qt_c)::value;
    // element r of tile KT2 is key key_base + h*32 + 16 KT2 + 4 pi(g) + r
    const int hi_rel = col_hi[qt] - h * kHB, lo_rel = col_lo[qt] - h * kHB;
    float tm = -INFINITY;
#pragma unroll
    for (int t2 = 0; t2 < 2; ++t2)
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        const int rel = t2 * 16 + r;
        float s = s_buf[BUF][t2][qt][r];
        s = rel > hi_rel ? -INFINITY : s;
        if (a.has_left) s = rel < lo_rel ? -INFINITY : s;
        s_buf[BUF][t2][qt][r] = s;
        tm = fmaxf(tm, s);
      }
    tmax[qt] = tm;
  };
  // half tile h of column tile qt needs the mask pass from mask_from[qt] on (diagonal, right window edge, partial
  // last tile) and below mask_below[qt] (left window edge)
  int mask_from[QT], mask_below[QT];
#pragma unroll
  for (int qt = 0; qt < QT; ++qt) {
    const int r_first = row0 + qt * 16;
    const int r_last = (r_first + 15 < q_len ? r_first + 15 : q_len - 1);
    int from = (k_len - key_base - kHB) < 0 ? 0 : (k_len - key_base - kHB) / kHB + 1;
    if (a.has_right) {
      const int bnd = r_first + shift + a.right_off_w - (kHB - 1) - key_base;
      const int f2 = bnd < 0 ? 0 : bnd / kHB + 1;
      from = from < f2 ? from : f2;
    }
    mask_from[qt] = from;
    const int lb = r_last + shift - a.left_off_w - key_base;
    mask_below[qt] = a.has_left ? (lb <= 0 ? 0 : (lb + kHB - 1) / kHB) : 0;
  }
  auto needs_mask = [&](int h, int qt) { return h >= mask_from[qt] || h < mask_below[qt]; };
  // The scores in buffer BUF are relative to the reference m_run they were scored with.  Where a lane finds one
  // more than 2^8 above it (or the row has no reference yet and sees its first key), the row's reference moves to
  // the new maximum: the waiting scores, O and the row sum are shifted by the difference.
  auto new_reference = [&](auto buf_c) {
    constexpr int BUF = decltype(buf_c)::value;
    bool any = false;
#pragma unroll
    for (int qt = 0; qt < QT; ++qt) any = any || tmax[qt] > 8.0f || (m_run[qt] == -INFINITY && tmax[qt] > -INFINITY);
    if (__builtin_amdgcn_ballot_w64(any) == 0) return;
    a_static_for<0, QT>([&](auto qc) {
      constexpr int qt = decltype(qc)::value;
      const bool fresh = m_run[qt] == -INFINITY;
      const float tm = xquad_max(tmax[qt]);
      const bool moved = tm > 8.0f || (fresh && tm > -INFINITY);
      if (__builtin_amdgcn_ballot_w64(moved) == 0) return;
      const float delta = moved ? tm : 0.f;
      const float alpha = __builtin_amdgcn_exp2f(-delta);
#pragma unroll
      for (int t2 = 0; t2 < 2; ++t2)
#pragma unroll
        for (int r = 0; r < 4; ++r) s_buf[BUF][t2][qt][r] -= delta;
#pragma unroll
      for (int dt = 0; dt < NPV; ++dt)
#pragma unroll
        for (int r = 0; r < 4; ++r) o_acc[qt][dt][r] *= alpha;
      if constexpr (ROWSUM_MFMA) {
#pragma unroll
        for (int r = 0; r < 4; ++r) l_acc[qt][r] *= alpha;
      } else {
        l_run[qt] *= alpha;
      }
      if (moved) m_run[qt] = (fresh ? 0.f : m_run[qt]) + delta;
      const float mm = m_run[qt] == -INFINITY ? 0.f : -m_run[qt];
      minit[qt] = f32x4{mm, mm, mm, mm};
    });
  };
  auto mask_where_needed = [&](int h, auto buf_c) {
    a_static_for<0, QT>([&](auto qc) {
      if (needs_mask(h, decltype(qc)::value)) mask_and_max(h, qc, buf_c);
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
    a_static_for<0, QT>([&](auto qc) { mask_and_max(0, qc, AInt<0>{}); });
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

  // ---- epilogue: lane (g, c) holds O^T[16 dt + 4 g + r][q = 16 QT + c] ---------------------------------
#pragma unroll
  for (int qt = 0; qt < QT; ++qt) {
    float l_row;
    if constexpr (ROWSUM_MFMA) l_row = l_acc[qt][0];   // already the sum over all keys of the row
    else l_row = xquad_sum(l_run[qt]);
    const int qrow = row0 + qt * 16 + c;
    if (qrow >= q_len) continue;
    const bool empty = l_row == 0.f || l_row != l_row;
    const float inv = empty ? 1.f : 1.f / l_row;
    if (p.lse != nullptr && g == 0) {
      p.lse[(int64_t)head * p.total_q + q_bos + qrow] = empty ? INFINITY : m_run[qt] * 0.6931471805599453f + logf(l_row);
    }
    T* op = (T*)p.out + (int64_t)(q_bos + qrow) * p.o_row_stride + (int64_t)head * p.o_head_stride;
#pragma unroll
    for (int dt = 0; dt < NPV; ++dt) {
      Pack<T, 4> o;
#pragma unroll
      for (int e = 0; e < 4; ++e) o.v[e] = (T)(o_acc[qt][dt][e] * inv);
      st_pack<T, 4>(op + dt * 16 + g * 4, o);
    }
  }
}

template <typename T, int D>
int launch_pipe(const AttnArgs& a, dim3 grid, hipStream_t st) {
  constexpr int LDS_BYTES = 2 * 2 * kBN * 2 * D;
  static hipError_t attr_err = hipFuncSetAttribute(reinterpret_cast<const void*>(attn_varlen_pipe_kernel<T, D>),
                                                   hipFuncAttributeMaxDynamicSharedMemorySize, LDS_BYTES);
  if (attr_err != hipSuccess) {
    fg_set_error("flash_attn_varlen_fwd: cannot reserve %d bytes of LDS: %s", LDS_BYTES, hipGetErrorString(attr_err));
    return FG_ERR_LAUNCH;
  }
  hipLaunchKernelGGL((attn_varlen_pipe_kernel<T, D>), grid, dim3(256), LDS_BYTES, st, a);
  return fg_check_launch("flash_attn_varlen_fwd");
}
