// Paged varlen attention forward, software-pipelined variant of the lean kernel (attn_fast.h) for the same
// cases: head dim 64 or 128, page size a power of two >= 16, at most 8192 keys per sequence, no ALiBi, no
// soft-cap.  Same work split (4 waves x 32 query rows, a GQA group's heads per workgroup), MFMA formulation
// (S^T = K.Q^T, O^T = V^T.P^T, MFMA 32x32x16), swizzled LDS tiles filled by global_load_lds, and lazily
// re-referenced base-2 online softmax.  What differs is the order of work inside a wave.
//
// Measured on gfx950, one wave issues a plain vector instruction every ~6 cycles and an exponential every
// ~17, and it cannot issue anything while it waits for a matrix result; a vector instruction placed between
// two MFMAs of the same wave that do not need its result costs nothing while the matrix pipe is busy (32
// cycles per MFMA).  The lean kernel runs QK^T, softmax and PV of a tile one after the other, so the matrix
// pipe idles through ~1200 cycles of softmax per tile and wave, and two waves per SIMD do not mesh well
// enough to fill the gap.  Here the work is cut into half tiles of 32 keys (one 32x32 score block per wave),
// and the softmax of half tile h is split in two, each part in the shadow of the MFMAs of a neighbour:
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
// The vector ALU's issue port, not the matrix pipe, is the scarce resource (an exponential holds it ~8 cycles,
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
// This header is included by attn_varlen.hip inside its unnamed namespace, behind attn_fast.h.

template <int N, typename V>
__device__ __forceinline__ void lds_wait_n(V& r) {
  asm volatile("s_waitcnt lgkmcnt(%1)" : "+v"(r) : "i"(N));
}
template <int N, typename V>
__device__ __forceinline__ void lds_wait_n2(V& r0, V& r1) {
  asm volatile("s_waitcnt lgkmcnt(%2)" : "+v"(r0), "+v"(r1) : "i"(N));
}

template <typename T, int D>
__global__ __launch_bounds__(256, 2) void attn_varlen_pipe_kernel(AttnArgs a) {
  typedef typename AttnMfma<T>::Frag Frag;
  constexpr int RB = 2 * D;            // bytes per key row in LDS
  constexpr int CPR = RB / 16;         // 16-byte chunks per row
  constexpr int KS = D / 16;           // MFMA k-steps over the head dim = MFMAs of phase A
  constexpr int DT = D / 32;           // 32-row output sub-tiles over the head dim
  constexpr int NPV = 2 * DT;          // MFMAs of phase B
  constexpr int OPB = kBN * RB;        // one operand tile
  constexpr int KPI = 1024 / RB;       // key rows per DMA instruction
  constexpr int IPW = kBN / KPI / 4;   // DMA instructions per wave, operand and tile
  constexpr int RING = KS < 4 ? KS : 4;  // fragment reads run this many MFMAs ahead
  constexpr int kHB = kBN / 2;         // keys per half tile
  static_assert(KS == NPV && KS >= RING, "both phases issue the same number of MFMAs");
  extern __shared__ __attribute__((aligned(16))) char lds[];  // K slot 0, K slot 1, V slot 0, V slot 1

  const FgFlashParams& p = a.p;
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int half = lane >> 5, ql = lane & 31;
  // long (late) row blocks first, order rotated per (sequence, head group): see attn_fast.h
  const int b = blockIdx.y, hgroup = blockIdx.z;
  const int m_block = (int)((gridDim.x - 1 - blockIdx.x + (unsigned)(b * 5 + hgroup * 3)) % gridDim.x);

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
  const int wave_row_last = (row0 + kRW - 1 < q_len ? row0 + kRW - 1 : q_len - 1);

  // ---- Q fragments ---------------------------------------------------------------------------------
  const int qrow = row0 + ql;
  Frag qf[KS];
  {
    const bool row_ok = qrow < q_len;
    const T* qp = (const T*)p.q + (int64_t)(q_bos + (row_ok ? qrow : 0)) * p.q_row_stride + (int64_t)head * p.q_head_stride;
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) {
      u32x4 v = {0u, 0u, 0u, 0u};
      if (row_ok) v = *reinterpret_cast<const u32x4*>(qp + ks * 16 + half * 8);
      Frag f = __builtin_bit_cast(Frag, v);
#pragma unroll
      for (int e = 0; e < 8; ++e) f[e] = (T)((float)f[e] * a.scale_log2);  // scores leave the MFMA in base-2 units
      qf[ks] = f;
    }
  }
  // the reference m enters the scores through the matrix pipe: ones_f (k-slots 0..2 of the lower half-wave) times
  // m_f (-m as three 16-bit pieces in the same slots of the lane that owns the row)
  Frag ones_f, m_f;
#pragma unroll
  for (int e = 0; e < 8; ++e) {
    ones_f[e] = (T)((half == 0 && e < 3) ? 1.0f : 0.0f);
    m_f[e] = (T)0.0f;
  }
  f32x16 o_acc[DT];
#pragma unroll
  for (int dt = 0; dt < DT; ++dt)
#pragma unroll
    for (int e = 0; e < 16; ++e) o_acc[dt][e] = 0.f;
  float m_run = -INFINITY, l_run = 0.f;

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
  const int last_page = k_len > 0 ? (k_len - 1) >> page_shift : 0;
  int pg_cache0, pg_cache1;
  {
    int pg0 = ((n_min + lane) * kBN + wave * (IPW * KPI)) >> page_shift;
    int pg1 = ((n_min + 64 + lane) * kBN + wave * (IPW * KPI)) >> page_shift;
    pg0 = pg0 < last_page ? pg0 : last_page;
    pg1 = pg1 < last_page ? pg1 : last_page;
    pg_cache0 = btab[pg0];
    pg_cache1 = btab[pg1];
  }
  // one operand tile (K: is_v = 0, V: is_v = 1) of key tile n_min + t into `slot` of its ring
  auto issue_op = [&](int t, int slot, auto is_v_c) {
    constexpr bool IS_V = decltype(is_v_c)::value != 0;
    const int nb = n_min + t;
    char* dst = lds + (IS_V ? 2 * OPB : 0) + slot * OPB + wave * (IPW * 1024);
    const char* base = IS_V ? vbase : kbase;
    const int64_t page_stride = IS_V ? p.v_page_stride : p.k_page_stride;
    const int64_t row_stride = IS_V ? p.v_row_stride : p.k_row_stride;
    if (nb * kBN + kBN <= k_len) {
      // full tile: every key exists; one scalar row base per instruction, one 32-bit lane offset
      const int tl = t < 127 ? t : 127;
      const int64_t page = __builtin_amdgcn_readlane(tl < 64 ? pg_cache0 : pg_cache1, tl & 63);
      const int key = nb * kBN + wave * (IPW * KPI);
      const int slot_in_page = key & page_mask;
      const char* rp = base + (page * page_stride + (int64_t)slot_in_page * row_stride) * 2;
#pragma unroll
      for (int j = 0; j < IPW; ++j) {
        // kept opaque so that the address stays "scalar base + 32-bit lane offset" (the compiler would otherwise
        // precompute a 64-bit lane offset per instruction and operand and hold sixteen register pairs for them)
        uint32_t c0 = lane_c0;
        asm volatile("" : "+v"(c0));
        const uint32_t voff = (IS_V ? lane_row_v : lane_row_k) + (c0 ^ (uint32_t)(j * 16));
        __builtin_amdgcn_global_load_lds(FG_GLBP(rp + (int64_t)j * KPI * row_stride * 2 + voff), FG_LDSP(dst + j * 1024), 16, 0, 0);
      }
    } else {
      // partial tile: keys past the end are clamped to the last one (their scores are masked)
#pragma unroll
      for (int j = 0; j < IPW; ++j) {
        int key = nb * kBN + (wave * IPW + j) * KPI + lane_key;
        key = key < k_len ? key : k_len - 1;
        const int64_t page = btab[key >> page_shift];
        const int slot_in_page = key & page_mask;
        uint32_t c0 = lane_c0;
        asm volatile("" : "+v"(c0));
        const char* rp = base + ((page * page_stride + (int64_t)slot_in_page * row_stride) * 2 + (c0 ^ (uint32_t)(j * 16)));
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

  // visible keys of this lane's row, relative to the first key of the workgroup: [col_lo, col_hi]
  const int col_hi = (a.has_right ? (qrow + shift + a.right_off_w < k_len - 1 ? qrow + shift + a.right_off_w : k_len - 1)
                                  : k_len - 1) - key_base - half * 8;
  const int col_lo = (a.has_left ? qrow + shift - a.left_off_w : 0) - key_base - half * 8;

  f32x16 s_buf[2];      // S(h) in buffer h & 1
  Frag pf[2];           // P(h) as the B operand of the PV MFMAs (2 x 16 keys)
  float psum = 0.f;
  float tmax_a = -INFINITY, tmax_b = -INFINITY;
  u32x4 kring[RING];
  u32x2 vring[RING][2];

  // fragment read for MFMA `i` of phase A (key sub-tile KT of K slot SK) or of phase B (the keys of sub-tile KT in
  // V slot SV)
  auto read_k = [&](auto i_c, auto sk_c, auto kt_c) {
    constexpr int i = decltype(i_c)::value, SK = decltype(sk_c)::value, KT = decltype(kt_c)::value;
    kring[i % RING] = lds_read_b128_imm<SK * OPB + KT * 32 * RB>(k_addr[i]);
  };
  auto read_v = [&](auto i_c, auto sv_c, auto kt_c) {
    constexpr int i = decltype(i_c)::value, SV = decltype(sv_c)::value, KT = decltype(kt_c)::value;
    constexpr int dt = i / 2, t4 = KT * 2 + i % 2;
    vring[i % RING][0] = lds_read_tr_b64_imm<SV * OPB + t4 * 16 * RB>(v_addr0[dt]);
    vring[i % RING][1] = lds_read_tr_b64_imm<SV * OPB + t4 * 16 * RB>(v_addr1[dt]);
  };

  // Phase A of the step whose scores S(h) sit in buffer CUR.  QK: S(h+1) = K.Q^T - m -> buffer CUR^1, from key
  // sub-tile CUR^1 of K slot SK.  EXP: P(h) = exp2(S(h)) and its row sum; the last RING slots then start the V
  // fragment reads of the phase B that follows (V slot SV).
  auto phase_a = [&](auto cur_c, auto sk_c, auto sv_c, auto qk_c, auto exp_c) {
    constexpr int CUR = decltype(cur_c)::value;
    constexpr bool QK = decltype(qk_c)::value != 0, EXP = decltype(exp_c)::value != 0;
    constexpr bool PRE_V = EXP;
    constexpr int NXT = CUR ^ 1;
    if constexpr (QK) {
      a_static_for<0, RING>([&](auto ic) { read_k(ic, sk_c, AInt<NXT>{}); });
#pragma unroll
      for (int e = 0; e < 16; ++e) s_buf[NXT][e] = 0.f;
      s_buf[NXT] = AttnMfma<T>::mma(ones_f, m_f, s_buf[NXT]);  // -m, while the first K fragments arrive
    }
    if constexpr (EXP) psum = 0.f;
    a_static_for<0, KS>([&](auto ic) {
      constexpr int i = decltype(ic)::value;
      if constexpr (QK) {
        // LDS operations younger than read i at this point: those issued in the RING - 1 slots before this one
        constexpr int y1 = (RING > 1) ? ((i + 1 < KS) ? 1 : (PRE_V ? 2 : 0)) : 0;
        constexpr int y2 = (RING > 2) ? ((i + 2 < KS) ? 1 : (PRE_V ? 2 : 0)) : 0;
        constexpr int y3 = (RING > 3) ? ((i + 3 < KS) ? 1 : (PRE_V ? 2 : 0)) : 0;
        lds_wait_n<y1 + y2 + y3>(kring[i % RING]);
        s_buf[NXT] = AttnMfma<T>::mma(__builtin_bit_cast(Frag, kring[i % RING]), qf[i], s_buf[NXT]);
        if constexpr (i + RING < KS) read_k(AInt<i + RING>{}, sk_c, AInt<NXT>{});
        else if constexpr (PRE_V) read_v(AInt<i + RING - KS>{}, sv_c, cur_c);
      } else if constexpr (PRE_V) {
        if constexpr (i + RING >= KS) read_v(AInt<i + RING - KS>{}, sv_c, cur_c);
      }
      if constexpr (EXP) {
        // 8 score pairs over KS slots: elements 2w, 2w+1 of half t2 -> word w of pf[t2]
        constexpr int per = 8 / KS > 0 ? 8 / KS : 1;
        a_static_for<0, per>([&](auto jc) {
          constexpr int pi = i * per + decltype(jc)::value;
          if constexpr (pi < 8) {
            constexpr int t2 = pi / 4, w = pi % 4;
            const float p0 = __builtin_amdgcn_exp2f(s_buf[CUR][t2 * 8 + 2 * w]);
            const float p1 = __builtin_amdgcn_exp2f(s_buf[CUR][t2 * 8 + 2 * w + 1]);
            typedef T T2 __attribute__((ext_vector_type(2)));
            const T2 pk = {(T)p0, (T)p1};
            psum += p0 + p1;  // (dot-product instructions would halve this, but they wait for the matrix pipe)
            u32x4 words = __builtin_bit_cast(u32x4, pf[t2]);
            words[w] = __builtin_bit_cast(uint32_t, pk);
            pf[t2] = __builtin_bit_cast(Frag, words);
          }
        });
      }
      __builtin_amdgcn_sched_barrier(0);
    });
    if constexpr (EXP) l_run += xhalf_sum(psum);
  };

  // Phase B.  PV: O += V(keys of sub-tile CUR of V slot SV)^T.P (the first RING fragment pairs were requested by
  // phase A).  MAX: the lane's maximum over S(h+1) in buffer CUR^1 (redone by mask_and_max where the half tile
  // needs a mask); it starts two MFMAs into the phase, when the last scores have left the matrix pipe.
  auto phase_b = [&](auto cur_c, auto sv_c, auto max_c) {
    constexpr int CUR = decltype(cur_c)::value;
    constexpr bool MAX = decltype(max_c)::value != 0;
    constexpr int NXT = CUR ^ 1;
    if constexpr (MAX) tmax_a = tmax_b = -INFINITY;
    a_static_for<0, NPV>([&](auto ic) {
      constexpr int i = decltype(ic)::value;
      constexpr int ahead = (i + RING - 1 < NPV) ? RING - 1 : (NPV - 1 - i);
      lds_wait_n2<2 * ahead>(vring[i % RING][0], vring[i % RING][1]);
      const u32x4 both = {vring[i % RING][0][0], vring[i % RING][0][1], vring[i % RING][1][0], vring[i % RING][1][1]};
      o_acc[i / 2] = AttnMfma<T>::mma(__builtin_bit_cast(Frag, both), pf[i % 2], o_acc[i / 2]);
      if constexpr (i + RING < NPV) read_v(AInt<i + RING>{}, sv_c, cur_c);
      if constexpr (MAX && i >= 2) {
        // the 8 score pairs over the slots from the third on
        constexpr int per = (8 + NPV - 3) / (NPV - 2);
        a_static_for<0, per>([&](auto jc) {
          constexpr int pi = (i - 2) * per + decltype(jc)::value;
          if constexpr (pi < 8) {
            if constexpr (pi % 2 == 0) tmax_a = fmaxf(fmaxf(tmax_a, s_buf[NXT][2 * pi]), s_buf[NXT][2 * pi + 1]);
            else tmax_b = fmaxf(fmaxf(tmax_b, s_buf[NXT][2 * pi]), s_buf[NXT][2 * pi + 1]);
          }
        });
        if constexpr (i == NPV - 1) asm volatile("" : "+v"(tmax_a), "+v"(tmax_b));  // keeps the maxima inside their slots
      }
      __builtin_amdgcn_sched_barrier(0);
    });
  };

  // masks on the scores of half tile h (in buffer BUF), then their maximum (diagonal, window edge and last tiles)
  auto mask_and_max = [&](int h, auto buf_c) {
    constexpr int BUF = decltype(buf_c)::value;
    // element e is key key_base + h*32 + half*8 + (e>>3)*16 + (e&7)
    const int hi_rel = col_hi - h * kHB, lo_rel = col_lo - h * kHB;
    float tm = -INFINITY;
#pragma unroll
    for (int e = 0; e < 16; ++e) {
      const int rel = (e >> 3) * 16 + (e & 7);
      float s = s_buf[BUF][e];
      s = rel > hi_rel ? -INFINITY : s;
      if (a.has_left) s = rel < lo_rel ? -INFINITY : s;
      s_buf[BUF][e] = s;
      tm = fmaxf(tm, s);
    }
    tmax_a = tm;
    tmax_b = -INFINITY;
  };
  auto needs_mask = [&](int h) {
    const int key0 = key_base + h * kHB;
    return (key0 + kHB > k_len) || (a.has_right && key0 + kHB - 1 > row0 + shift + a.right_off_w) ||
           (a.has_left && key0 < wave_row_last + shift - a.left_off_w);
  };
  // The scores in buffer BUF are relative to the reference m_run they were scored with.  Where a lane finds one
  // more than 2^8 above it (or the row has no reference yet and sees its first key), the row's reference moves to
  // the new maximum: the waiting scores, O and the row sum are shifted by the difference and -m is split anew.
  // Any reference gives the same result as long as P and the running sum use the same one.
  auto new_reference = [&](auto buf_c) {
    constexpr int BUF = decltype(buf_c)::value;
    const float tl = fmaxf(tmax_a, tmax_b);
    const bool fresh = m_run == -INFINITY;
    if (__builtin_amdgcn_ballot_w64(tl > 8.0f || (fresh && tl > -INFINITY)) == 0) return;
    const float tmax = xhalf_max(tl);
    const bool moved = tmax > 8.0f || (fresh && tmax > -INFINITY);
    const float delta = moved ? tmax : 0.f;
    const float alpha = __builtin_amdgcn_exp2f(-delta);
#pragma unroll
    for (int e = 0; e < 16; ++e) s_buf[BUF][e] -= delta;
#pragma unroll
    for (int dt = 0; dt < DT; ++dt)
#pragma unroll
      for (int e = 0; e < 16; ++e) o_acc[dt][e] *= alpha;
    l_run *= alpha;
    if (moved) m_run = (fresh ? 0.f : m_run) + delta;
    // -m_run as three pieces of the input type (their sum is exact to ~2^-24 of m), in k-slots 0..2 of the lane
    // of the lower half-wave that owns the row
    const float mm = (m_run == -INFINITY || half != 0) ? 0.f : -m_run;
    const T hi = (T)mm;
    const float r1 = mm - (float)hi;
    const T mid = (T)r1;
    const T lo = (T)(r1 - (float)mid);
    m_f[0] = hi;
    m_f[1] = mid;
    m_f[2] = lo;
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
      if (needs_mask(h + 1)) mask_and_max(h + 1, AInt<KT ^ 1>{});
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
    mask_and_max(0, AInt<0>{});
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
      Pack<T, 4> o;
#pragma unroll
      for (int e = 0; e < 4; ++e) o.v[e] = (T)(o_acc[dt][g * 4 + e] * inv);
      st_pack<T, 4>(op + d, o);
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
