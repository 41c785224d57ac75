// Paged varlen attention forward, head-pair variant of the lean kernel (head dim 128, an even number of
// query heads per KV head; otherwise the same preconditions as attn_varlen_fast_kernel).
//
// The lean kernel runs, per wave, S = K.Q^T (matrix cores), then the softmax (vector ALU), then O += V^T.P
// (matrix cores) strictly one after the other, and relies on a second workgroup on the CU to fill the gaps;
// measured, the matrix cores are busy a third of the time.  Here a wave owns the same 32 query rows of TWO
// heads that share a KV head, holds all its state in the 512 registers of a SIMD that it has to itself, and
// runs a software pipeline over the key tiles in which every matrix instruction is followed by a slice of
// vector work that does not depend on it:
//
//   step t:   O += V(t-1)^T.P(t-1)   four groups of 8 MFMAs  |  running max of S(t), first half of p = exp2(S(t) - ref)
//             -- tile t+1 has landed: barrier --
//             S(t+1) = K(t+1).Q^T    four groups of 8 MFMAs  |  second half of the exponentials, copy of tile t+3
//
//   * every K and V fragment read from LDS feeds two MFMAs (one per head), which halves the LDS traffic per
//     flop; at one fragment per MFMA the LDS port would be as busy as the matrix cores.
//   * P(t) overwrites P(t-1) quarter by quarter, each quarter after the PV MFMAs that read it have been
//     issued; S(t+1) overwrites S(t) half by half after the exponentials that read it.  Nothing is double
//     buffered in registers.
//   * four LDS stages: step t reads V(t-1) and K(t+1) while V(t) waits for the next step and tiles t+2 and
//     t+3 are in flight (one workgroup per CU: nobody else hides the latency of the copies); one barrier per
//     step, in the middle.
//   * rows that a tile does not reach (causal bound below the tile) are not skipped: their scores are masked,
//     the probabilities are exact zeros.
//   * the accumulators live in the accumulator half of the register file, where the vector ALU cannot
//     multiply them, so O is never rescaled: the reference of a row's exponentials is the maximum of the
//     first tile that reaches the row and stays put (softmax is invariant under the choice of reference as
//     long as nothing overflows).  A later score that exceeds the reference by more than kRefLimit powers of
//     two marks the workgroup in a flag array instead (its output is then meaningless); the host launches the
//     lean kernel right behind this one for exactly the marked blocks.  With real attention scores nothing
//     is ever marked and that second launch finds no work.
//
// Status: numerically equivalent to the lean kernel and selectable with FG_ATTN_KERNEL=pair, but not the
// default.  Measured on MI355X (16 causal sequences of 512..4096 tokens, 32/8 heads): 595 TFLOP/s against
// 780 for the lean kernel.  Cycle stamps inside the step show why:
//   * the vector ALU needs about 27 cycles per score (fma 5, exp 10, add 5, half a convert, plus the issue
//     slots the neighbouring MFMA takes), so a quarter of the exponentials keeps a group of 8 MFMAs busy for
//     435 cycles instead of 256: with one wave per SIMD the step is bound by the vector ALU, not by the
//     matrix cores, at about 4300 cycles for 2048 cycles of MFMA;
//   * one workgroup per CU leaves nothing to hide the start of a workgroup (sequence lengths, page ids, Q,
//     the first tile: several dependent round trips to memory, about 11 us) or the tail of the grid; a fifth
//     of a wave's lifetime is spent outside the steps, a quarter of all SIMD cycles in no wave at all.
// A vector-ALU read of an accumulator in the accumulator half of the register file waits for every MFMA in
// flight (100 cycles instead of 8), which is why the scores are kept in ordinary registers by asm MFMAs.
// This header is included by attn_varlen.hip inside its unnamed namespace, after attn_fast.h.

template <typename T> __device__ __forceinline__ uint32_t pack_pair(float lo, float hi) {
  typedef float f32x2v __attribute__((ext_vector_type(2)));
  typedef T t16x2 __attribute__((ext_vector_type(2)));
  const f32x2v f = {lo, hi};
  const t16x2 t = __builtin_convertvector(f, t16x2);
  return __builtin_bit_cast(uint32_t, t);
}
// The S MFMAs are written as asm so that their accumulators sit in ordinary registers, where the softmax
// reads them at full speed, while O (compiler-generated MFMAs) sits in the accumulator half of the register
// file together with Q: a vector-ALU read of the accumulator half waits for every MFMA in flight, which
// would undo the overlap this kernel is built around.  The compiler does not know that these statements are
// MFMAs and inserts no wait states after them: the step keeps two other MFMAs between the last write of a
// score and its first read, and the masking pass, which runs right after a step, waits explicitly.
template <typename T> struct PairMfma;
template <> struct PairMfma<bf16_t> {
  static __device__ __forceinline__ void first(f32x16& d, u32x4 k, u32x4 q) {
    asm volatile("v_mfma_f32_32x32x16_bf16 %0, %1, %2, 0" : "=&v"(d) : "v"(k), "a"(q));
  }
  static __device__ __forceinline__ void next(f32x16& d, u32x4 k, u32x4 q) {
    asm volatile("v_mfma_f32_32x32x16_bf16 %0, %1, %2, %0" : "+v"(d) : "v"(k), "a"(q));
  }
};
template <> struct PairMfma<f16_t> {
  static __device__ __forceinline__ void first(f32x16& d, u32x4 k, u32x4 q) {
    asm volatile("v_mfma_f32_32x32x16_f16 %0, %1, %2, 0" : "=&v"(d) : "v"(k), "a"(q));
  }
  static __device__ __forceinline__ void next(f32x16& d, u32x4 k, u32x4 q) {
    asm volatile("v_mfma_f32_32x32x16_f16 %0, %1, %2, %0" : "+v"(d) : "v"(k), "a"(q));
  }
};
__device__ __forceinline__ void mfma_settle() { asm volatile("s_nop 15\n\ts_nop 15" ::: "memory"); }
__device__ __forceinline__ void lds_wait_k(u32x4 (&r)[4]) {
  asm volatile("s_waitcnt lgkmcnt(0)" : "+v"(r[0]), "+v"(r[1]), "+v"(r[2]), "+v"(r[3]));
}

template <typename T, int D>
__global__ __launch_bounds__(256, 1) void attn_varlen_pair_kernel(AttnArgs a) {
  typedef typename AttnMfma<T>::Frag Frag;
  static_assert(D == 128, "the step schedule below is written for head dim 128");
  constexpr int RB = 2 * D;            // bytes per key row in LDS
  constexpr int CPR = RB / 16;         // 16-byte chunks per row
  constexpr int KS = D / 16;           // MFMA k-steps over the head dim
  constexpr int DT = D / 32;           // 32-row output sub-tiles over the head dim
  constexpr int OPB = kBN * RB;        // one operand tile
  constexpr int STAGEB = 2 * OPB;      // K tile + V tile
  constexpr int KPI = 1024 / RB;       // key rows per DMA instruction
  constexpr int IPW = kBN / KPI / 4;   // DMA instructions per wave, operand and tile
  extern __shared__ __attribute__((aligned(16))) char lds[];

  const FgFlashParams& p = a.p;
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int half = lane >> 5, ql = lane & 31;
  const int b = blockIdx.y, hgroup = blockIdx.z;
  // long row blocks first, rotated per (sequence, head group) as in the lean kernel
  const int m_block = (int)((gridDim.x - 1 - blockIdx.x + (unsigned)(b * 5 + hgroup * 3)) % gridDim.x);

  const int q_bos = p.cu_seqlens_q[b];
  const int q_len = p.cu_seqlens_q[b + 1] - q_bos;
  const int k_len = p.seqused_k[b];
  const int block_row0 = m_block * a.rows_per_block;
  // The block's redo flag starts at zero.  The exchange returns a value, so it has completed before this
  // thread reaches the first barrier; a wave that sets the flag does so after that barrier.
  int* const redo_flag = a.redo_flags + ((int64_t)blockIdx.z * gridDim.y + blockIdx.y) * gridDim.x + m_block;
  if (tid == 0) (void)__hip_atomic_exchange(redo_flag, 0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  if (block_row0 >= q_len) return;

  const int wpp = 8 / a.hpb;  // waves per head pair: 4 (one pair per workgroup) or 2 (two pairs)
  const int head0 = hgroup * a.hpb + (wave / wpp) * 2;
  const int row0 = block_row0 + (wave % wpp) * kRW;
  const int kv_head = head0 / (p.Hq / p.Hk);

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
  const int NT = n_max - n_min;  // tiles of this workgroup

  // ---- Q fragments of both heads ------------------------------------------------------------------------
  const int qrow = row0 + ql;
  // Loaded straight into the accumulator half of the register file, where the S MFMAs read them: a value
  // that only ever exists there is never copied around by the compiler.  Rows past the end of the sequence
  // read row 0 instead; what they compute is never stored.
  u32x4 qf[2][KS];
  {
    const bool row_ok = qrow < q_len;
    const T* qp = (const T*)p.q + (int64_t)(q_bos + (row_ok ? qrow : 0)) * p.q_row_stride + (int64_t)head0 * p.q_head_stride;
#pragma unroll
    for (int h = 0; h < 2; ++h)
#pragma unroll
      for (int ks = 0; ks < KS; ++ks) {
        const T* src = qp + (int64_t)h * p.q_head_stride + ks * 16 + half * 8;
        asm volatile("global_load_dwordx4 %0, %1, off" : "=a"(qf[h][ks]) : "v"(src) : "memory");
      }
  }
  f32x16 o_acc[2][DT];
  // exponent headroom of P (bf16 has fp32's range; fp16 tops out at 2^16) and of the fp32 row sums
  constexpr float kRefLimit = sizeof(T) == 2 && std::is_same<T, f16_t>::value ? 14.0f : 80.0f;
  float m_ref[2] = {-INFINITY, -INFINITY}, m_hi[2] = {-INFINITY, -INFINITY};

  // ---- DMA geometry (as in the lean kernel) --------------------------------------------------------------
  const int wave_s = wave;
  const int32_t* btab = p.block_table + (int64_t)b * p.block_table_stride;
  const char* kbase = (const char*)((const T*)p.k_cache + (int64_t)kv_head * p.k_head_stride);
  const char* vbase = (const char*)((const T*)p.v_cache + (int64_t)kv_head * p.v_head_stride);
  const int page_shift = a.page_shift, page_mask = p.page_size - 1;
  const int lane_key = lane / CPR, lane_pos = lane % CPR;
  uint32_t voff_k[IPW], voff_v[IPW];
  int lane_c16[IPW];
#pragma unroll
  for (int j = 0; j < IPW; ++j) {
    const int key_l = (wave * IPW + j) * KPI + lane_key;
    const int c = lane_pos ^ swz<CPR>(key_l);
    lane_c16[j] = c * 16;
    voff_k[j] = (uint32_t)(lane_key * (int)p.k_row_stride * 2 + c * 16);
    voff_v[j] = (uint32_t)(lane_key * (int)p.v_row_stride * 2 + c * 16);
  }
  const int last_page = k_len > 0 ? (k_len - 1) >> page_shift : 0;
  int pg_cache0, pg_cache1;
  {
    int pg0 = ((n_min + lane) * kBN + wave_s * (IPW * KPI)) >> page_shift;
    int pg1 = ((n_min + 64 + lane) * kBN + wave_s * (IPW * KPI)) >> page_shift;
    pg0 = pg0 < last_page ? pg0 : last_page;
    pg1 = pg1 < last_page ? pg1 : last_page;
    pg_cache0 = btab[pg0];
    pg_cache1 = btab[pg1];
  }
  FG_WAIT_VM(0);  // nothing loaded above is still pending when the first tile copy is issued
  // A full tile is copied in IPW slices (one K and one V instruction each) from scalar bases set up once per
  // tile, so that the slices can sit between the MFMAs of a step.
  const char* dma_kp = nullptr;
  const char* dma_vp = nullptr;
  char* dma_dst = nullptr;
  auto setup_full = [&](int nb, int stage_off) {
    dma_dst = lds + stage_off + wave_s * (IPW * 1024);
    const int tl = nb - n_min < 127 ? nb - n_min : 127;
    const int64_t page = __builtin_amdgcn_readlane(tl < 64 ? pg_cache0 : pg_cache1, tl & 63);
    const int key = nb * kBN + wave_s * (IPW * KPI);
    const int slot = key & page_mask;
    dma_kp = kbase + (page * p.k_page_stride + (int64_t)slot * p.k_row_stride) * 2;
    dma_vp = vbase + (page * p.v_page_stride + (int64_t)slot * p.v_row_stride) * 2;
  };
  auto issue_slice = [&](auto jc) {
    constexpr int j = decltype(jc)::value;
    __builtin_amdgcn_global_load_lds(FG_GLBP(dma_kp + (int64_t)j * KPI * p.k_row_stride * 2 + voff_k[j]), FG_LDSP(dma_dst + j * 1024), 16, 0, 0);
    __builtin_amdgcn_global_load_lds(FG_GLBP(dma_vp + (int64_t)j * KPI * p.v_row_stride * 2 + voff_v[j]), FG_LDSP(dma_dst + OPB + j * 1024), 16, 0, 0);
  };
  auto issue_full = [&](int nb, int stage_off) {
    setup_full(nb, stage_off);
    a_static_for<0, IPW>([&](auto jc) { issue_slice(jc); });
  };
  auto issue_partial = [&](int nb, int stage_off) {
    char* kdst = lds + stage_off + wave_s * (IPW * 1024);
#pragma unroll
    for (int j = 0; j < IPW; ++j) {
      int key = nb * kBN + (wave * IPW + j) * KPI + lane_key;
      key = key < k_len ? key : k_len - 1;
      const int64_t page = btab[key >> page_shift];
      const int slot = key & page_mask;
      const char* kp = kbase + (page * p.k_page_stride + (int64_t)slot * p.k_row_stride) * 2 + lane_c16[j];
      const char* vp = vbase + (page * p.v_page_stride + (int64_t)slot * p.v_row_stride) * 2 + lane_c16[j];
      __builtin_amdgcn_global_load_lds(FG_GLBP(kp), FG_LDSP(kdst + j * 1024), 16, 0, 0);
      __builtin_amdgcn_global_load_lds(FG_GLBP(vp), FG_LDSP(kdst + OPB + j * 1024), 16, 0, 0);
    }
  };
  auto issue_tile = [&](int nb, int stage_off) {
    if (nb * kBN + kBN <= k_len) issue_full(nb, stage_off);
    else issue_partial(nb, stage_off);
  };

  // ---- fragment addresses (lane-constant; the stage offset is added once per step) ------------------------
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
    v_addr0[dt] = lds0 + OPB + v_key0 * RB + v_byte + (((dt * 4) ^ vx0) * 16);
    v_addr1[dt] = lds0 + OPB + (v_key0 + 4) * RB + v_byte + (((dt * 4) ^ vx1) * 16);
  }

  const int wave_row_last = (row0 + kRW - 1 < q_len ? row0 + kRW - 1 : q_len - 1);
  const float sc = a.scale_log2;
  const int col_hi = a.has_right ? (qrow + shift + a.right_off_w < k_len - 1 ? qrow + shift + a.right_off_w : k_len - 1)
                                 : k_len - 1;
  const int col_lo = a.has_left ? qrow + shift - a.left_off_w : 0;

  // ---- pipeline state ------------------------------------------------------------------------------------
  f32x16 s_acc[2][2];   // [head][32-key half of the tile]
  u32x4 pf[2][4];       // [head][16-key quarter]: P as MFMA operand
  float m_use[2] = {0.f, 0.f}, psum[2] = {0.f, 0.f};
  bool ovf_lane = false;
  u32x4 kf[2][4];
  u32x2 vf[2][8];
  // stages of tiles t-1, t, t+1, t+2 (t = -1 at the start: tile 0 sits in stage 0, tile 1 in stage 1)
  uint32_t st_a = 2 * STAGEB, st_b = 3 * STAGEB, st_c = 0, st_d = 1 * STAGEB;

  // One step of the pipeline for tile index t (relative to n_min).
  auto step = [&](int t) __attribute__((always_inline)) {
    constexpr bool PV = true, SM = true, SN = true, MASK = false;
    uint32_t v0s[DT], v1s[DT], kst[KS];
#pragma unroll
    for (int dt = 0; dt < DT; ++dt) {
      v0s[dt] = v_addr0[dt] + st_a;
      v1s[dt] = v_addr1[dt] + st_a;
    }
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) kst[ks] = k_addr[ks] + st_c;
    auto read_v = [&](auto tc, u32x2 (&dst)[8]) {
      constexpr int t4 = decltype(tc)::value;
      a_static_for<0, DT>([&](auto dc) {
        constexpr int dt = decltype(dc)::value;
        dst[2 * dt] = lds_read_tr_b64_imm<t4 * 16 * RB>(v0s[dt]);
        dst[2 * dt + 1] = lds_read_tr_b64_imm<t4 * 16 * RB>(v1s[dt]);
      });
    };
    auto read_k = [&](auto gc, u32x4 (&dst)[4]) {
      constexpr int g = decltype(gc)::value, kt = g / 2;
      a_static_for<0, 4>([&](auto rc) {
        constexpr int r = decltype(rc)::value, ks = (g % 2) * 4 + r;
        dst[r] = lds_read_b128_imm<kt * 32 * RB>(kst[ks]);
      });
    };
    // ---- vector work, in slices ----
    const int key0 = (n_min + t) * kBN;
    float tmax_h = 0.f;
    const int hi_rel = col_hi - key0 - half * 8, lo_rel = col_lo - key0 - half * 8;
    auto score = [&](auto hc, auto ktc, auto ec) {  // raw score of element (kt, e) of head h, masked
      constexpr int h = decltype(hc)::value, kt = decltype(ktc)::value, e = decltype(ec)::value;
      float v = s_acc[h][kt][e];
      if constexpr (MASK) {
        constexpr int rel = kt * 32 + (e >> 3) * 16 + (e & 7);
        v = (rel > hi_rel || (a.has_left && rel < lo_rel)) ? -INFINITY : v;
      }
      return v;
    };
    auto max_part = [&](auto hc) {  // raw maximum of head h over the tile
      float tm = -INFINITY;
      a_static_for<0, 2>([&](auto ktc) {
        a_static_for<0, 16>([&](auto ec) { tm = fmaxf(tm, score(hc, ktc, ec)); });
      });
      tmax_h = tm;
    };
    auto max_fin = [&](auto hc) {
      constexpr int h = decltype(hc)::value;
      const float tm = xhalf_max(tmax_h * sc);
      m_hi[h] = fmaxf(m_hi[h], tm);
      const bool unset = m_ref[h] == -INFINITY;
      ovf_lane = ovf_lane || (!unset && tm > m_ref[h] + kRefLimit);
      m_ref[h] = unset ? tm : m_ref[h];
      m_use[h] = m_ref[h] == -INFINITY ? 0.f : m_ref[h];
    };
    float pv_hold = 0.f;
    auto exp_elem = [&](auto nc) {  // element n of the tile's 64 per lane: quarter n/16, head (n/8)%2, slot n%8
      constexpr int n = decltype(nc)::value;
      constexpr int q = n / 16, h = (n / 8) % 2, i = n % 8, kt = q / 2, idx = (q % 2) * 8 + i;
      const float pv = __builtin_amdgcn_exp2f(fmaf(score(AInt<h>{}, AInt<kt>{}, AInt<idx>{}), sc, -m_use[h]));
      psum[h] += pv;
      if constexpr (i % 2 == 0) pv_hold = pv;
      else pf[h][q][i / 2] = pack_pair<T>(pv_hold, pv);
    };
    bool dma_slices = false;
    auto pin_slice = [&](auto hc, auto qc, auto full_c) {
      constexpr int h = decltype(hc)::value, q = decltype(qc)::value;
      u32x4& done = pf[h][q];
      asm volatile("" : "+v"(psum[h]));
      if constexpr (decltype(full_c)::value != 0) asm volatile("" : "+v"(done));
    };
    // slice (o, r): what the vector ALU does next to pair r of MFMA group o
    auto valu = [&](auto oc, auto rc) {
      constexpr int o = decltype(oc)::value, r = decltype(rc)::value;
      if constexpr (SM) {
        if constexpr (o == 0) {
          if constexpr (r == 0) max_part(AInt<0>{});
          if constexpr (r == 1) max_fin(AInt<0>{});
          if constexpr (r == 2) max_part(AInt<1>{});
          if constexpr (r == 3) max_fin(AInt<1>{});
          if constexpr (r == 0 || r == 2) asm volatile("" : "+v"(tmax_h));
          if constexpr (r == 1 || r == 3) asm volatile("" : "+v"(m_use[r / 2]));
        } else if constexpr (o == 1 || o == 2 || o == 4 || o == 5) {
          // quarters 0 and 1 next to the accumulation, 2 and 3 next to the first half of the new scores (which
          // overwrites the half of S that quarters 0 and 1 have read)
          constexpr int q = o < 3 ? o - 1 : o - 2;
          a_static_for<0, 4>([&](auto jc) { exp_elem(AInt<q * 16 + r * 4 + decltype(jc)::value>{}); });
          // keep the slice here: its results are only used in the next step, and the compiler would otherwise
          // sink the whole softmax below the barrier, behind the MFMAs it is meant to run next to
          pin_slice(AInt<r / 2>{}, AInt<q>{}, AInt<r % 2>{});
        } else if constexpr (o == 6) {
          if (dma_slices) issue_slice(rc);
        }
      }
    };

    // ---- groups 0..3: O^T += V(t-1)^T . P(t-1)^T, quarter t4 of the keys per group ----
    a_static_for<0, 4>([&](auto tc) {
      constexpr int t4 = decltype(tc)::value;
      if constexpr (PV) {
        lds_wait_all(vf[t4 & 1]);
        if constexpr (t4 + 1 < 4) read_v(AInt<t4 + 1>{}, vf[(t4 + 1) & 1]);
      }
      a_static_for<0, DT>([&](auto dc) {
        constexpr int dt = decltype(dc)::value;
        if constexpr (PV) {
          const u32x4 both = {vf[t4 & 1][2 * dt][0], vf[t4 & 1][2 * dt][1], vf[t4 & 1][2 * dt + 1][0], vf[t4 & 1][2 * dt + 1][1]};
          o_acc[0][dt] = AttnMfma<T>::mma(__builtin_bit_cast(Frag, both), __builtin_bit_cast(Frag, pf[0][t4]), o_acc[0][dt]);
          o_acc[1][dt] = AttnMfma<T>::mma(__builtin_bit_cast(Frag, both), __builtin_bit_cast(Frag, pf[1][t4]), o_acc[1][dt]);
        }
        valu(tc, dc);
        __builtin_amdgcn_sched_barrier(0);
      });
    });
    // ---- tile t+1 has landed everywhere (tile t+2 may still be in flight: 2 * IPW copies per wave);
    // the stage of tile t-1 is free for tile t+3 ----
    if constexpr (SN) {
      if (t + 2 < NT) FG_WAIT_VM(2 * IPW);
      else FG_WAIT_VM(0);
      __builtin_amdgcn_s_barrier();
      dma_slices = false;
      if (t + 3 < NT) {
        const int nb = n_min + t + 3;
        if (nb * kBN + kBN <= k_len) {
          setup_full(nb, (int)st_a);  // copied slice by slice next to the MFMAs of group 6
          dma_slices = true;
        } else {
          issue_partial(nb, (int)st_a);
        }
      }
      read_k(AInt<0>{}, kf[0]);
    }

    __builtin_amdgcn_sched_barrier(0);
    // ---- groups 4..7: S(t+1)^T = K(t+1) . Q^T ----
    a_static_for<0, 4>([&](auto gc) {
      constexpr int g = decltype(gc)::value, kt = g / 2;
      if constexpr (SN) {
        lds_wait_k(kf[g & 1]);
        if constexpr (g + 1 < 4) {
          read_k(AInt<g + 1>{}, kf[(g + 1) & 1]);
        } else {
          // first V group of the next step: V(t) sits in stage b
#pragma unroll
          for (int dt = 0; dt < DT; ++dt) {
            v0s[dt] = v_addr0[dt] + st_b;
            v1s[dt] = v_addr1[dt] + st_b;
          }
          read_v(AInt<0>{}, vf[0]);
        }
      }
      a_static_for<0, 4>([&](auto rc) {
        constexpr int r = decltype(rc)::value, ks = (g % 2) * 4 + r;
        if constexpr (SN) {
          if constexpr (ks == 0) {
            PairMfma<T>::first(s_acc[0][kt], kf[g & 1][r], qf[0][ks]);
            PairMfma<T>::first(s_acc[1][kt], kf[g & 1][r], qf[1][ks]);
          } else {
            PairMfma<T>::next(s_acc[0][kt], kf[g & 1][r], qf[0][ks]);
            PairMfma<T>::next(s_acc[1][kt], kf[g & 1][r], qf[1][ks]);
          }
        }
        valu(AInt<4 + g>{}, rc);
        __builtin_amdgcn_sched_barrier(0);
      });
    });
    if constexpr (!SN && SM) {
      // no S group ran: the first V group of the final accumulation still has to be fetched
#pragma unroll
      for (int dt = 0; dt < DT; ++dt) {
        v0s[dt] = v_addr0[dt] + st_b;
        v1s[dt] = v_addr1[dt] + st_b;
      }
      read_v(AInt<0>{}, vf[0]);
    }
    const uint32_t tmp = st_a;
    st_a = st_b;
    st_b = st_c;
    st_c = st_d;
    st_d = tmp;
  };

  auto tile_needs_mask = [&](int t) {
    const int key0 = (n_min + t) * kBN;
    return (key0 + kBN > k_len) || (a.has_right && key0 + kBN - 1 > row0 + shift + a.right_off_w) ||
           (a.has_left && key0 < wave_row_last + shift - a.left_off_w);
  };

  // The loop runs the same step for t = -1 .. NT.  Step -1 only has S(0) to compute and step NT only the
  // last accumulation; their other halves run on neutral data instead of being compiled as variants of
  // their own (every variant costs the register allocator dearly): the scores start at -inf and P at zero,
  // the V halves of the two stages that no tile has reached yet are zero-filled, tile NT is masked as a whole.
#pragma unroll
  for (int h = 0; h < 2; ++h) {
#pragma unroll
    for (int dt = 0; dt < DT; ++dt)
#pragma unroll
      for (int e = 0; e < 16; ++e) o_acc[h][dt][e] = 0.f;
#pragma unroll
    for (int kt = 0; kt < 2; ++kt)
#pragma unroll
      for (int e = 0; e < 16; ++e) s_acc[h][kt][e] = -INFINITY;
#pragma unroll
    for (int q = 0; q < 4; ++q) pf[h][q] = u32x4{0u, 0u, 0u, 0u};
  }
  if (NT > 0) {  // (a block whose rows see no key at all has no tiles: its output is zero, its lse +inf)
    {
      const u32x4 z = {0u, 0u, 0u, 0u};
#pragma unroll
      for (int i = 0; i < 2 * OPB / (256 * 16); ++i) {
        const int o = (i * 256 + tid) * 16;  // byte o of the two V halves, OPB bytes each
        *reinterpret_cast<u32x4*>(lds + (2 + o / OPB) * STAGEB + OPB + o % OPB) = z;
      }
    }
    issue_tile(n_min, 0);
    if (NT > 1) issue_tile(n_min + 1, STAGEB);
    __syncthreads();
    a_static_for<0, DT>([&](auto dc) {
      constexpr int dt = decltype(dc)::value;
      vf[0][2 * dt] = lds_read_tr_b64_imm<0>(v_addr0[dt] + st_a);
      vf[0][2 * dt + 1] = lds_read_tr_b64_imm<0>(v_addr1[dt] + st_a);
    });
    for (int t = -1; t <= NT; ++t) {
      if (t == NT || (t >= 0 && tile_needs_mask(t))) {
        // masked scores of tile t, in place (a tile on the diagonal or at the end of the keys; tile NT as a whole)
        const int key0 = (n_min + t) * kBN;
        const int hi_rel = col_hi - key0 - half * 8, lo_rel = col_lo - key0 - half * 8;
        mfma_settle();  // the last MFMAs of the step before wrote these scores
#pragma unroll
        for (int h = 0; h < 2; ++h)
#pragma unroll
          for (int kt = 0; kt < 2; ++kt)
#pragma unroll
            for (int e = 0; e < 16; ++e) {
              const int rel = kt * 32 + (e >> 3) * 16 + (e & 7);
              s_acc[h][kt][e] = (rel > hi_rel || (a.has_left && rel < lo_rel)) ? -INFINITY : s_acc[h][kt][e];
            }
      }
      step(t);
    }
    // a score left the headroom above its row's reference: this block has to be redone
    if (__builtin_amdgcn_ballot_w64(ovf_lane) != 0 && lane == 0)
      (void)__hip_atomic_fetch_or(redo_flag, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  }

  // ---- epilogue --------------------------------------------------------------------------------------
  if (qrow >= q_len) return;
#pragma unroll
  for (int h = 0; h < 2; ++h) {
    const float lr = xhalf_sum(psum[h]);
    const bool empty = lr == 0.f || lr != lr;
    const float inv = empty ? 1.f : 1.f / lr;
    if (p.lse != nullptr && half == 0) {
      p.lse[(int64_t)(head0 + h) * p.total_q + q_bos + qrow] = empty ? INFINITY : m_use[h] * 0.6931471805599453f + logf(lr);
    }
    T* op = (T*)p.out + (int64_t)(q_bos + qrow) * p.o_row_stride + (int64_t)(head0 + h) * p.o_head_stride;
#pragma unroll
    for (int dt = 0; dt < DT; ++dt)
#pragma unroll
      for (int g = 0; g < 4; ++g) {
        const int d = dt * 32 + g * 8 + half * 4;
        Pack<T, 4> o;
#pragma unroll
        for (int e = 0; e < 4; ++e) o.v[e] = (T)(o_acc[h][dt][g * 4 + e] * inv);
        st_pack<T, 4>(op + d, o);
      }
  }
}

template <typename T, int D>
int launch_pair(const AttnArgs& a, dim3 grid, hipStream_t st) {
  constexpr int LDS_BYTES = 4 * 2 * kBN * 2 * D;  // four stages
  static hipError_t attr_err = hipFuncSetAttribute(reinterpret_cast<const void*>(attn_varlen_pair_kernel<T, D>),
                                                   hipFuncAttributeMaxDynamicSharedMemorySize, LDS_BYTES);
  if (attr_err != hipSuccess) {
    fg_set_error("flash_attn_varlen_fwd: cannot reserve %d bytes of LDS: %s", LDS_BYTES, hipGetErrorString(attr_err));
    return FG_ERR_LAUNCH;
  }
  hipLaunchKernelGGL((attn_varlen_pair_kernel<T, D>), grid, dim3(256), LDS_BYTES, st, a);
  return fg_check_launch("flash_attn_varlen_fwd");
}
