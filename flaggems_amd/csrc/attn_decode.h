// Paged attention for single-token queries (decode): every sequence contributes one query row per
// head.  The work is a stream over the K/V cache, so the kernel is organised around bytes in flight,
// not around the matrix cores:
//   * a workgroup takes one (sequence, KV head, key range); the G = Hq/Hk query heads that share the
//     KV head are the rows of one 32-row MFMA block (rows >= G are zero), so each K/V byte is read
//     once for the whole group -- the query-group / sequence swap of the reference's launch code
//     (src/flag_gems/ops/flash_api.py:313-345);
//   * each of the 4 waves streams its own 32-key tiles (tile t of the range goes to wave t mod 4)
//     through its own two LDS stages by global_load_lds and keeps its own running maximum, sum and
//     output; no barrier in the loop, the four states are merged once at the end through LDS;
//   * long sequences (or few of them) are cut into key ranges over the x dimension of the grid
//     ("split-KV"); a range then leaves its unnormalised output and (maximum, sum) in a workspace and
//     a second kernel merges the ranges.  A range holds at most 256 pages, whose ids sit in four
//     registers (a lane each) loaded before the loop.
// MFMA formulation, LDS row layout (swz) and the base-2 online softmax are those of the prefill
// kernels.  Conditions (checked on the host): head dim 64 or 128, page size a power of two >= 16,
// max_seqlen_q == 1, G <= 32, no ALiBi, no soft-cap, no left window.
// This header is included by attn_varlen.hip inside its unnamed namespace, after attn_pipe.h.

struct DecodeArgs {
  FgFlashParams p;
  float scale_log2;
  int page_shift;
  int group;             // query heads per KV head
  int splits;            // key ranges per sequence (grid x)
  int tiles_per_split;   // most 32-key tiles per range, a multiple of 4 (cut for max_seqlen_k)
  int min_tiles;         // fewest 32-key tiles per range of a shorter sequence, a multiple of 4
  float* part_o;         // [splits][batch][Hq][D] fp32, unnormalised   (splits > 1)
  float* part_ml;        // [splits][batch][Hq][2] fp32: maximum (base 2), sum
};

constexpr int kDecTile = 32;  // keys per wave tile

// Tiles per key range of one sequence.  The host cuts the ranges for max_seqlen_k, which it knows; a sequence
// may be much shorter (a batch with one long sequence, or a caller that passes the model's limit), and with the
// host's cut its keys would fill the first range or two and leave the other workgroups of the sequence without
// work.  So each sequence spreads its own tiles over all `splits` ranges, down to `min_tiles` per range.
__device__ inline int decode_range_tiles(const DecodeArgs& a, int tiles_total) {
  int t = (tiles_total + a.splits - 1) / a.splits;
  t = (t + 3) & ~3;
  t = t < a.min_tiles ? a.min_tiles : t;
  return t < a.tiles_per_split ? t : a.tiles_per_split;
}
// cache-policy bits of the K/V tile loads: non-temporal, every byte of the cache is read once per launch
// (measured 5.4 -> 5.7-5.9 TB/s on 64 x 4096 keys, 5.7 -> 6.2 on 256 x 2048)
constexpr int kDecLoadAux = 2;

template <typename T, int D>
__global__ __launch_bounds__(256) void attn_decode_kernel(DecodeArgs a) {
  typedef typename AttnMfma<T>::Frag Frag;
  constexpr int RB = 2 * D;                 // bytes per key row in LDS
  constexpr int CPR = RB / 16;              // 16-byte chunks per row
  constexpr int KS = D / 16;                // MFMA k-steps over the head dim
  constexpr int DT = D / 32;                // 32-row output sub-tiles over the head dim
  constexpr int OPB = kDecTile * RB;        // one operand tile of one wave
  constexpr int STAGEB = 2 * OPB;           // K tile + V tile
  constexpr int WAVEB = 2 * STAGEB;         // two stages
  constexpr int KPI = 1024 / RB;            // key rows per DMA instruction (4 / 8)
  constexpr int NI = kDecTile / KPI;        // DMA instructions per operand tile (8 / 4)
  extern __shared__ __attribute__((aligned(16))) char lds[];

  const FgFlashParams& p = a.p;
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int half = lane >> 5, ql = lane & 31;
  const int b = blockIdx.y, kvh = blockIdx.z;
  // Key range, rotated per (sequence, KV head): workgroups go round-robin to the 8 XCDs by their linear id, and a
  // short sequence has work in range 0 only, so with 8 ranges every short sequence of a batch would land on one XCD.
  const int split = (int)((blockIdx.x + (unsigned)(b * 5 + kvh * 3)) % gridDim.x);
  const int G = a.group;

  const int q_bos = p.cu_seqlens_q[b];
  const int q_len = p.cu_seqlens_q[b + 1] - q_bos;
  const int k_len = p.seqused_k[b];
  const int tiles_total = (k_len + kDecTile - 1) / kDecTile;
  const int range_tiles = decode_range_tiles(a, tiles_total);
  const int t_begin = split * range_tiles;
  int t_end = t_begin + range_tiles;
  t_end = t_end < tiles_total ? t_end : tiles_total;
  // exactly one query token: in a mixed batch the sequences with more belong to the prefill kernels
  if (q_len != 1) return;
  // a key range past the end of this sequence: nothing to do, and the merge does not read its partial results
  // (range 0 always reports, so that a sequence without keys still gets its zeros)
  if (split > 0 && t_begin >= t_end) return;
  const bool has_work = t_begin < t_end;

#if !FG_V_DECODE_Q_EARLY
  // ---- Q fragments: row r < G is query head kvh*G + r of this sequence's token; other rows are zero ---------
  Frag qf[KS];
  {
    const bool row_ok = ql < G && q_len == 1;
    const T* qp = (const T*)p.q + (int64_t)q_bos * p.q_row_stride + (int64_t)(kvh * G + (row_ok ? ql : 0)) * p.q_head_stride;
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) {
      u32x4 v = {0u, 0u, 0u, 0u};
      if (row_ok) v = *reinterpret_cast<const u32x4*>(qp + ks * 16 + half * 8);
      qf[ks] = __builtin_bit_cast(Frag, v);
    }
  }
#endif
  f32x16 o_acc[DT];
#pragma unroll
  for (int dt = 0; dt < DT; ++dt)
#pragma unroll
    for (int e = 0; e < 16; ++e) o_acc[dt][e] = 0.f;
  float m_run = -INFINITY, l_run = 0.f;

  // ---- page ids of the range: lane l of pgc[r] <- block_table[first page of the range + 64 r + l] ------------
  const int32_t* btab = p.block_table + (int64_t)b * p.block_table_stride;
  const int page_shift = a.page_shift, page_mask = p.page_size - 1;
  const int last_page = k_len > 0 ? (k_len - 1) >> page_shift : 0;
  const int pg_first = (t_begin * kDecTile) >> page_shift;
  int pgc[4];
#pragma unroll
  for (int r = 0; r < 4; ++r) {
    int pg = pg_first + r * 64 + lane;
    pg = pg < last_page ? pg : last_page;
    pgc[r] = has_work ? btab[pg] : 0;
  }
  const int last_page_id = has_work ? btab[last_page] : 0;
#if FG_V_DECODE_Q_EARLY
  // ---- Q fragments (variant FG_V_DECODE_Q_EARLY, variants.h): row r < G is query head kvh*G + r of this
  // sequence's token; other rows are zero.
  // Requested unconditionally (qp is clamped to a row that exists) together with the page ids, and not touched
  // before the one wait below: under a branch of its own each load was waited for before the next request, and the
  // page ids went out a trip later.
  const bool q_row_ok = ql < G && q_len == 1;
  u32x4 qraw[KS];
  {
    const T* qp = (const T*)p.q + (int64_t)q_bos * p.q_row_stride + (int64_t)(kvh * G + (q_row_ok ? ql : 0)) * p.q_head_stride;
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) qraw[ks] = *reinterpret_cast<const u32x4*>(qp + ks * 16 + half * 8);
  }
#endif
  // Everything loaded so far is complete from here on (stated explicitly: once tile DMAs are in flight the
  // compiler could only wait for all of them together with these loads).
  FG_WAIT_VM(0);
#if FG_V_DECODE_Q_EARLY
  Frag qf[KS];
#pragma unroll
  for (int ks = 0; ks < KS; ++ks) {
    u32x4 v = qraw[ks];
    asm volatile("" : "+v"(v));  // (keeps the zeroing, and with it a wait of the compiler's own, behind the wait above)
    if (!q_row_ok) v = u32x4{0u, 0u, 0u, 0u};
    qf[ks] = __builtin_bit_cast(Frag, v);
  }
#endif

  const char* kbase = (const char*)((const T*)p.k_cache + (int64_t)kvh * p.k_head_stride);
  const char* vbase = (const char*)((const T*)p.v_cache + (int64_t)kvh * p.v_head_stride);
  const int lane_key = lane / CPR, lane_pos = lane % CPR;
  int c16[NI];  // the lane's swizzled chunk per instruction
#pragma unroll
  for (int j = 0; j < NI; ++j) c16[j] = (lane_pos ^ swz<CPR>(j * KPI + lane_key)) * 16;
  const uint32_t krow_off = (uint32_t)(lane_key * (int)p.k_row_stride * 2);
  const uint32_t vrow_off = (uint32_t)(lane_key * (int)p.v_row_stride * 2);
  char* const my_lds = lds + wave * WAVEB;

  // one 32-key tile (K and V) of this wave into stage `stage`
  auto issue_tile = [&](int t, int stage) {
    char* kdst = my_lds + stage * STAGEB;
    const bool full = t * kDecTile + kDecTile <= k_len;
    const char* klast = kbase + ((int64_t)last_page_id * p.k_page_stride + (int64_t)((k_len - 1) & page_mask) * p.k_row_stride) * 2;
    const char* vlast = vbase + ((int64_t)last_page_id * p.v_page_stride + (int64_t)((k_len - 1) & page_mask) * p.v_row_stride) * 2;
#pragma unroll
    for (int j = 0; j < NI; ++j) {
      const int key = t * kDecTile + j * KPI;                 // first key of the instruction (scalar)
      const int pi = (key >> page_shift) - pg_first;          // page index within the range, < 256
      const int sel = pi >> 6;
      const int pv = sel == 0 ? pgc[0] : (sel == 1 ? pgc[1] : (sel == 2 ? pgc[2] : pgc[3]));
      const int64_t page = __builtin_amdgcn_readlane(pv, pi & 63);
      const int slot = key & page_mask;
      const char* kp = kbase + (page * p.k_page_stride + (int64_t)slot * p.k_row_stride) * 2;
      const char* vp = vbase + (page * p.v_page_stride + (int64_t)slot * p.v_row_stride) * 2;
      if (full) {
        __builtin_amdgcn_global_load_lds(FG_GLBP(kp + (krow_off + c16[j])), FG_LDSP(kdst + j * 1024), 16, 0, kDecLoadAux);
        __builtin_amdgcn_global_load_lds(FG_GLBP(vp + (vrow_off + c16[j])), FG_LDSP(kdst + OPB + j * 1024), 16, 0, kDecLoadAux);
      } else {
        // rows past the end read the last valid key instead (their scores are masked; stale cache contents
        // must not reach the accumulators)
        const bool valid = key + lane_key < k_len;
        const char* ks = valid ? kp + (krow_off + c16[j]) : klast + c16[j];
        const char* vs = valid ? vp + (vrow_off + c16[j]) : vlast + c16[j];
        __builtin_amdgcn_global_load_lds(FG_GLBP(ks), FG_LDSP(kdst + j * 1024), 16, 0, kDecLoadAux);
        __builtin_amdgcn_global_load_lds(FG_GLBP(vs), FG_LDSP(kdst + OPB + j * 1024), 16, 0, kDecLoadAux);
      }
    }
  };

  // ---- fragment addresses (lane constants; stage and sub-tile offsets are immediates) ------------------------
  const uint32_t lds0 = lds_off(my_lds);
  const int k_row = sigma(ql);
  const int kx = half ^ swz<CPR>(k_row);
  uint32_t k_addr[KS];
#pragma unroll
  for (int ks = 0; ks < KS; ++ks) k_addr[ks] = lds0 + k_row * RB + (((ks * 2) ^ kx) * 16);
  const int vs_ = lane & 15;
  const int v_key0 = half * 8 + (vs_ >> 2);
  const int v_cc = 2 * ((lane >> 4) & 1) + ((vs_ & 3) >> 1);
  const int v_byte = (vs_ & 1) * 8;
  const int vx0 = v_cc ^ swz<CPR>(v_key0), vx1 = v_cc ^ swz<CPR>(v_key0 + 4);
  uint32_t v_addr0[DT], v_addr1[DT];
#pragma unroll
  for (int dt = 0; dt < DT; ++dt) {
    v_addr0[dt] = lds0 + OPB + v_key0 * RB + v_byte + (((dt * 4) ^ vx0) * 16);
    v_addr1[dt] = lds0 + OPB + (v_key0 + 4) * RB + v_byte + (((dt * 4) ^ vx1) * 16);
  }
  const float sc = a.scale_log2;

  auto tile = [&](int t, auto stage_c) {
    constexpr int S = decltype(stage_c)::value;
    // this wave's DMAs for tile t have landed once only those of the tile after it are outstanding
    if (t + 4 < t_end) {
      issue_tile(t + 4, S ^ 1);
      FG_WAIT_VM(2 * NI);
    } else {
      FG_WAIT_VM(0);
    }
    // ---- S^T = K . Q^T for 32 keys --------------------------------------------------------------------------
    f32x16 s_acc;
#pragma unroll
    for (int e = 0; e < 16; ++e) s_acc[e] = 0.f;
    u32x4 kf[8];
    if constexpr (KS < 8) {
#pragma unroll
      for (int i = KS; i < 8; ++i) kf[i] = u32x4{0u, 0u, 0u, 0u};
    }
    a_static_for<0, KS>([&](auto kc) {
      constexpr int ks = decltype(kc)::value;
      kf[ks] = lds_read_b128_imm<S * STAGEB>(k_addr[ks]);
    });
    lds_wait_all(kf);
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) s_acc = AttnMfma<T>::mma(__builtin_bit_cast(Frag, kf[ks]), qf[ks], s_acc);
    // V fragments of the first output sub-tiles are requested now and arrive under the softmax arithmetic
    u32x2 vf[2][8];
    auto issue_v = [&](auto dc, u32x2 (&dst)[8]) {
      constexpr int dt = decltype(dc)::value;
      a_static_for<0, 2>([&](auto tc) {
        constexpr int t4 = decltype(tc)::value;
        dst[2 * t4] = lds_read_tr_b64_imm<S * STAGEB + t4 * 16 * RB>(v_addr0[dt]);
        dst[2 * t4 + 1] = lds_read_tr_b64_imm<S * STAGEB + t4 * 16 * RB>(v_addr1[dt]);
      });
#pragma unroll
      for (int i = 4; i < 8; ++i) dst[i] = u32x2{0u, 0u};
    };
    issue_v(AInt<0>{}, vf[0]);
    // ---- mask keys past the end; running maximum --------------------------------------------------------------
    const int key0 = t * kDecTile;
    if (key0 + kDecTile > k_len) {
      const int hi_rel = k_len - 1 - key0 - half * 8;   // element e is key key0 + half*8 + (e>>3)*16 + (e&7)
#pragma unroll
      for (int e = 0; e < 16; ++e) {
        const int rel = (e >> 3) * 16 + (e & 7);
        s_acc[e] = rel > hi_rel ? -INFINITY : s_acc[e];
      }
    }
    float tmax = -INFINITY;
#pragma unroll
    for (int e = 0; e < 16; ++e) tmax = fmaxf(tmax, s_acc[e]);
    tmax *= sc;
    tmax = xhalf_max(tmax);
    const bool moved = tmax > m_run + 8.0f;
    const float m_new = moved ? tmax : m_run;
    const float m_use = m_new == -INFINITY ? 0.f : m_new;
    const float alpha = moved ? __builtin_amdgcn_exp2f(m_run - m_use) : 1.0f;
    float psum = 0.f;
    Frag pf[2];
#pragma unroll
    for (int t2 = 0; t2 < 2; ++t2) {
      T tmp[8];
#pragma unroll
      for (int e = 0; e < 8; ++e) {
        const float pv = __builtin_amdgcn_exp2f(fmaf(s_acc[t2 * 8 + e], sc, -m_use));
        psum += pv;
        tmp[e] = (T)pv;
      }
      pf[t2] = *reinterpret_cast<Frag*>(tmp);
    }
    psum = xhalf_sum(psum);
    l_run = l_run * alpha + psum;
    m_run = m_new;
    if (__builtin_amdgcn_ballot_w64(moved) != 0) {
#pragma unroll
      for (int dt = 0; dt < DT; ++dt)
#pragma unroll
        for (int e = 0; e < 16; ++e) o_acc[dt][e] *= alpha;
    }
    // ---- O^T += V^T . P^T (two k-steps of 16 keys per output sub-tile) ----------------------------------------
    a_static_for<0, DT>([&](auto dc) {
      constexpr int dt = decltype(dc)::value;
      lds_wait_all(vf[dt & 1]);
      if constexpr (dt + 1 < DT) issue_v(AInt<dt + 1>{}, vf[(dt + 1) & 1]);
#pragma unroll
      for (int t4 = 0; t4 < 2; ++t4) {
        const u32x4 both = {vf[dt & 1][2 * t4][0], vf[dt & 1][2 * t4][1], vf[dt & 1][2 * t4 + 1][0], vf[dt & 1][2 * t4 + 1][1]};
        o_acc[dt] = AttnMfma<T>::mma(__builtin_bit_cast(Frag, both), pf[t4], o_acc[dt]);
      }
    });
  };

  if (has_work) {
    const int t0 = t_begin + wave;
    if (t0 < t_end) issue_tile(t0, 0);
    for (int t = t0; t < t_end; t += 8) {
      tile(t, AInt<0>{});
      if (t + 4 < t_end) tile(t + 4, AInt<1>{});
    }
  }

  // ---- merge the four waves through LDS: (m, l) per row first, then the rescaled outputs -------------------------
  __syncthreads();  // every wave is done with its tile stages
  float* ml = reinterpret_cast<float*>(lds);                 // [4 waves][32 rows][2]
  float* osum = reinterpret_cast<float*>(lds) + 256;         // [4 waves][G rows][D]
  if (half == 0) {
    ml[(wave * 32 + ql) * 2] = m_run;
    ml[(wave * 32 + ql) * 2 + 1] = l_run;
  }
  __syncthreads();
  float m_all = -INFINITY;
#pragma unroll
  for (int w = 0; w < 4; ++w) m_all = fmaxf(m_all, ml[(w * 32 + ql) * 2]);
  float l_all = 0.f;
#pragma unroll
  for (int w = 0; w < 4; ++w) {
    const float mw = ml[(w * 32 + ql) * 2];
    l_all += mw == -INFINITY ? 0.f : ml[(w * 32 + ql) * 2 + 1] * __builtin_amdgcn_exp2f(mw - m_all);
  }
  const float my_scale = m_run == -INFINITY ? 0.f : __builtin_amdgcn_exp2f(m_run - m_all);
  if (ql < G) {
#pragma unroll
    for (int dt = 0; dt < DT; ++dt)
#pragma unroll
      for (int g = 0; g < 4; ++g)
#pragma unroll
        for (int e = 0; e < 4; ++e) osum[(wave * G + ql) * D + dt * 32 + g * 8 + half * 4 + e] = o_acc[dt][g * 4 + e] * my_scale;
  }
  __syncthreads();
  if (q_len != 1) return;
  // thread i sums element i of the [G][D] block over the waves
  for (int i = tid; i < G * D; i += 256) {
    const int r = i / D, d = i - r * D;
    const float o = osum[(0 * G + r) * D + d] + osum[(1 * G + r) * D + d] + osum[(2 * G + r) * D + d] + osum[(3 * G + r) * D + d];
    float mr = -INFINITY, lr = 0.f;
#pragma unroll
    for (int w = 0; w < 4; ++w) mr = fmaxf(mr, ml[(w * 32 + r) * 2]);
#pragma unroll
    for (int w = 0; w < 4; ++w) {
      const float mw = ml[(w * 32 + r) * 2];
      lr += mw == -INFINITY ? 0.f : ml[(w * 32 + r) * 2 + 1] * __builtin_amdgcn_exp2f(mw - mr);
    }
    const int head = kvh * G + r;
    if (a.splits == 1) {
      const bool empty = lr == 0.f || lr != lr;
      ((T*)p.out)[(int64_t)q_bos * p.o_row_stride + (int64_t)head * p.o_head_stride + d] = (T)(empty ? 0.f : o / lr);
      if (d == 0 && p.lse != nullptr)
        p.lse[(int64_t)head * p.total_q + q_bos] = empty ? INFINITY : mr * 0.6931471805599453f + logf(lr);
    } else {
      const int64_t row = ((int64_t)split * p.batch + b) * p.Hq + head;
      a.part_o[row * D + d] = o;
      if (d == 0) {
        a.part_ml[row * 2] = mr;
        a.part_ml[row * 2 + 1] = lr;
      }
    }
  }
  (void)l_all;
}

// Merges the key ranges of a sequence: one thread per (sequence, head, d).
template <typename T>
__global__ __launch_bounds__(256) void attn_decode_combine_kernel(DecodeArgs a) {
  const FgFlashParams& p = a.p;
  const int D = p.D;
  const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
  const int64_t total = (int64_t)p.batch * p.Hq * D;
  if (i >= total) return;
  const int d = (int)(i % D);
  const int64_t bh = i / D;
  const int head = (int)(bh % p.Hq);
  const int b = (int)(bh / p.Hq);
  const int q_bos = p.cu_seqlens_q[b];
  if (p.cu_seqlens_q[b + 1] - q_bos != 1) return;
  // key ranges that hold keys of this sequence (the others were not written)
  const int tiles_total = (p.seqused_k[b] + kDecTile - 1) / kDecTile;
  const int range_tiles = decode_range_tiles(a, tiles_total);
  int ns = (tiles_total + range_tiles - 1) / range_tiles;
  ns = ns < 1 ? 1 : (ns > a.splits ? a.splits : ns);
  float m = -INFINITY;
  for (int s = 0; s < ns; ++s) m = fmaxf(m, a.part_ml[(((int64_t)s * p.batch + b) * p.Hq + head) * 2]);
  float l = 0.f, o = 0.f;
  for (int s = 0; s < ns; ++s) {
    const int64_t row = ((int64_t)s * p.batch + b) * p.Hq + head;
    const float ms = a.part_ml[row * 2];
    if (ms == -INFINITY) continue;
    const float w = exp2f(ms - m);
    l += a.part_ml[row * 2 + 1] * w;
    o += a.part_o[row * D + d] * w;
  }
  const bool empty = l == 0.f || l != l;
  ((T*)p.out)[(int64_t)q_bos * p.o_row_stride + (int64_t)head * p.o_head_stride + d] = (T)(empty ? 0.f : o / l);
  if (d == 0 && p.lse != nullptr) p.lse[(int64_t)head * p.total_q + q_bos] = empty ? INFINITY : m * 0.6931471805599453f + logf(l);
}

// Key ranges per sequence: enough to hand every CU about two workgroups, never more than 256 pages
// (and 4096 keys) per range, never fewer than 512 keys per range.
inline void decode_plan(const FgFlashParams& p, int page_shift, int num_cu, int* splits, int* tiles_per_split) {
  const int64_t max_k = p.max_seqlen_k > 0 ? p.max_seqlen_k : 1;
  const int64_t range_cap = (int64_t)256 << page_shift < 4096 ? (int64_t)256 << page_shift : 4096;  // keys
  int64_t need = fg_cdiv(max_k, range_cap);
  const int64_t wgs = (int64_t)p.batch * p.Hk;
  int per_cu = 2;
  if (fg_options().decode_wg_per_cu > 0) per_cu = fg_options().decode_wg_per_cu;
  int64_t want = fg_cdiv((int64_t)per_cu * num_cu, wgs > 0 ? wgs : 1);
  const int64_t most = max_k / 512 > 1 ? max_k / 512 : 1;
  if (want > most) want = most;
  int64_t s = need > want ? need : want;
  int64_t tps = fg_cdiv(fg_cdiv(max_k, kDecTile), s);
  tps = (tps + 3) / 4 * 4;
  s = fg_cdiv(fg_cdiv(max_k, kDecTile), tps);
  *splits = (int)(s > 0 ? s : 1);
  *tiles_per_split = (int)tps;
}

inline size_t decode_workspace_bytes(const FgFlashParams& p, int splits) {
  if (splits <= 1) return 0;
  return (size_t)splits * p.batch * p.Hq * ((size_t)p.D + 2) * sizeof(float);
}

template <typename T, int D>
int launch_decode(const DecodeArgs& a, hipStream_t st) {
  constexpr int LDS_BYTES = 4 * 2 * 2 * kDecTile * 2 * D;  // 4 waves x 2 stages x (K + V) tile
  static hipError_t attr_err = hipFuncSetAttribute(reinterpret_cast<const void*>(attn_decode_kernel<T, D>),
                                                   hipFuncAttributeMaxDynamicSharedMemorySize, LDS_BYTES);
  if (attr_err != hipSuccess) {
    fg_set_error("flash_attn_varlen_fwd: cannot reserve %d bytes of LDS: %s", LDS_BYTES, hipGetErrorString(attr_err));
    return FG_ERR_LAUNCH;
  }
  const FgFlashParams& p = a.p;
  hipLaunchKernelGGL((attn_decode_kernel<T, D>), dim3((unsigned)a.splits, (unsigned)p.batch, (unsigned)p.Hk), dim3(256),
                     LDS_BYTES, st, a);
  if (a.splits > 1) {
    const int64_t total = (int64_t)p.batch * p.Hq * D;
    hipLaunchKernelGGL((attn_decode_combine_kernel<T>), dim3((unsigned)fg_cdiv(total, 256)), dim3(256), 0, st, a);
  }
  return fg_check_launch("flash_attn_varlen_fwd");
}
