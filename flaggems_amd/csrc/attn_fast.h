// Paged varlen attention forward, lean variant of the asynchronous-tile kernel for the common case:
// head dim 64 or 128, page size a power of two >= 16, at most 8192 keys per sequence, no ALiBi, no
// soft-cap.  Same work split, MFMA formulation, LDS layout and online softmax as
// attn_varlen_async_kernel (4 waves x 32 query rows, 64-key tiles, two LDS stages); what differs is
// that nothing address-like is recomputed per tile on the vector ALU, which the general kernel
// spends more time on than on the softmax itself:
//   * A wave moves 16 consecutive key rows of every tile, which lie in one page.  So the page id and
//     the row base are wave-uniform: the ids of all tiles sit in two registers (a lane each), read
//     once before the loop, and become a 64-bit scalar base; each lane adds a 32-bit offset fixed
//     for the whole kernel (its row within the instruction and its swizzled chunk).
//   * The tile loop is unrolled over the two LDS stages, so stage, sub-tile and k-step offsets of
//     every fragment read are instruction immediates on top of 8 + 8 lane-constant registers.
//   * Masking works on the raw scores with one compare and one select per element against a
//     lane-constant bound; interior tiles skip it.
// The last, partial tile of a sequence clamps keys per lane and therefore looks its pages up per
// lane; that path runs once per sequence.
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

template <typename T, int D>
__global__ __launch_bounds__(256, 2) void attn_varlen_fast_kernel(AttnArgs a) {
  typedef typename AttnMfma<T>::Frag Frag;
  constexpr int RB = 2 * D;            // bytes per key row in LDS (no padding for 64 / 128)
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
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);  // scalar: everything derived from it is wave-uniform
  const int half = lane >> 5, ql = lane & 31;
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
  // As the second pass behind the head-pair kernel: only blocks that kernel has marked (its blocks hold two
  // of these in the row direction).
  if (a.redo_rows != 0 &&
      a.redo_flags[((int64_t)blockIdx.z * gridDim.y + blockIdx.y) * a.redo_grid_x + (m_block >> 1)] == 0)
    return;

  const int waves_per_head = 4 / a.hpb;
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
      qf[ks] = __builtin_bit_cast(Frag, v);
    }
  }
  f32x16 o_acc[DT];
#pragma unroll
  for (int dt = 0; dt < DT; ++dt)
#pragma unroll
    for (int e = 0; e < 16; ++e) o_acc[dt][e] = 0.f;
  float m_run = -INFINITY, l_run = 0.f;

  // ---- DMA geometry -----------------------------------------------------------------------------------
  const int wave_s = wave;
  const int32_t* btab = p.block_table + (int64_t)b * p.block_table_stride;
  const char* kbase = (const char*)((const T*)p.k_cache + (int64_t)kv_head * p.k_head_stride);
  const char* vbase = (const char*)((const T*)p.v_cache + (int64_t)kv_head * p.v_head_stride);
  const int page_shift = a.page_shift, page_mask = p.page_size - 1;
  const int lane_key = lane / CPR, lane_pos = lane % CPR;
  uint32_t voff_k[IPW], voff_v[IPW];   // lane-constant byte offsets below an instruction's row base
  int lane_c16[IPW];                   // the lane's swizzled chunk offset alone (partial-tile path)
#pragma unroll
  for (int j = 0; j < IPW; ++j) {
    const int key_l = (wave * IPW + j) * KPI + lane_key;
    const int c = lane_pos ^ swz<CPR>(key_l);
    lane_c16[j] = c * 16;
    voff_k[j] = (uint32_t)(lane_key * (int)p.k_row_stride * 2 + c * 16);
    voff_v[j] = (uint32_t)(lane_key * (int)p.v_row_stride * 2 + c * 16);
  }
  // A wave moves 16 consecutive key rows of every tile (IPW * KPI), which lie in one page (page size
  // >= 16): one page id per wave and tile.  The ids of tiles n_min + l (pg_cache0) and n_min + 64 + l
  // (pg_cache1) sit in lane l of two registers, loaded once, so that no load is left in the tile loop
  // (it would be ordered behind the tile DMAs); the id of a tile is a v_readlane away.  The host routes
  // key ranges of more than 128 tiles to the general kernel.
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
  // full tile: every key exists; one scalar row base per tile and operand
  auto issue_full = [&](int nb, int stage) {
    char* kdst = lds + stage * STAGEB + wave_s * (IPW * 1024);
    // (a caller whose max_seqlen_k understates seqused_k gets the page of tile 127 for later tiles: wrong
    // numbers for a wrong argument, but always a page of this sequence)
    const int tl = nb - n_min < 127 ? nb - n_min : 127;
    const int64_t page = __builtin_amdgcn_readlane(tl < 64 ? pg_cache0 : pg_cache1, tl & 63);
    const int key = nb * kBN + wave_s * (IPW * KPI);
    const int slot = key & page_mask;
    const char* kp = kbase + (page * p.k_page_stride + (int64_t)slot * p.k_row_stride) * 2;
    const char* vp = vbase + (page * p.v_page_stride + (int64_t)slot * p.v_row_stride) * 2;
#pragma unroll
    for (int j = 0; j < IPW; ++j) {
      __builtin_amdgcn_global_load_lds(FG_GLBP(kp + (int64_t)j * KPI * p.k_row_stride * 2 + voff_k[j]), FG_LDSP(kdst + j * 1024), 16, 0, 0);
      __builtin_amdgcn_global_load_lds(FG_GLBP(vp + (int64_t)j * KPI * p.v_row_stride * 2 + voff_v[j]), FG_LDSP(kdst + OPB + j * 1024), 16, 0, 0);
    }
  };
  // partial tile: keys past the end are clamped to the last one (their scores are masked)
  auto issue_partial = [&](int nb, int stage) {
    char* kdst = lds + stage * STAGEB + wave_s * (IPW * 1024);
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
  auto issue_tile = [&](int nb, int stage) {
    if (nb * kBN + kBN <= k_len) {
      issue_full(nb, stage);
    } else {
      issue_partial(nb, stage);
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
    v_addr0[dt] = lds0 + v_key0 * RB + v_byte + (((dt * 4) ^ vx0) * 16);
    v_addr1[dt] = lds0 + (v_key0 + 4) * RB + v_byte + (((dt * 4) ^ vx1) * 16);
  }

  const bool wave_rows_ok = row0 < q_len;
  const int wave_row_last = (row0 + kRW - 1 < q_len ? row0 + kRW - 1 : q_len - 1);
  const float sc = a.scale_log2;
  // visible keys of this lane's row: [col_lo, col_hi]
  const int col_hi = a.has_right ? (qrow + shift + a.right_off_w < k_len - 1 ? qrow + shift + a.right_off_w : k_len - 1)
                                 : k_len - 1;
  const int col_lo = a.has_left ? qrow + shift - a.left_off_w : 0;

  auto tile = [&](int nb, auto stage_c) {
    constexpr int S = decltype(stage_c)::value;
    FG_WAIT_VM(0);                   // this wave's share of tile nb has landed
    __builtin_amdgcn_s_barrier();    // ... everybody's has, and nobody still reads the other stage
    if (nb + 1 < n_max) issue_tile(nb + 1, S ^ 1);

    const int key0 = nb * kBN;
    if (!wave_rows_ok) return;
    if (a.has_right && key0 > wave_row_last + shift + a.right_off_w) return;
    if (a.has_left && key0 + kBN - 1 < row0 + shift - a.left_off_w) return;

    // ---- S^T = K . Q^T : groups of GS fragment reads, one group ahead of the MFMAs -----------------------
    constexpr int GS = KS < 8 ? KS : 8;
    constexpr int NGK = 2 * KS / GS;
    f32x16 s_acc[2];
#pragma unroll
    for (int kt = 0; kt < 2; ++kt)
#pragma unroll
      for (int e = 0; e < 16; ++e) s_acc[kt][e] = 0.f;
    {
      u32x4 kf[2][8];
      auto issue_k = [&](auto gc, u32x4 (&dst)[8]) {
        constexpr int g = decltype(gc)::value;
        a_static_for<0, GS>([&](auto rc) {
          constexpr int r = decltype(rc)::value;
          constexpr int idx = g * GS + r, kt = idx / KS, ks = idx % KS;
          dst[r] = lds_read_b128_imm<S * STAGEB + kt * 32 * RB>(k_addr[ks]);
        });
      };
      issue_k(AInt<0>{}, kf[0]);
      a_static_for<0, NGK>([&](auto gc) {
        constexpr int g = decltype(gc)::value;
        lds_wait_all(kf[g & 1]);
        if constexpr (g + 1 < NGK) issue_k(AInt<g + 1>{}, kf[(g + 1) & 1]);
#pragma unroll
        for (int r = 0; r < GS; ++r) {
          const int idx = g * GS + r, kt = idx / KS, ks = idx % KS;
          s_acc[kt] = AttnMfma<T>::mma(__builtin_bit_cast(Frag, kf[g & 1][r]), qf[ks], s_acc[kt]);
        }
      });
    }

    // ---- masks (raw scores), running max ------------------------------------------------------------------
    const bool need_mask = (key0 + kBN > k_len) || (a.has_right && key0 + kBN - 1 > row0 + shift + a.right_off_w) ||
                           (a.has_left && key0 < wave_row_last + shift - a.left_off_w);
    if (need_mask) {
      // element (kt, e) is key key0 + half*8 + kt*32 + (e>>3)*16 + (e&7); compare the constant part
      const int hi_rel = col_hi - key0 - half * 8, lo_rel = col_lo - key0 - half * 8;
#pragma unroll
      for (int kt = 0; kt < 2; ++kt)
#pragma unroll
        for (int e = 0; e < 16; ++e) {
          const int rel = kt * 32 + (e >> 3) * 16 + (e & 7);
          s_acc[kt][e] = rel > hi_rel ? -INFINITY : s_acc[kt][e];
        }
      if (a.has_left) {
#pragma unroll
        for (int kt = 0; kt < 2; ++kt)
#pragma unroll
          for (int e = 0; e < 16; ++e) {
            const int rel = kt * 32 + (e >> 3) * 16 + (e & 7);
            s_acc[kt][e] = rel < lo_rel ? -INFINITY : s_acc[kt][e];
          }
      }
    }
    float tmax = -INFINITY;
#pragma unroll
    for (int kt = 0; kt < 2; ++kt)
#pragma unroll
      for (int e = 0; e < 16; ++e) tmax = fmaxf(tmax, s_acc[kt][e]);
    tmax *= sc;  // scale > 0, so the maximum commutes with it
    tmax = xhalf_max(tmax);
    // The reference maximum of a row moves only when the new maximum exceeds it by more than 2^8: any
    // reference gives the same result as long as p and the running sum use the same one.
    const bool moved = tmax > m_run + 8.0f;
    const float m_new = moved ? tmax : m_run;
    const float m_use = m_new == -INFINITY ? 0.f : m_new;
    const float alpha = moved ? __builtin_amdgcn_exp2f(m_run - m_use) : 1.0f;
    float psum = 0.f;
    Frag pf[4];
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

    // ---- O^T = O^T * alpha + V^T . P^T ---------------------------------------------------------------------
    if (__builtin_amdgcn_ballot_w64(moved) != 0) {
#pragma unroll
      for (int dt = 0; dt < DT; ++dt)
#pragma unroll
        for (int e = 0; e < 16; ++e) o_acc[dt][e] *= alpha;
    }
    {
      u32x2 vf[2][8];
      auto issue_v = [&](auto dc, u32x2 (&dst)[8]) {
        constexpr int dt = decltype(dc)::value;
        a_static_for<0, 4>([&](auto tc) {
          constexpr int t4 = decltype(tc)::value;
          dst[2 * t4] = lds_read_tr_b64_imm<S * STAGEB + OPB + t4 * 16 * RB>(v_addr0[dt]);
          dst[2 * t4 + 1] = lds_read_tr_b64_imm<S * STAGEB + OPB + t4 * 16 * RB>(v_addr1[dt]);
        });
      };
      issue_v(AInt<0>{}, vf[0]);
      a_static_for<0, DT>([&](auto dc) {
        constexpr int dt = decltype(dc)::value;
        lds_wait_all(vf[dt & 1]);
        if constexpr (dt + 1 < DT) issue_v(AInt<dt + 1>{}, vf[(dt + 1) & 1]);
#pragma unroll
        for (int t4 = 0; t4 < 4; ++t4) {
          const u32x4 both = {vf[dt & 1][2 * t4][0], vf[dt & 1][2 * t4][1], vf[dt & 1][2 * t4 + 1][0], vf[dt & 1][2 * t4 + 1][1]};
          o_acc[dt] = AttnMfma<T>::mma(__builtin_bit_cast(Frag, both), pf[t4], o_acc[dt]);
        }
      });
    }
  };

  if (n_min < n_max) issue_tile(n_min, 0);
  for (int nb = n_min; nb < n_max; nb += 2) {
    tile(nb, AInt<0>{});
    if (nb + 1 < n_max) tile(nb + 1, AInt<1>{});
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
int launch_fast(const AttnArgs& a, dim3 grid, hipStream_t st) {
  constexpr int LDS_BYTES = 2 * 2 * kBN * 2 * D;
  static hipError_t attr_err = hipFuncSetAttribute(reinterpret_cast<const void*>(attn_varlen_fast_kernel<T, D>),
                                                   hipFuncAttributeMaxDynamicSharedMemorySize, LDS_BYTES);
  if (attr_err != hipSuccess) {
    fg_set_error("flash_attn_varlen_fwd: cannot reserve %d bytes of LDS: %s", LDS_BYTES, hipGetErrorString(attr_err));
    return FG_ERR_LAUNCH;
  }
  hipLaunchKernelGGL((attn_varlen_fast_kernel<T, D>), grid, dim3(256), LDS_BYTES, st, a);
  return fg_check_launch("flash_attn_varlen_fwd");
}
