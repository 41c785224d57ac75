// Rotary position embedding for gfx950.
//
// q [n_tokens, Hq, D] and k [n_tokens, Hk, D] are addressed through {token, head, dim} element
// strides, so slices of a fused qkv buffer work in place.  The unit of work is a pack of VEC
// rotation pairs of one head of one token; packs are numbered token-major and dealt to threads
// one each, so a wave reads 64 consecutive packs (1 KiB runs at 16 B per lane) whatever the head
// count.  Half-rotation ("neox") pairs element i with i + D/2: a thread loads one pack from each
// half.  Interleaved pairs (2j, 2j+1): a thread loads one pack of adjacent elements.  Arithmetic is
// fp32 (x*cos -/+ x_pair*sin as two products and a sum), rounded once on store.  Every thread
// loads all of its inputs before it stores, and no element belongs to two threads, so the
// in-place form is race free.
#include "fg_common.h"

namespace {

template <typename TC, int VEC>
__device__ __forceinline__ void load_cs(const TC* p, float out[VEC]) {
  constexpr int CH = (sizeof(TC) * VEC > 16) ? (16 / sizeof(TC)) : VEC;  // elements per 16-byte chunk
#pragma unroll
  for (int c = 0; c < VEC / CH; ++c) {
    Pack<TC, CH> pk = ld_pack<TC, CH>(p + c * CH);
#pragma unroll
    for (int e = 0; e < CH; ++e) out[c * CH + e] = (float)pk.v[e];
  }
}

struct RopeArgs {
  void* q_out;
  void* k_out;
  const void* q;
  const void* k;
  const void* cos;
  const void* sin;
  const void* pos;
  int64_t n_tokens, seq_len;
  int64_t qs[3], ks[3], qos[3], kos[3];
  int64_t pos_stride, cos_stride, sin_stride;
  int Hq, Hk, D;
  int pos_is_i64;
};

// VEC > 1 requires unit dim strides and 16-byte aligned rows; VEC == 1 takes anything.
template <typename T, typename TC, int VEC, bool INTERLEAVED>
__global__ __launch_bounds__(256) void rope_kernel(RopeArgs a) {
  // packs per head: neox D/2/VEC pair packs; interleaved D/VEC element packs (VEC/2 pairs each,
  // or one pair when VEC == 1).
  const int half = a.D / 2;
  const int pph = INTERLEAVED ? (VEC == 1 ? half : a.D / VEC) : half / VEC;
  const int heads = a.Hq + a.Hk;
  const int64_t per_token = (int64_t)heads * pph;
  const int64_t item = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (item >= a.n_tokens * per_token) return;
  const int64_t tok = item / per_token;
  const int r = (int)(item - tok * per_token);
  const int h = r / pph;
  const int c = r - h * pph;

  // Variant FG_V_ROPE_ARGS (variants.h; off: arguments fetched where used, strides selected through a pointer).
  constexpr bool ARGS_EARLY = FG_V_ROPE_ARGS != 0;
  if constexpr (ARGS_EARLY) {
    // the arguments of the second half of the kernel are fetched with the first ones, not behind the position load
    asm volatile("" : : "s"(a.cos), "s"(a.sin), "s"(a.cos_stride), "s"(a.sin_stride), "s"(a.q), "s"(a.k), "s"(a.q_out), "s"(a.k_out));
    asm volatile("" : : "s"(a.qs[0]), "s"(a.qs[1]), "s"(a.ks[0]), "s"(a.ks[1]), "s"(a.qos[0]), "s"(a.qos[1]), "s"(a.kos[0]), "s"(a.kos[1]));
  }
  int64_t pos;
  if (a.pos == nullptr) {
    pos = tok % a.seq_len;
  } else if (a.pos_is_i64) {
    pos = ((const int64_t*)a.pos)[tok * a.pos_stride];
  } else {
    pos = ((const int32_t*)a.pos)[tok * a.pos_stride];
  }
  const TC* cosr = (const TC*)a.cos + pos * a.cos_stride;
  const TC* sinr = (const TC*)a.sin + pos * a.sin_stride;

  const bool is_q = h < a.Hq;
  const int hh = is_q ? h : h - a.Hq;
#if FG_V_ROPE_ARGS
  // the strides are selected by value: selecting a pointer into the argument block makes them a vector load from
  // memory, a trip of its own in front of the row
  const int64_t is[3] = {is_q ? a.qs[0] : a.ks[0], is_q ? a.qs[1] : a.ks[1], is_q ? a.qs[2] : a.ks[2]};
  const int64_t os[3] = {is_q ? a.qos[0] : a.kos[0], is_q ? a.qos[1] : a.kos[1], is_q ? a.qos[2] : a.kos[2]};
#else
  const int64_t* is = is_q ? a.qs : a.ks;
  const int64_t* os = is_q ? a.qos : a.kos;
#endif
  const T* src = (const T*)(is_q ? a.q : a.k) + tok * is[0] + hh * is[1];
  T* dst = (T*)(is_q ? a.q_out : a.k_out) + tok * os[0] + hh * os[1];

  if constexpr (VEC == 1) {
    const int i0 = INTERLEAVED ? 2 * c : c;
    const int i1 = INTERLEAVED ? 2 * c + 1 : c + half;
    const float cs = (float)cosr[c], sn = (float)sinr[c];
    const float x0 = (float)src[i0 * is[2]], x1 = (float)src[i1 * is[2]];
    const float y0 = x0 * cs + x1 * (-sn);
    const float y1 = x1 * cs + x0 * sn;
    dst[i0 * os[2]] = (T)y0;
    dst[i1 * os[2]] = (T)y1;
  } else if constexpr (INTERLEAVED) {
    constexpr int HV = VEC / 2;
    float cs[HV], sn[HV];
    load_cs<TC, HV>(cosr + c * HV, cs);
    load_cs<TC, HV>(sinr + c * HV, sn);
    Pack<T, VEC> x = ld_pack<T, VEC>(src + c * VEC), y;
#pragma unroll
    for (int e = 0; e < HV; ++e) {
      const float x0 = (float)x.v[2 * e], x1 = (float)x.v[2 * e + 1];
      y.v[2 * e] = (T)(x0 * cs[e] + x1 * (-sn[e]));
      y.v[2 * e + 1] = (T)(x1 * cs[e] + x0 * sn[e]);
    }
    st_pack<T, VEC>(dst + c * VEC, y);
  } else {
    float cs[VEC], sn[VEC];
    load_cs<TC, VEC>(cosr + c * VEC, cs);
    load_cs<TC, VEC>(sinr + c * VEC, sn);
    Pack<T, VEC> x0 = ld_pack<T, VEC>(src + c * VEC), x1 = ld_pack<T, VEC>(src + half + c * VEC), y0, y1;
#pragma unroll
    for (int e = 0; e < VEC; ++e) {
      const float a0 = (float)x0.v[e], a1 = (float)x1.v[e];
      y0.v[e] = (T)(a0 * cs[e] + a1 * (-sn[e]));
      y1.v[e] = (T)(a1 * cs[e] + a0 * sn[e]);
    }
    st_pack<T, VEC>(dst + c * VEC, y0);
    st_pack<T, VEC>(dst + half + c * VEC, y1);
  }
}

template <typename T, typename TC>
int rope_dispatch(const RopeArgs& a, bool interleaved, hipStream_t st) {
  constexpr int VEC = 16 / sizeof(T);
  const int half = a.D / 2;
  auto rows_ok = [&](const void* p, const int64_t* s) {
    return fg_aligned(p, 16) && s[2] == 1 && s[0] % VEC == 0 && s[1] % VEC == 0;
  };
  const int cs_pack = interleaved ? VEC / 2 : VEC;  // cos/sin elements one thread loads at once
  const size_t cs_bytes = sizeof(TC) * cs_pack > 16 ? 16 : sizeof(TC) * cs_pack;
  const bool vec_ok = rows_ok(a.q, a.qs) && rows_ok(a.k, a.ks) && rows_ok(a.q_out, a.qos) && rows_ok(a.k_out, a.kos) &&
                      (interleaved ? a.D % VEC == 0 : half % VEC == 0) && fg_aligned(a.cos, cs_bytes) &&
                      fg_aligned(a.sin, cs_bytes) && (a.cos_stride * sizeof(TC)) % cs_bytes == 0 &&
                      (a.sin_stride * sizeof(TC)) % cs_bytes == 0;
  const int pph = vec_ok ? (interleaved ? a.D / VEC : half / VEC) : half;
  const int64_t items = a.n_tokens * (int64_t)(a.Hq + a.Hk) * pph;
  const int64_t grid = fg_cdiv(items, 256);
  FG_REQUIRE(grid < ((int64_t)1 << 31), FG_ERR_UNSUPPORTED, "rope: problem too large for one launch");
  if (vec_ok) {
    if (interleaved) hipLaunchKernelGGL((rope_kernel<T, TC, VEC, true>), dim3((unsigned)grid), dim3(256), 0, st, a);
    else hipLaunchKernelGGL((rope_kernel<T, TC, VEC, false>), dim3((unsigned)grid), dim3(256), 0, st, a);
  } else {
    if (interleaved) hipLaunchKernelGGL((rope_kernel<T, TC, 1, true>), dim3((unsigned)grid), dim3(256), 0, st, a);
    else hipLaunchKernelGGL((rope_kernel<T, TC, 1, false>), dim3((unsigned)grid), dim3(256), 0, st, a);
  }
  return fg_check_launch("rope");
}

template <typename T>
int rope_dispatch_cs(const RopeArgs& a, bool interleaved, int cs_dtype, hipStream_t st) {
  switch (cs_dtype) {
    case FG_F16: return rope_dispatch<T, f16_t>(a, interleaved, st);
    case FG_BF16: return rope_dispatch<T, bf16_t>(a, interleaved, st);
    case FG_F32: return rope_dispatch<T, float>(a, interleaved, st);
  }
  fg_set_error("rope: unsupported cos/sin dtype %d", cs_dtype);
  return FG_ERR_INVALID;
}

}  // namespace

extern "C" int fg_rope(void* q_out, void* k_out, const void* q, const void* k, const void* cos, const void* sin,
                       const void* pos, int pos_is_i64, int64_t n_tokens, int64_t seq_len, int Hq, int Hk, int D,
                       const int64_t q_strides[3], const int64_t k_strides[3], const int64_t qo_strides[3],
                       const int64_t ko_strides[3], int64_t pos_stride, int64_t cos_stride, int64_t sin_stride,
                       int64_t max_pos, int interleaved, int dtype, int cs_dtype, void* stream) {
  FG_REQUIRE(n_tokens >= 0 && Hq >= 0 && Hk >= 0 && D >= 0, FG_ERR_INVALID, "rope: negative size");
  FG_REQUIRE(D % 2 == 0, FG_ERR_INVALID, "rope: head_dim %d must be even", D);
  if (n_tokens == 0 || D == 0 || Hq + Hk == 0) return FG_OK;
  FG_REQUIRE(q && k && q_out && k_out && cos && sin, FG_ERR_INVALID, "rope: null pointer");
  FG_REQUIRE(q_strides && k_strides && qo_strides && ko_strides, FG_ERR_INVALID, "rope: null stride array");
  FG_REQUIRE(pos != nullptr || seq_len > 0, FG_ERR_INVALID, "rope: seq_len must be positive without position ids");
  FG_REQUIRE(max_pos > 0, FG_ERR_INVALID, "rope: empty cos/sin table");
  RopeArgs a;
  a.q_out = q_out; a.k_out = k_out; a.q = q; a.k = k; a.cos = cos; a.sin = sin; a.pos = pos;
  a.n_tokens = n_tokens; a.seq_len = seq_len;
  for (int i = 0; i < 3; ++i) {
    a.qs[i] = q_strides[i]; a.ks[i] = k_strides[i]; a.qos[i] = qo_strides[i]; a.kos[i] = ko_strides[i];
  }
  a.pos_stride = pos_stride; a.cos_stride = cos_stride; a.sin_stride = sin_stride;
  a.Hq = Hq; a.Hk = Hk; a.D = D; a.pos_is_i64 = pos_is_i64;
  hipStream_t st = (hipStream_t)stream;
  switch (dtype) {
    case FG_F16: return rope_dispatch_cs<f16_t>(a, interleaved != 0, cs_dtype, st);
    case FG_BF16: return rope_dispatch_cs<bf16_t>(a, interleaved != 0, cs_dtype, st);
    case FG_F32: return rope_dispatch_cs<float>(a, interleaved != 0, cs_dtype, st);
  }
  fg_set_error("rope: unsupported dtype %d", dtype);
  return FG_ERR_INVALID;
}
