// Shared device/host helpers for the gfx950 kernels of libfg_mi355.so.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>
#include <stdio.h>
#include <stdarg.h>
#include "../../include/fg_mi355.h"
#include "variants.h"

// ---------------------------------------------------------------------------------------------
// host side: error reporting
// ---------------------------------------------------------------------------------------------
void fg_set_error(const char* fmt, ...);
int fg_check_launch(const char* what);

#define FG_REQUIRE(cond, code, ...) \
  do {                              \
    if (!(cond)) {                  \
      fg_set_error(__VA_ARGS__);    \
      return (code);                \
    }                               \
  } while (0)

// Measurement and test switches, read from the environment once (first use) and again only when
// fg_reload_options() is called; no entry point calls getenv().
struct FgOptions {
  bool gemm_no_dma;       // FG_GEMM_NO_DMA: keep 16-bit GEMMs off the direct-to-LDS kernels
  bool gemm_sk_even;      // FG_GEMM_SK_EVEN: stream-K always in equal shares
  int gemm_tile_bm, gemm_tile_bn;  // FG_GEMM_TILE=256x128: forced direct-to-LDS tile (bm == 0: not forced)
  bool skinny_no_lds;     // FG_SKINNY_NO_LDS
  bool skinny_rows64;     // FG_SKINNY_ROWS64
  int skinny_tile;        // FG_SKINNY_TILE=16|32 (0: not set)
  char attn_kernel[8];    // FG_ATTN_KERNEL ("" when not set)
  int attn_mixed;         // FG_ATTN_MIXED: 0 / 1 (-1: not set)
  int decode_min_tiles;   // FG_DECODE_MIN_TILES (0: not set)
  int decode_wg_per_cu;   // FG_DECODE_WG_PER_CU (0: not set)
};
const FgOptions& fg_options();

static inline bool fg_aligned(const void* p, size_t a) { return (reinterpret_cast<uintptr_t>(p) % a) == 0; }
static inline int64_t fg_cdiv(int64_t a, int64_t b) { return (a + b - 1) / b; }

// ---------------------------------------------------------------------------------------------
// element types.  __bf16 / _Float16 are native on gfx950 (v_cvt_pk_bf16_f32 rounds to nearest even).
// ---------------------------------------------------------------------------------------------
typedef __bf16 bf16_t;
typedef _Float16 f16_t;

typedef float f32x2 __attribute__((ext_vector_type(2)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef bf16_t bf16x4 __attribute__((ext_vector_type(4)));
typedef bf16_t bf16x8 __attribute__((ext_vector_type(8)));
typedef f16_t f16x4 __attribute__((ext_vector_type(4)));
typedef f16_t f16x8 __attribute__((ext_vector_type(8)));
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));

template <typename T> struct fg_type_id;
template <> struct fg_type_id<f16_t> { static constexpr int value = FG_F16; };
template <> struct fg_type_id<bf16_t> { static constexpr int value = FG_BF16; };
template <> struct fg_type_id<float> { static constexpr int value = FG_F32; };

// A VEC-wide pack of T moved with one memory instruction when VEC*sizeof(T) is 4, 8 or 16 bytes.
template <typename T, int VEC> struct alignas(sizeof(T) * VEC) Pack {
  T v[VEC];
};

template <typename T, int VEC>
__device__ __forceinline__ Pack<T, VEC> ld_pack(const T* p) {
  return *reinterpret_cast<const Pack<T, VEC>*>(p);
}
template <typename T, int VEC>
__device__ __forceinline__ void st_pack(T* p, const Pack<T, VEC>& v) {
  *reinterpret_cast<Pack<T, VEC>*>(p) = v;
}
// Streaming variants: data that is touched once should not displace reusable lines in L2.
template <typename T, int VEC>
__device__ __forceinline__ Pack<T, VEC> ld_pack_nt(const T* p) {
  if constexpr (sizeof(T) * VEC == 16) {
    u32x4 r = __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(p));
    return *reinterpret_cast<Pack<T, VEC>*>(&r);
  } else if constexpr (sizeof(T) * VEC == 8) {
    u32x2 r = __builtin_nontemporal_load(reinterpret_cast<const u32x2*>(p));
    return *reinterpret_cast<Pack<T, VEC>*>(&r);
  } else {
    return *reinterpret_cast<const Pack<T, VEC>*>(p);
  }
}
template <typename T, int VEC>
__device__ __forceinline__ void st_pack_nt(T* p, const Pack<T, VEC>& v) {
  if constexpr (sizeof(T) * VEC == 16) {
    __builtin_nontemporal_store(*reinterpret_cast<const u32x4*>(&v), reinterpret_cast<u32x4*>(p));
  } else if constexpr (sizeof(T) * VEC == 8) {
    __builtin_nontemporal_store(*reinterpret_cast<const u32x2*>(&v), reinterpret_cast<u32x2*>(p));
  } else {
    *reinterpret_cast<Pack<T, VEC>*>(p) = v;
  }
}

// Element-aligned variants: the address is a multiple of sizeof(T) only.  The compiler still emits one wide
// access (the target handles unaligned vector-memory accesses), split by the hardware where it crosses a line.
template <typename T, int VEC>
__device__ __forceinline__ Pack<T, VEC> ld_pack_u(const T* p) {
  Pack<T, VEC> v;
  __builtin_memcpy(&v, p, sizeof(T) * VEC);
  return v;
}
template <typename T, int VEC>
__device__ __forceinline__ void st_pack_u(T* p, const Pack<T, VEC>& v) {
  __builtin_memcpy(p, &v, sizeof(T) * VEC);
}

// Waits until every vector-memory operation this wave has issued, stores included, has completed.
// A workgroup-scope release fence does not emit this wait on gfx950 (the waves of a workgroup share
// one L1, so the fence has nothing to order for them), and a device-scope release would write the
// whole L2 back.  Publishing device-coherent (write-through) stores to another workgroup through a
// later atomic therefore spells the wait out: stores complete, then the barrier, then the atomic.
__device__ __forceinline__ void fg_wait_vmem_done() {
  __builtin_amdgcn_s_waitcnt((7 << 4) | (0xF << 8));  // vmcnt(0); expcnt and lgkmcnt not waited for
}

// ---------------------------------------------------------------------------------------------
// wavefront-64 reductions.  The first four butterfly steps stay inside a row of 16 lanes and use
// DPP modifiers (no LDS traffic); the last two cross rows through ds_bpermute.
// ---------------------------------------------------------------------------------------------
template <int CTRL>
__device__ __forceinline__ float dpp_mov(float v) {
  return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), CTRL, 0xF, 0xF, true));
}
struct OpSum {
  __device__ __forceinline__ float operator()(float a, float b) const { return a + b; }
};
struct OpMax {
  __device__ __forceinline__ float operator()(float a, float b) const { return fmaxf(a, b); }
};
// All 64 lanes end up with the reduction over the whole wave.
template <typename Op>
__device__ __forceinline__ float wave_allreduce(float v, Op op) {
  v = op(v, dpp_mov<0xB1>(v));   // quad_perm [1,0,3,2]
  v = op(v, dpp_mov<0x4E>(v));   // quad_perm [2,3,0,1]
  v = op(v, dpp_mov<0x141>(v));  // row_half_mirror
  v = op(v, dpp_mov<0x140>(v));  // row_mirror
  v = op(v, __shfl_xor(v, 16, 64));
  v = op(v, __shfl_xor(v, 32, 64));
  return v;
}
__device__ __forceinline__ float wave_sum(float v) { return wave_allreduce(v, OpSum()); }
__device__ __forceinline__ float wave_max(float v) { return wave_allreduce(v, OpMax()); }
