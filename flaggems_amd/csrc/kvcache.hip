// reshape_and_cache_flash and reshape_and_cache for gfx950: scatter of K and V token rows into the paged caches.
//
// One wave copies one (token, tensor) row of n = H*D elements: lanes stride through the row in
// 16-byte pieces, so both the gather side (token stride arbitrary) and the scatter side (slot
// anywhere in the cache) move in contiguous 1 KiB wave accesses.  Blocks hold four waves.  The
// copy is on raw bytes: no arithmetic touches the data, so the result is bit-exact.  Rows whose
// base or length defeats 16-byte access fall back to element-sized pieces.
#include "fg_common.h"

namespace {

template <typename U, typename SLOT>
__global__ __launch_bounds__(256) void cache_scatter_kernel(const char* __restrict__ key, const char* __restrict__ value,
                                                           char* __restrict__ kc, char* __restrict__ vc,
                                                           const SLOT* __restrict__ slots, int64_t num_tokens,
                                                           int64_t row_bytes, int64_t key_stride_b,
                                                           int64_t value_stride_b, int64_t block_stride_b,
                                                           int block_size) {
  const int64_t w = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);  // (token, tensor) pair
  const int64_t tok = w >> 1;
  if (tok >= num_tokens) return;
#if FG_V_SCATTER_EARLY
  // Variant (variants.h): the first four pieces of the row are requested together with the slot, which only the
  // stores depend on (a padding token's row is read for nothing): behind the slot they would cost a trip to memory
  // of their own.
  const bool is_v = w & 1;
  const U* src = reinterpret_cast<const U*>(is_v ? value + tok * value_stride_b : key + tok * key_stride_b);
  const int64_t n = row_bytes / (int64_t)sizeof(U);
  // four pieces per lane in flight: the row is short, so the copy lives on memory-level parallelism
  int64_t i = threadIdx.x & 63;
  asm volatile("" : : "s"(kc), "s"(vc), "s"(block_stride_b), "s"(block_size));  // fetched with the other arguments
  const bool first4 = i + 192 < n;
  U a0, b0, c0, d0;
  if (first4) {
    a0 = __builtin_nontemporal_load(src + i);
    b0 = __builtin_nontemporal_load(src + i + 64);
    c0 = __builtin_nontemporal_load(src + i + 128);
    d0 = __builtin_nontemporal_load(src + i + 192);
  }
  const int64_t slot = (int64_t)slots[tok];
  if (slot < 0) return;  // padding token
  const int64_t blk = slot / block_size;
  const int64_t off = slot - blk * block_size;
  U* dst = reinterpret_cast<U*>((is_v ? vc : kc) + blk * block_stride_b + off * row_bytes);
  if (first4) {
    __builtin_nontemporal_store(a0, dst + i);
    __builtin_nontemporal_store(b0, dst + i + 64);
    __builtin_nontemporal_store(c0, dst + i + 128);
    __builtin_nontemporal_store(d0, dst + i + 192);
    i += 256;
  }
#else
  const int64_t slot = (int64_t)slots[tok];
  if (slot < 0) return;  // padding token
  const int64_t blk = slot / block_size;
  const int64_t off = slot - blk * block_size;
  const bool is_v = w & 1;
  const U* src = reinterpret_cast<const U*>(is_v ? value + tok * value_stride_b : key + tok * key_stride_b);
  U* dst = reinterpret_cast<U*>((is_v ? vc : kc) + blk * block_stride_b + off * row_bytes);
  const int64_t n = row_bytes / (int64_t)sizeof(U);
  // four pieces per lane in flight: the row is short, so the copy lives on memory-level parallelism
  int64_t i = threadIdx.x & 63;
#endif
  // streaming accesses: neither the token rows nor the cache lines written here are read again soon
  for (; i + 192 < n; i += 256) {
    const U a = __builtin_nontemporal_load(src + i), b = __builtin_nontemporal_load(src + i + 64),
            c = __builtin_nontemporal_load(src + i + 128), d = __builtin_nontemporal_load(src + i + 192);
    __builtin_nontemporal_store(a, dst + i);
    __builtin_nontemporal_store(b, dst + i + 64);
    __builtin_nontemporal_store(c, dst + i + 128);
    __builtin_nontemporal_store(d, dst + i + 192);
  }
  for (; i < n; i += 64) __builtin_nontemporal_store(__builtin_nontemporal_load(src + i), dst + i);
}

template <typename SLOT>
int cache_dispatch(const void* key, const void* value, void* kc, void* vc, const SLOT* slots, int64_t num_tokens,
                   int64_t row_elems, int block_size, int64_t key_stride, int64_t value_stride, int64_t block_stride,
                   int eb, hipStream_t st) {
  const int64_t row_b = row_elems * eb, ks_b = key_stride * eb, vs_b = value_stride * eb, bs_b = block_stride * eb;
  const int64_t grid = fg_cdiv(num_tokens * 2, 4);
  FG_REQUIRE(grid < ((int64_t)1 << 31), FG_ERR_UNSUPPORTED, "reshape_and_cache_flash: too many tokens");
  auto ok = [&](int64_t a) {
    return row_b % a == 0 && ks_b % a == 0 && vs_b % a == 0 && bs_b % a == 0 && fg_aligned(key, a) &&
           fg_aligned(value, a) && fg_aligned(kc, a) && fg_aligned(vc, a);
  };
#define FG_LAUNCH(U)                                                                                              \
  hipLaunchKernelGGL((cache_scatter_kernel<U, SLOT>), dim3((unsigned)grid), dim3(256), 0, st, (const char*)key,     \
                     (const char*)value, (char*)kc, (char*)vc, slots, num_tokens, row_b, ks_b, vs_b, bs_b, block_size)
  if (ok(16)) FG_LAUNCH(u32x4);
  else if (ok(8)) FG_LAUNCH(u32x2);
  else if (ok(4)) FG_LAUNCH(uint32_t);
  else if (ok(2)) FG_LAUNCH(uint16_t);
  else FG_LAUNCH(uint8_t);
#undef FG_LAUNCH
  return fg_check_launch("reshape_and_cache_flash");
}

// The older cache layout: key_cache [blocks, H, D/x, block_size, x], value_cache [blocks, H, D, block_size]
// (x elements = 16 bytes of one head stay together in the key cache; the value cache is transposed so that
// the tokens of a page are contiguous per feature).  One workgroup per token, one element per thread and
// step: the value side is a scatter of single elements by construction.
template <typename U, typename SLOT>
__global__ __launch_bounds__(256) void cache_scatter_v0_kernel(const U* __restrict__ key, const U* __restrict__ value,
                                                              U* __restrict__ kc, U* __restrict__ vc,
                                                              const SLOT* __restrict__ slots, int H, int D,
                                                              int block_size, int x, int64_t num_blocks,
                                                              int64_t key_stride, int64_t value_stride) {
  const int64_t tok = blockIdx.x;
  const int64_t slot = (int64_t)slots[tok];
  if (slot < 0) return;  // padding token
  const int64_t blk = slot / block_size;
  if (blk >= num_blocks) return;  // a slot outside the cache is dropped rather than written somewhere
  const int64_t off = slot - blk * block_size;
  const int n = H * D, dx = D / x;
  for (int i = threadIdx.x; i < n; i += 256) {
    const int head = i / D, ho = i - head * D;
    const int xi = ho / x, xo = ho - xi * x;
    kc[(((blk * H + head) * dx + xi) * block_size + off) * x + xo] = key[tok * key_stride + i];
    vc[((blk * H + head) * D + ho) * block_size + off] = value[tok * value_stride + i];
  }
}

template <typename U>
int cache_v0_launch(const void* key, const void* value, void* kc, void* vc, const void* slots, int slot_is_i64,
                    int64_t num_tokens, int H, int D, int block_size, int x, int64_t num_blocks, int64_t key_stride,
                    int64_t value_stride, hipStream_t st) {
  if (slot_is_i64)
    hipLaunchKernelGGL((cache_scatter_v0_kernel<U, int64_t>), dim3((unsigned)num_tokens), dim3(256), 0, st, (const U*)key,
                       (const U*)value, (U*)kc, (U*)vc, (const int64_t*)slots, H, D, block_size, x, num_blocks,
                       key_stride, value_stride);
  else
    hipLaunchKernelGGL((cache_scatter_v0_kernel<U, int32_t>), dim3((unsigned)num_tokens), dim3(256), 0, st, (const U*)key,
                       (const U*)value, (U*)kc, (U*)vc, (const int32_t*)slots, H, D, block_size, x, num_blocks,
                       key_stride, value_stride);
  return fg_check_launch("reshape_and_cache");
}

}  // namespace

extern "C" int fg_reshape_and_cache(const void* key, const void* value, void* key_cache, void* value_cache,
                                    const void* slot_mapping, int slot_is_i64, int64_t num_tokens, int H, int D,
                                    int block_size, int x, int64_t num_blocks, int64_t key_stride,
                                    int64_t value_stride, int elem_bytes, void* stream) {
  FG_REQUIRE(num_tokens >= 0 && H >= 0 && D >= 0 && num_blocks >= 0, FG_ERR_INVALID, "reshape_and_cache: negative size");
  FG_REQUIRE(block_size > 0 && x > 0, FG_ERR_INVALID, "reshape_and_cache: block_size and x must be positive");
  FG_REQUIRE(D % x == 0, FG_ERR_INVALID, "reshape_and_cache: head size %d is not a multiple of x = %d", D, x);
  FG_REQUIRE(elem_bytes == 1 || elem_bytes == 2 || elem_bytes == 4, FG_ERR_INVALID,
             "reshape_and_cache: element size %d", elem_bytes);
  if (num_tokens == 0 || (int64_t)H * D == 0 || num_blocks == 0) return FG_OK;
  FG_REQUIRE(key && value && key_cache && value_cache && slot_mapping, FG_ERR_INVALID, "reshape_and_cache: null pointer");
  FG_REQUIRE(num_tokens < ((int64_t)1 << 31) && (int64_t)H * D < ((int64_t)1 << 31), FG_ERR_UNSUPPORTED,
             "reshape_and_cache: problem too large for one launch");
  FG_REQUIRE(key_stride >= (int64_t)H * D && value_stride >= (int64_t)H * D, FG_ERR_INVALID,
             "reshape_and_cache: token stride smaller than a token (%d x %d)", H, D);
  hipStream_t st = (hipStream_t)stream;
  if (elem_bytes == 2)
    return cache_v0_launch<uint16_t>(key, value, key_cache, value_cache, slot_mapping, slot_is_i64, num_tokens, H, D,
                                     block_size, x, num_blocks, key_stride, value_stride, st);
  if (elem_bytes == 4)
    return cache_v0_launch<uint32_t>(key, value, key_cache, value_cache, slot_mapping, slot_is_i64, num_tokens, H, D,
                                     block_size, x, num_blocks, key_stride, value_stride, st);
  return cache_v0_launch<uint8_t>(key, value, key_cache, value_cache, slot_mapping, slot_is_i64, num_tokens, H, D,
                                  block_size, x, num_blocks, key_stride, value_stride, st);
}

extern "C" int fg_reshape_and_cache_flash(const void* key, const void* value, void* key_cache, void* value_cache,
                                          const void* slot_mapping, int slot_is_i64, int64_t num_tokens, int H, int D,
                                          int block_size, int64_t key_stride, int64_t value_stride,
                                          int64_t block_stride, int elem_bytes, void* stream) {
  FG_REQUIRE(num_tokens >= 0 && H >= 0 && D >= 0, FG_ERR_INVALID, "reshape_and_cache_flash: negative size");
  FG_REQUIRE(block_size > 0, FG_ERR_INVALID, "reshape_and_cache_flash: block_size must be positive");
  FG_REQUIRE(elem_bytes == 1 || elem_bytes == 2 || elem_bytes == 4 || elem_bytes == 8, FG_ERR_INVALID,
             "reshape_and_cache_flash: element size %d", elem_bytes);
  if (num_tokens == 0 || (int64_t)H * D == 0) return FG_OK;
  FG_REQUIRE(key && value && key_cache && value_cache && slot_mapping, FG_ERR_INVALID,
             "reshape_and_cache_flash: null pointer");
  FG_REQUIRE(block_stride >= (int64_t)block_size * H * D, FG_ERR_INVALID,
             "reshape_and_cache_flash: block stride %lld smaller than a page (%d x %d x %d)", (long long)block_stride,
             block_size, H, D);
  hipStream_t st = (hipStream_t)stream;
  if (slot_is_i64)
    return cache_dispatch<int64_t>(key, value, key_cache, value_cache, (const int64_t*)slot_mapping, num_tokens,
                                   (int64_t)H * D, block_size, key_stride, value_stride, block_stride, elem_bytes, st);
  return cache_dispatch<int32_t>(key, value, key_cache, value_cache, (const int32_t*)slot_mapping, num_tokens,
                                 (int64_t)H * D, block_size, key_stride, value_stride, block_stride, elem_bytes, st);
}
