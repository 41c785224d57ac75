/*
 * kv_oracle.c -- plain-C restatement of the byte/integer parts of the path.
 *
 * TEST INFRASTRUCTURE ONLY: linked by tests/, __graft_entry__.smoke() and bench.py's cpu_baseline
 * leg; never by the product library.  Every function cites the reference code it follows (paths
 * relative to the FlagGems tree).  The reference ships no golden vectors for these functions; they
 * are pinned in tests/test_oracle.py by brute force on tiny inputs, invariants (every unit covered
 * exactly once, untouched bytes stay untouched) and agreement with the Python loop of the
 * reference's own test (tests/test_attention_ops.py:1459-1467, restated in oracle/torch_ref.py).
 */
#include <stdint.h>
#include <string.h>

/* Scatter of token rows into a paged cache.
 * Follows reshape_and_cache_flash_kernel, src/flag_gems/fused/reshape_and_cache_flash.py:14-58:
 * slot = slot_mapping[t]; slot < 0 skips; block = slot / block_size; offset = slot % block_size;
 * copy n = H*D elements from key + t*key_stride to cache + block*block_stride + offset*n.
 * All strides in elements; elem_bytes is the element width. */
void oracle_reshape_and_cache_flash(const uint8_t* key, const uint8_t* value, uint8_t* key_cache, uint8_t* value_cache,
                                    const int64_t* slot_mapping, int64_t num_tokens, int64_t n, int64_t block_size,
                                    int64_t key_stride, int64_t value_stride, int64_t block_stride, int elem_bytes) {
  for (int64_t t = 0; t < num_tokens; ++t) {
    const int64_t slot = slot_mapping[t];
    if (slot < 0) continue;
    const int64_t blk = slot / block_size, off = slot % block_size;
    const size_t bytes = (size_t)n * elem_bytes;
    memcpy(key_cache + (size_t)(blk * block_stride + off * n) * elem_bytes, key + (size_t)(t * key_stride) * elem_bytes, bytes);
    memcpy(value_cache + (size_t)(blk * block_stride + off * n) * elem_bytes, value + (size_t)(t * value_stride) * elem_bytes,
           bytes);
  }
}

/* Virtual key index -> element offset of its row in the paged cache.
 * Follows virtual_to_cache, src/flag_gems/ops/flash_kernel.py:1161-1182:
 * page = page_table[virt / block_size]; row = page * block_size + virt % block_size; times k_row_stride. */
int64_t oracle_virtual_to_cache(int64_t virt, const int32_t* page_table, int64_t block_size, int64_t k_row_stride) {
  const int64_t page = page_table[virt / block_size];
  return (page * block_size + virt % block_size) * k_row_stride;
}

/* Stream-K split.  Follows streamk_mm, src/flag_gems/ops/mm_streamk.py:466-485, and the per-program
 * ranges of first_wave, :198-199: cooperative tiles = tiles % workers, plus one full wave when other
 * tiles exist and the remainder is below half a wave, or zero when other tiles exist and the remainder
 * exceeds 0.8 of a wave; the cooperative tiles' K iterations are dealt to `workers` programs,
 * iters_per_pid each, the first iters_remaining programs taking one more, contiguous in tile-major order.
 * Returns the number of cooperative tiles. */
int64_t oracle_streamk_partition(int64_t tiles, int64_t iters_per_tile, int64_t workers, int64_t* begin, int64_t* end) {
  int64_t coop = tiles % workers;
  const int64_t other = tiles - coop;
  if (other > 0 && (double)coop < (double)workers * 0.5) coop += workers;
  else if (other > 0 && (double)coop > (double)workers * 0.8) coop = 0;
  const int64_t total = coop * iters_per_tile;
  const int64_t per = total / workers, rem = total % workers;
  int64_t start = 0;
  for (int64_t pid = 0; pid < workers; ++pid) {
    const int64_t n = per + (pid < rem ? 1 : 0);
    begin[pid] = start;
    end[pid] = start + n;
    start += n;
  }
  return coop;
}

/* fused_add_rms_norm in scalar fp32 (one row at a time), the arithmetic of
 * fused_add_rms_norm_kernel, src/flag_gems/fused/fused_add_rms_norm.py:38-54: x += r; r <- x;
 * var = sum(x*x/N); rrms = 1/sqrt(var+eps); x <- x*rrms*w.  Used as the scalar-port CPU baseline. */
#include <math.h>
void oracle_fused_add_rms_norm_f32(float* x, float* residual, const float* w, int64_t M, int64_t N, float eps) {
  for (int64_t r = 0; r < M; ++r) {
    float* xr = x + r * N;
    float* rr = residual + r * N;
    float var = 0.f;
    for (int64_t c = 0; c < N; ++c) {
      const float v = xr[c] + rr[c];
      rr[c] = v;
      var += v * v / (float)N;
    }
    const float rrms = 1.0f / sqrtf(var + eps);
    for (int64_t c = 0; c < N; ++c) xr[c] = rr[c] * rrms * w[c];
  }
}
