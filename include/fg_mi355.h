/*
 * fg_mi355.h — C ABI of libfg_mi355.so: hand-written gfx950 (CDNA4) kernels for the
 * LLM-inference operator path of FlagGems (mm/addmm, softmax, rms_norm, fused_add_rms_norm,
 * rotary embedding, reshape_and_cache_flash, silu_and_mul, flash_attn_varlen_func).
 *
 * Conventions
 *   - every pointer is a DEVICE pointer unless its comment says "host";
 *   - sizes and strides are int64 and counted in ELEMENTS, never bytes;
 *   - `stream` is a hipStream_t passed as void* (NULL = the null stream);
 *   - entry points validate on the host, launch asynchronously on `stream`, never
 *     synchronise and never allocate device memory;
 *   - return value: FG_OK (0) or a negative FG_ERR_* code; fg_last_error() gives the
 *     thread-local message of the last failure.  No C++ exception crosses this boundary.
 *
 * Each declaration cites the reference interface it stands in for (paths are relative to
 * the FlagGems source tree).  The operator entry points come first; a "Diagnostics" section at the
 * end holds the few host-side hooks of the library's own tests and benchmark.
 */
#ifndef FG_MI355_H
#define FG_MI355_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

enum { FG_F16 = 0, FG_BF16 = 1, FG_F32 = 2 };

enum {
  FG_OK = 0,
  FG_ERR_INVALID = -1,     /* bad shape / stride / null pointer / dtype */
  FG_ERR_UNSUPPORTED = -2, /* valid request this build has no kernel for */
  FG_ERR_LAUNCH = -3,      /* hipGetLastError() reported a failure after the launch */
  FG_ERR_WORKSPACE = -4    /* workspace missing or too small */
};

/* Message of the last failing call on this thread ("" if none). */
const char* fg_last_error(void);

/* ABI version of this header (bumped on any signature change). */
int fg_abi_version(void);

/* Device facts the host-side heuristics use (CU count stands in for the reference's
 * multi_processor_count: src/flag_gems/ops/mm.py:24, src/flag_gems/ops/flash_api.py:524-530).
 * Also performs the library's only per-device set-up (the address of fg_gemm_skinny_static's scratch array), so a
 * caller that queries its devices at start-up may issue every later call under stream capture. */
int fg_device_info(int device, int* num_cu, int* lds_bytes, int* gcn_arch);

/* rms_norm forward.  y[m,:] = x[m,:] * rsqrt(mean(x[m,:]^2) + eps) * w, fp32 arithmetic,
 * one rounding on store; inv_rms[m] (fp32) is written when non-NULL; w may be NULL (= ones).
 * Replaces rms_norm_kernel, src/flag_gems/ops/rms_norm.py:15-51, and
 * flag_gems::rms_norm, lib/rms_norm.cpp:15-71. */
int fg_rms_norm(const void* x, const void* w, void* y, float* inv_rms, int64_t M, int64_t N,
                int64_t x_row_stride, int64_t y_row_stride, float eps, int dtype, void* stream);

/* In-place pair update: residual = x + residual (rounded to dtype on store), x =
 * rmsnorm(unrounded sum) * w.
 * Replaces fused_add_rms_norm_kernel, src/flag_gems/fused/fused_add_rms_norm.py:14-54, and
 * flag_gems::fused_add_rms_norm, lib/fused_add_rms_norm.cpp:14-72. */
int fg_fused_add_rms_norm(void* x, void* residual, const void* w, int64_t M, int64_t N,
                          int64_t x_row_stride, int64_t r_row_stride, float eps, int dtype,
                          void* stream);

/* softmax over the middle axis of a contiguous [M, N, K] view (K == 1: innermost axis).
 * fp32 arithmetic, out_dtype == in_dtype or FG_F32 (half_to_float).
 * Replaces softmax_kernel_inner / softmax_kernel_non_inner,
 * src/flag_gems/ops/softmax.py:15-72,87-159, and flag_gems::softmax, lib/softmax.cpp:28-73. */
int fg_softmax(const void* in, void* out, int64_t M, int64_t N, int64_t K, int in_dtype,
               int out_dtype, void* stream);

/* log_softmax over the middle axis of a contiguous [M, N, K] view: (x - max) - log(sum exp(x - max)), fp32
 * arithmetic, out_dtype == in_dtype or FG_F32.  Same kernels as fg_softmax with a different last step.
 * Replaces log_softmax_kernel, src/flag_gems/ops/log_softmax.py:15-58,98-128. */
int fg_log_softmax(const void* in, void* out, int64_t M, int64_t N, int64_t K, int in_dtype,
               int out_dtype, void* stream);

/* Backward of softmax / log_softmax over the middle axis of contiguous [M, N, K] views, from the forward's
 * OUTPUT: grad_in = out * (grad_out - sum(out * grad_out))  resp.  grad_out - exp(out) * sum(grad_out),
 * fp32 arithmetic.  out and grad_out share `dtype`; grad_in_dtype equals it, or is a 16-bit type when
 * `dtype` is FG_F32 (the forward widened its result).
 * Replace softmax_backward_kernel_{inner,non_inner}, src/flag_gems/ops/softmax.py:163-280,321-355, and
 * log_softmax_backward_kernel, src/flag_gems/ops/log_softmax.py:60-96,131-160. */
int fg_softmax_backward(const void* out, const void* grad_out, void* grad_in, int64_t M, int64_t N,
                        int64_t K, int dtype, int grad_in_dtype, void* stream);
int fg_log_softmax_backward(const void* out, const void* grad_out, void* grad_in, int64_t M,
                            int64_t N, int64_t K, int dtype, int grad_in_dtype, void* stream);

/* Backward of rms_norm for contiguous x, dy, dx [M, N] and the inv_rms [M] that fg_rms_norm wrote:
 * g = dy * w, xh = x * inv_rms, dx = (g - xh * mean(xh * g)) * inv_rms (w == NULL: ones).
 * When dw_partial is non-NULL it is fp32 [partial_rows, N], 32-byte aligned, 1 <= partial_rows <= M: row p
 * receives the sums of x * dy * inv_rms over rows [p * ceil(M / partial_rows), ...); the column sum of
 * dw_partial is the weight gradient.  fg_rms_norm_backward_partial_rows proposes a partial_rows that fills
 * the device.  One kernel computes both gradients (x and dy are read once).  fg_rms_norm_backward_dw adds the
 * rows of dw_partial up in fp32, in a fixed order, and writes the weight gradient dw [N] in `dtype`, rounded once
 * (the reference rounds its partial rows to the input dtype and sums them with torch.sum, rms_norm.py:205-218).
 * Replaces rms_norm_grad_dx_kernel and rms_norm_grad_dw_kernel, src/flag_gems/ops/rms_norm.py:54-146,171-218. */
int64_t fg_rms_norm_backward_partial_rows(int64_t M, int64_t N, int dtype, int device);
int fg_rms_norm_backward(const void* x, const void* dy, const float* inv_rms, const void* w, void* dx,
                         float* dw_partial, int64_t partial_rows, int64_t M, int64_t N, int dtype,
                         void* stream);
int fg_rms_norm_backward_dw(const float* dw_partial, int64_t partial_rows, int64_t N, void* dw, int dtype,
                            void* stream);

/* dst[c, r] = src[r, c] for a [rows, cols] source with unit column stride and a [cols, rows] destination with unit
 * column stride (row strides in elements), elements of 2 or 4 bytes moved as bits.  No counterpart in the reference,
 * whose Triton GEMMs read operands through any strides (src/flag_gems/ops/mm.py:54-134): the host side of mm uses
 * it to turn a column-major A into the K-contiguous layout the fast GEMM kernels read. */
int fg_transpose2d(const void* src, void* dst, int64_t rows, int64_t cols, int64_t src_row_stride,
                   int64_t dst_row_stride, int elem_bytes, void* stream);

/* Rotary embedding of q [n_tokens,Hq,D] and k [n_tokens,Hk,D] (element strides given as
 * {token, head, dim}); cos/sin [max_pos, D/2] with unit inner stride.  pos == NULL means
 * position = token_index % seq_len.  q_out/k_out may alias q/k (in-place).
 * Replaces apply_rotary_pos_emb_kernel / _inplace_kernel,
 * src/flag_gems/fused/rotary_embedding.py:15-178, and flag_gems::rotary_embedding(_inplace),
 * lib/rotary_embedding.cpp:96-281. */
int fg_rope(void* q_out, void* k_out, const void* q, const void* k, const void* cos,
            const void* sin, const void* pos, int pos_is_i64, int64_t n_tokens, int64_t seq_len,
            int Hq, int Hk, int D, const int64_t q_strides[3], const int64_t k_strides[3],
            const int64_t qo_strides[3], const int64_t ko_strides[3], int64_t pos_stride,
            int64_t cos_stride, int64_t sin_stride, int64_t max_pos, int interleaved, int dtype,
            int cs_dtype, void* stream);

/* Scatter of K/V token rows (H*D dense elements each) into the paged caches
 * [num_blocks, block_size, H, D]; slot < 0 skips the token.  Pure byte copy.
 * Replaces reshape_and_cache_flash_kernel, src/flag_gems/fused/reshape_and_cache_flash.py:14-58,
 * and flag_gems::reshape_and_cache_flash, lib/reshape_and_cache_flash.cpp:11-67. */
int fg_reshape_and_cache_flash(const void* key, const void* value, void* key_cache,
                               void* value_cache, const void* slot_mapping, int slot_is_i64,
                               int64_t num_tokens, int H, int D, int block_size,
                               int64_t key_stride, int64_t value_stride, int64_t block_stride,
                               int elem_bytes, void* stream);

/* The same scatter into the older cache layout: key_cache [num_blocks, H, D/x, block_size, x] and
 * value_cache [num_blocks, H, D, block_size], both contiguous; key/value [num_tokens, H, D] with a dense
 * [H, D] block per token and the given token strides (elements).  Slots < 0 and slots past the last block
 * are skipped.  Bit-exact copy of elem_bytes-sized elements.
 * Replaces reshape_and_cache_kernel, src/flag_gems/fused/reshape_and_cache.py:12-112. */
int fg_reshape_and_cache(const void* key, const void* value, void* key_cache, void* value_cache,
                         const void* slot_mapping, int slot_is_i64, int64_t num_tokens, int H, int D,
                         int block_size, int x, int64_t num_blocks, int64_t key_stride,
                         int64_t value_stride, int elem_bytes, void* stream);

/* out[r,c] = silu(a[r,c]) * b[r,c] (fp32 arithmetic), rows of unit inner stride.
 * Replaces silu_and_mul_kernel, src/flag_gems/fused/silu_and_mul.py:12-17,47-53. */
int fg_silu_and_mul(const void* a, const void* b, void* out, int64_t rows, int64_t cols,
                    int64_t a_row_stride, int64_t b_row_stride, int64_t o_row_stride, int dtype,
                    void* stream);

/* Gradients of fg_silu_and_mul: with s = 1 / (1 + exp(-a)),
 *   grad_a = grad_out * b * s * (1 + a * (1 - s)),   grad_b = grad_out * a * s   (fp32 arithmetic),
 * five [rows, cols] operands of one dtype with unit inner stride and independent row strides.
 * FG_ERR_UNSUPPORTED from a build that leaves the kernel out (csrc/variants.h, FG_V_SILU_GRAD_KERNEL).
 * Replaces silu_and_mul_grad_kernel, src/flag_gems/fused/silu_and_mul.py:20-44. */
int fg_silu_and_mul_backward(const void* a, const void* b, const void* grad_out, void* grad_a, void* grad_b,
                             int64_t rows, int64_t cols, int64_t a_row_stride, int64_t b_row_stride,
                             int64_t g_row_stride, int64_t ga_row_stride, int64_t gb_row_stride, int dtype,
                             void* stream);

/* GEMM schedules. */
enum { FG_SCHED_AUTO = 0, FG_SCHED_DATA_PARALLEL = 1, FG_SCHED_STREAM_K = 2 };

/* Bytes of device scratch fg_gemm needs for this problem under `schedule` (0 for the
 * data-parallel schedule).  The caller owns the buffer: 256-byte aligned, zero-filled ONCE when
 * it is allocated (the kernels leave their ticket counters at zero), and used by one stream at a
 * time.
 * Stands in for the per-call `locks`/`P` allocation of src/flag_gems/ops/mm_streamk.py:488-491. */
size_t fg_gemm_workspace_bytes(int64_t M, int64_t N, int64_t K, int ab_dtype, int schedule,
                               int device);

/* The largest value fg_gemm_workspace_bytes can return on `device` (a function of its CU count only), and the
 * size of the buffer's header: the part that must read zero when a launch starts (the ticket counters, which
 * the kernels return to zero).  A caller that sizes one buffer per stream to *max_bytes never has to replace
 * it, so pointers recorded in HIP graphs stay valid.  Stands in for the per-call allocation of
 * src/flag_gems/ops/mm_streamk.py:488-491. */
int fg_gemm_workspace_layout(int device, size_t* max_bytes /*host*/, size_t* header_bytes /*host*/);

/* *id = 0 when `stream` is not capturing into a HIP graph, otherwise a non-zero number unique to the capture in
 * progress.  Host code uses it to record one clearing of the workspace header per captured graph.  No counterpart
 * in the reference (its Triton launches allocate and clear per call). */
int fg_stream_capture_id(void* stream, unsigned long long* id /*host*/);

/* C[M,N] = alpha * (A[M,K] . B[K,N]) + beta * bias (bias == NULL: C = A.B), fp32 accumulate.
 * A, B, C and bias are addressed through (row, col) element strides; bias strides may be 0
 * (broadcast).  Which schedule ran is reported through *schedule_used when non-NULL.
 * Replaces mm_kernel_general (src/flag_gems/ops/mm.py:54-134), addmm_kernel
 * (src/flag_gems/ops/addmm.py:15-80), streamk_mm (src/flag_gems/ops/mm_streamk.py:451-576) and
 * their C++ twins lib/mm.cpp:71-332, lib/addmm.cpp:11-123. */
int fg_gemm(const void* A, const void* B, const void* bias, void* C, int64_t M, int64_t N,
            int64_t K, int64_t sam, int64_t sak, int64_t sbk, int64_t sbn, int64_t sim,
            int64_t sin_, int64_t scm, int64_t scn, float alpha, float beta, int ab_dtype,
            int c_dtype, int bias_dtype, int schedule, void* workspace, size_t workspace_bytes,
            int* schedule_used, void* stream);

/* fg_gemm for skinny problems WITHOUT a caller-provided workspace and without any device allocation: the
 * stream-K partial tiles and ticket counters live in a static device array of 4 198 656 bytes inside the library
 * (one copy per GPU, held until the process ends).  No counterpart in the reference; it is for callers that
 * cannot allocate: code under HIP graph capture, tight serving loops, harnesses that forbid hipMalloc.
 * Accepts what the skinny stream-K kernels accept: 16-bit inputs, M <= 64, K >= 1024, A with unit K stride and
 * 16-byte aligned rows, B row-major (M <= 16) or K-contiguous; anything else returns FG_ERR_UNSUPPORTED with a
 * message (use fg_gemm).  Results are bit-identical to fg_gemm's stream-K schedule.  All calls on one GPU share
 * the array: calls that overlap on one GPU (different streams) race; calls on one stream are safe.
 * The array's device address is looked up on the first call on a device (or by fg_device_info for that device);
 * the lookup cannot be made while the stream is being captured, so a first call that arrives under capture returns
 * FG_ERR_UNSUPPORTED with a message instead of breaking the capture. */
int fg_gemm_skinny_static(const void* A, const void* B, const void* bias, void* C, int64_t M, int64_t N,
                          int64_t K, int64_t sam, int64_t sak, int64_t sbk, int64_t sbn, int64_t sim,
                          int64_t sin_, int64_t scm, int64_t scn, float alpha, float beta, int ab_dtype,
                          int c_dtype, int bias_dtype, void* stream);

/* C[b] = A[b] . B[b] for b in [0, batch), fp32 accumulate, every operand addressed through
 * (matrix, row, col) element strides (a matrix stride of 0 broadcasts one operand).  Matrix b is
 * one data-parallel fg_gemm launch; the launches follow each other on the stream.
 * Verified envelope: at most FG_BMM_MAX_BATCH matrices and FG_BMM_MAX_OUT_ELEMS output elements per call; a call
 * beyond it returns FG_ERR_UNSUPPORTED with a message and launches nothing (a larger batch once ended in a GPU
 * memory fault whose cause is not known; callers split the batch or use the vendor library).
 * Replaces bmm_kernel (src/flag_gems/ops/bmm.py:15-136) and its C++ twin lib/bmm.cpp. */
#define FG_BMM_MAX_BATCH 16
#define FG_BMM_MAX_OUT_ELEMS (1LL << 24)
int fg_bmm(const void* A, const void* B, void* C, int64_t batch, int64_t M, int64_t N, int64_t K,
           int64_t sab, int64_t sam, int64_t sak, int64_t sbb, int64_t sbk, int64_t sbn,
           int64_t scb, int64_t scm, int64_t scn, int dtype, void* stream);

/* Host-side stream-K partition (pure integer function; also used by the tests).
 * Given `tiles` output tiles of `iters_per_tile` K-iterations each and `workers` persistent
 * workgroups, worker w owns the half-open range [begin[w], end[w]) of the tile-major iteration
 * space of the stream-K tiles; *sk_tiles receives how many tiles are cooperative.
 * Follows the split of src/flag_gems/ops/mm_streamk.py:466-485. */
int fg_streamk_partition(int64_t tiles, int64_t iters_per_tile, int64_t workers,
                         int64_t* sk_tiles, int64_t* begin /*host, [workers]*/,
                         int64_t* end /*host, [workers]*/);

/* POD mirror of the fields of FlashFwdParams (include/flag_gems/operators.h:126-194) that the
 * varlen paged forward uses. */
typedef struct FgFlashParams {
  const void* q;           /* [total_q, Hq, D] */
  const void* k_cache;     /* [num_pages, page_size, Hk, D] */
  const void* v_cache;     /* [num_pages, page_size, Hk, D] */
  void* out;               /* [total_q, Hq, D] */
  float* lse;              /* [Hq, total_q] fp32, may be NULL */
  const int32_t* cu_seqlens_q; /* [batch + 1] */
  const int32_t* seqused_k;    /* [batch] */
  const int32_t* block_table;  /* [batch, max_pages_per_seq] */
  const float* alibi_slopes;   /* [Hq] or [batch, Hq], may be NULL */
  int64_t q_row_stride, q_head_stride;     /* elements */
  int64_t o_row_stride, o_head_stride;
  int64_t k_page_stride, k_row_stride, k_head_stride;
  int64_t v_page_stride, v_row_stride, v_head_stride;
  int64_t block_table_stride;  /* elements between batch rows of block_table */
  int64_t alibi_batch_stride;  /* 0 when alibi_slopes is [Hq] */
  int64_t total_q;
  int32_t batch, Hq, Hk, D, page_size;
  int32_t max_seqlen_q, max_seqlen_k;
  int32_t is_causal;
  int32_t window_left, window_right; /* -1 = unbounded */
  float softmax_scale;
  float softcap;            /* 0 = off */
  int32_t dtype;            /* FG_F16 or FG_BF16 */
  void* workspace;          /* device scratch (split key ranges of single-token queries), may be NULL (see
                               fg_flash_attn_workspace_bytes) */
  int64_t workspace_bytes;
} FgFlashParams;

/* Forward of variable-length attention over a paged KV cache (FA2 semantics: bottom-right
 * aligned causal mask, GQA by head mapping, optional sliding window / softcap / alibi).
 * Replaces flash_varlen_fwd_kernel (src/flag_gems/ops/flash_kernel.py:1216-1577) and the launch
 * half of mha_varlan_fwd (src/flag_gems/ops/flash_api.py:230-569,
 * lib/flash_attn_varlen_func.cpp:14-481). */
int fg_flash_attn_varlen_fwd(const FgFlashParams* p /*host*/, void* stream);

/* Scratch the forward would like for these parameters: non-zero only for single-token queries
 * (max_seqlen_q == 1) whose key ranges are worth splitting over several workgroups; the partial
 * results of the ranges go there (the role of the reference's out_accum / softmax_lse_accum,
 * src/flag_gems/ops/flash_api.py:752-800).  The forward never needs it: without it (NULL or too
 * small) it runs unsplit.  Uninitialised memory is fine; one stream at a time. */
size_t fg_flash_attn_workspace_bytes(const FgFlashParams* p /*host*/, int device);

/* ------------------------------------------------------------------------------------------------------------
 * Diagnostics.  Not part of the operator interface: nothing above depends on a caller using them, and a binder of
 * the operators can leave them out.  They exist for the library's own tests and benchmark: host-side views of
 * decisions the kernels and launchers make (so that those can be checked without a GPU), the matrix-core
 * calibration loop, and the re-reading of the FG_* switches.  None has a counterpart in the reference's operator
 * interface; where a comment names reference code, it is the logic the reported decision stands in for.
 * ------------------------------------------------------------------------------------------------------------ */

/* Re-reads the FG_* measurement and test switches from the environment.  The library reads them once, on first
 * use; no entry point consults the environment per call.  No counterpart in the reference. */
void fg_reload_options(void);

/* Calibration of the matrix-core roofline (no counterpart in the reference; used by bench.py):
 * every wave of `blocks` 256-thread workgroups issues 64 * iters MFMA 16x16x32 bf16 on operand
 * fragments read once from `operands` (8 * 256 * 16 bytes).  `out` receives blocks * 256 floats;
 * *flops the floating-point operations of the launch.  The sustained rate depends on the operand
 * bits (power): random operands give the ceiling a real bf16 GEMM can approach on this part. */
int fg_mfma_probe(const void* operands, float* out, int blocks, int iters, double* flops, void* stream);

/* What fg_gemm's automatic schedule selects for 16-bit operands that qualify for the direct-to-LDS kernels (16-byte
 * aligned rows, unit stride along K or N, K a multiple of 64) on a device of `num_cu` compute units (<= 0: the
 * current device's): the workgroup tile of the data-parallel launch with its modelled duration in microseconds, and
 * the number of workgroups and modelled duration of the stream-K launch on 128x128 tiles (*streamk_workers = 0 when
 * the problem does not qualify for it: more tiles than CUs or fewer than four K steps per CU).  *streamk_chosen tells
 * which of the two the automatic schedule takes when a workspace is given.  Host arithmetic only when num_cu > 0: no
 * device is touched.  Any output pointer may be NULL.
 * Stands in for the tuned-configuration lookup of src/flag_gems/ops/mm.py:54-62 and the schedule test
 * streamk_scenario, src/flag_gems/ops/mm.py:186-197. */
int fg_gemm_plan(int64_t M, int64_t N, int64_t K, int num_cu, int* tile_m /*host*/, int* tile_n /*host*/,
                 double* dp_us /*host*/, int* streamk_workers /*host*/, double* streamk_us /*host*/,
                 int* streamk_chosen /*host*/);

/* The order in which a data-parallel launch of tiles_m x tiles_n workgroup tiles walks its grid: workgroup id i
 * computes tile (tile_m[i], tile_n[i]); both arrays hold tiles_m * tiles_n entries.  Workgroup i runs on XCD i mod 8,
 * so the order decides which A and B panels share an L2.  b_k_contiguous selects the variant used for B = W^T
 * (non-zero) or row-major B.  Host arithmetic only; the kernels call the same function.
 * Stands in for the grouped ordering of mm_kernel_general, src/flag_gems/ops/mm.py:83-91 (GROUP_M grouping of the program ids). */
int fg_gemm_tile_order(int tiles_m, int tiles_n, int b_k_contiguous, int* tile_m /*host*/, int* tile_n /*host*/);

#ifdef __cplusplus
}
#endif
#endif /* FG_MI355_H */
