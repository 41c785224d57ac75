// Compile-time switches for kernel variants that have not yet passed the parity suite on an MI355X.
//
// Every switch defaults to the code the suite last passed on (0, or the value stated).  A variant is built by passing
// -DFG_V_<NAME>=1 to the compiler (csrc/build.py: FG_VARIANTS="ROWS_UPFRONT=1,..." with FG_LIB_SUFFIX naming the
// library it lands in), goes through `pytest -m gpu` before it is timed, and becomes the default only with both in
// hand.  With every switch at its default the device assembly of the library is, kernel by kernel, that of the tested
// sources.
#pragma once

// rms_rows_kernel, softmax_rows_kernel, bwd_rows_kernel: every pack of a thread (and, up to two packs, the norm weight)
// is loaded unconditionally at the top of the kernel, from clamped addresses, and the tail's kernel arguments are named
// there, so that one wait covers them all.  Tested code: each pack is loaded under its own bounds check.
#ifndef FG_V_ROWS_UPFRONT
#define FG_V_ROWS_UPFRONT 0
#endif

// rms_norm / fused_add_rms_norm, rows of one pack per thread on 256-1024 threads, up to 32768 rows: two rows per
// workgroup (rms_rows2_kernel), all requests of both rows up front, one LDS exchange for both row sums.  Halves the
// rounds of workgroups of a small matrix ([4096, 4096]: four rounds -> two).  Tested code: one row per workgroup.
#ifndef FG_V_RMS_TWO_ROWS
#define FG_V_RMS_TWO_ROWS 0
#endif

// rms_short_kernel, softmax_short_kernel, bwd_short_kernel (one wave per short or unaligned row): elements loaded
// unconditionally from clamped columns before the first use.  Tested code: each element under its own bounds check.
#ifndef FG_V_SHORT_UPFRONT
#define FG_V_SHORT_UPFRONT 0
#endif

// cache_scatter_kernel: the first four 16-byte pieces of a token's row are requested together with its slot.
// Tested code: the slot is read first, the row behind it.
#ifndef FG_V_SCATTER_EARLY
#define FG_V_SCATTER_EARLY 0
#endif

// rope_kernel: q/k strides selected by value and the arguments of the second half named at the top.
// Tested code: strides selected through a pointer into the argument block.
#ifndef FG_V_ROPE_ARGS
#define FG_V_ROPE_ARGS 0
#endif

// attn_varlen_pipe_kernel: Q loaded unconditionally from the clamped row address and zeroed afterwards.
// Tested code: each 16-byte Q load under the row bounds check.
#ifndef FG_V_ATTN_Q_UNCOND
#define FG_V_ATTN_Q_UNCOND 0
#endif

// attn_varlen_pipe_kernel: the softmax row sums are taken by one extra MFMA per column tile and half-tile step (a
// fragment of ones times P^T) instead of sixteen vector additions per step; the normaliser then sums P as rounded for
// the PV product.  Tested code: lane-local fp32 sums on the vector ALU, added across lane groups in the epilogue.
#ifndef FG_V_ATTN_ROWSUM_MFMA
#define FG_V_ATTN_ROWSUM_MFMA 0
#endif

// attn_decode_kernel: Q requested together with the page ids, in front of the one wait before the first tile copies.
// Tested code: Q loaded at the top of the kernel under the row check.
#ifndef FG_V_DECODE_Q_EARLY
#define FG_V_DECODE_Q_EARLY 0
#endif

// rms_bwd_fetch (rms_norm backward without prefetch): packs of rows past the end zeroed as whole 16-byte values, which
// keeps the two-pack variant (rows of 8193-16384 elements) out of scratch memory.  Tested code: zeroed element by element.
#ifndef FG_V_RMS_BWD_ZERO_PACK
#define FG_V_RMS_BWD_ZERO_PACK 0
#endif

// gemm_skinny_kc_kernel with more than 8 rows of A: the A fragments are loaded by asm and made valid by the counted
// wait the LDS copies already use, instead of compiler-placed waits, which drain everything in flight once per trip of
// the main loop (every RING steps).  Tested code: plain loads, compiler-placed waits.
#ifndef FG_V_SKINNY_ASM_A
#define FG_V_SKINNY_ASM_A 0
#endif

// dma_tile_epilogue: the broadcast-bias case of addmm takes a branch of its own.
// Tested code: one branch for both kinds of bias.
#ifndef FG_V_ADDMM_BCAST_BRANCH
#define FG_V_ADDMM_BCAST_BRANCH 0
#endif

// gemm_dma main loop: the tile's two operand bases are made scalar once, in front of the loop, with the five wait
// states a scalar register written by a vector instruction needs before a memory instruction may read it; the asm
// copies are invisible to the compiler's hazard recognizer.  Tested code: the bases are made scalar per K step, and
// the build's assembly scan (isa_check.py) verifies that the scheduler left enough instructions in between.
#ifndef FG_V_DMA_SCALAR_BASES
#define FG_V_DMA_SCALAR_BASES 0
#endif

// gemm_dma main loop: quarter steps of a K step that issue copies.  2 = the tested loop; 3 = three quarters on the
// 256x256 two-stage tile (timed at +2-6 % with products checked on five shapes, never through the parity suite).
#ifndef FG_V_DMA_COPY_RUNS
#define FG_V_DMA_COPY_RUNS 2
#endif

// fg_silu_and_mul_backward: the gradient kernel of silu_and_mul (silu_mul_grad_kernel).  A new kernel, not a change to
// a tested one; it is compiled only with the switch on, and until then the entry point answers FG_ERR_UNSUPPORTED and
// the Python operator takes its gradient from the vendor's elementwise kernels.
#ifndef FG_V_SILU_GRAD_KERNEL
#define FG_V_SILU_GRAD_KERNEL 0
#endif
