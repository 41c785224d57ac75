"""`torch.ops.flag_gems.*`: the custom-operator namespace of the reference's C extension, for the
operators of this path.

The reference defines these schemas in C++ (src/flag_gems/csrc/cstub.cpp:26-90) and binds them to its
C++ wrappers on the CUDA key (:91-129); its Python layer calls them when `config.use_c_extension` is
set (src/flag_gems/ops/attention.py:1199-1229, fused/reshape_and_cache_flash.py:71-83,
modules/normalization.py:38-55, modules/rotary_embedding.py:45-60).  Here the schema strings are the
reference's, and every kernel registered on the CUDA key is the Python wrapper of this package, which
makes one C-ABI call into libfg_mi355.so.  Argument meaning follows the C++ wrappers: norms take the
weight's length as the normalised extent (lib/rms_norm.cpp:15-22, lib/fused_add_rms_norm.cpp:14-27),
flash_attn_varlen_func always returns (out, softmax_lse) (lib/flash_attn_varlen_func.cpp:487-579).
"""
import torch

# (schema, name of the kernel function below).  Strings as in cstub.cpp, whitespace normalised.
SCHEMAS = (
    ("addmm(Tensor self, Tensor mat1, Tensor mat2, *, Scalar beta=1, Scalar alpha=1) -> Tensor", "_addmm"),
    ("bmm(Tensor self, Tensor mat2) -> Tensor", "_bmm"),
    ("mm(Tensor self, Tensor mat2) -> Tensor", "_mm"),
    ("rms_norm(Tensor input, Tensor weight, float epsilon) -> Tensor", "_rms_norm"),
    ("fused_add_rms_norm(Tensor! input, Tensor! residual, Tensor weight, float epsilon) -> ()",
     "_fused_add_rms_norm"),
    ("rotary_embedding_inplace(Tensor! q, Tensor! k, Tensor cos, Tensor sin, Tensor? position_ids=None, "
     "bool rotary_interleaved=False) -> ()", "_rotary_embedding_inplace"),
    ("rotary_embedding(Tensor q, Tensor k, Tensor cos, Tensor sin, Tensor? position_ids=None, "
     "bool rotary_interleaved=False) -> (Tensor, Tensor)", "_rotary_embedding"),
    ("softmax(Tensor input, int dim, bool half_to_float=False) -> Tensor", "_softmax"),
    ("softmax_backward(Tensor grad_output, Tensor output, int dim, ScalarType input_dtype) -> Tensor",
     "_softmax_backward"),
    ("reshape_and_cache_flash(Tensor key, Tensor value, Tensor(a!) key_cache, Tensor(b!) value_cache, "
     "Tensor slot_mapping, str kv_cache_dtype, Tensor? k_scale=None, Tensor? v_scale=None) -> ()",
     "_reshape_and_cache_flash"),
    ("flash_attn_varlen_func(Tensor q, Tensor k, Tensor v, SymInt max_seqlen_q, Tensor cu_seqlens_q, "
     "SymInt max_seqlen_k, Tensor? cu_seqlens_k=None, Tensor? seqused_k=None, Tensor? q_v=None, "
     "float dropout_p=0.0, float? softmax_scale=None, bool causal=False, SymInt[]? window_size=None, "
     "float softcap=0.0, Tensor? alibi_slopes=None, bool deterministic=False, bool return_attn_probs=False, "
     "Tensor? block_table=None, bool return_softmax_lse=False, Tensor? out=None, "
     "Tensor? scheduler_metadata=None, Tensor? q_descale=None, Tensor? k_descale=None, "
     "Tensor? v_descale=None, SymInt fa_version=2) -> (Tensor, Tensor)", "_flash_attn_varlen_func"),
)


def _addmm(self, mat1, mat2, *, beta=1, alpha=1):
    from .ops import addmm
    return addmm(self, mat1, mat2, beta=beta, alpha=alpha)


def _bmm(self, mat2):
    from .ops import bmm
    return bmm(self, mat2)


def _mm(self, mat2):
    from .ops import mm
    return mm(self, mat2)


def _rms_norm(input, weight, epsilon):
    from .ops import rms_norm
    return rms_norm(input, [weight.shape[0]], weight, epsilon)


def _fused_add_rms_norm(input, residual, weight, epsilon):
    from .fused import fused_add_rms_norm
    if input.shape != residual.shape:
        raise RuntimeError(
            f"Input and residual must have the same shape, but got {list(input.shape)} vs {list(residual.shape)}")
    y, r = fused_add_rms_norm(input, residual, [weight.shape[0]], weight, epsilon)
    # the schema promises mutation of the arguments; the wrapper works on copies of tensors whose
    # rows are not dense
    if y.data_ptr() != input.data_ptr():
        input.copy_(y)
    if r.data_ptr() != residual.data_ptr():
        residual.copy_(r)


def _rotary_embedding_inplace(q, k, cos, sin, position_ids=None, rotary_interleaved=False):
    from .fused import apply_rotary_pos_emb
    apply_rotary_pos_emb(q, k, cos, sin, position_ids, rotary_interleaved, inplace=True)


def _rotary_embedding(q, k, cos, sin, position_ids=None, rotary_interleaved=False):
    from .fused import apply_rotary_pos_emb
    return apply_rotary_pos_emb(q, k, cos, sin, position_ids, rotary_interleaved, inplace=False)


def _softmax(input, dim, half_to_float=False):
    from .ops import softmax
    return softmax(input, dim, half_to_float)


def _softmax_backward(grad_output, output, dim, input_dtype):
    from .ops import softmax_backward
    return softmax_backward(grad_output, output, dim, input_dtype)


def _reshape_and_cache_flash(key, value, key_cache, value_cache, slot_mapping, kv_cache_dtype, k_scale=None,
                             v_scale=None):
    from .fused import reshape_and_cache_flash
    reshape_and_cache_flash(key, value, key_cache, value_cache, slot_mapping, kv_cache_dtype, k_scale, v_scale)


def _flash_attn_varlen_func(q, k, v, max_seqlen_q, cu_seqlens_q, max_seqlen_k, cu_seqlens_k=None, seqused_k=None,
                            q_v=None, dropout_p=0.0, softmax_scale=None, causal=False, window_size=None, softcap=0.0,
                            alibi_slopes=None, deterministic=False, return_attn_probs=False, block_table=None,
                            return_softmax_lse=False, out=None, scheduler_metadata=None, q_descale=None,
                            k_descale=None, v_descale=None, fa_version=2):
    from .ops import flash_attn_varlen_func
    res, lse = flash_attn_varlen_func(
        q, k, v, max_seqlen_q, cu_seqlens_q, max_seqlen_k, cu_seqlens_k=cu_seqlens_k, seqused_k=seqused_k, q_v=q_v,
        dropout_p=dropout_p, softmax_scale=softmax_scale, causal=causal,
        window_size=None if window_size is None else list(window_size), softcap=softcap, alibi_slopes=alibi_slopes,
        deterministic=deterministic, return_attn_probs=return_attn_probs, block_table=block_table,
        return_softmax_lse=True, out=out, scheduler_metadata=scheduler_metadata, q_descale=q_descale,
        k_descale=k_descale, v_descale=v_descale, fa_version=fa_version)
    return res, lse


# A namespace can be defined once per process: both import names (flaggems_amd, flag_gems) share this module.
_def_lib = torch.library.Library("flag_gems", "DEF")
_impl_lib = torch.library.Library("flag_gems", "IMPL")
for _schema, _fn in SCHEMAS:
    _def_lib.define(_schema)
    _impl_lib.impl(_schema.split("(", 1)[0], globals()[_fn], "CUDA")


def op_names():
    """Names defined under torch.ops.flag_gems."""
    return [s.split("(", 1)[0] for s, _ in SCHEMAS]
