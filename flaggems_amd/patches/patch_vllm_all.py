"""vLLM layer methods re-implemented on this package's operators, and the function that installs them
(reference: src/flag_gems/patches/patch_vllm_all.py:9-368).

Installed: RMSNorm.forward_cuda, RotaryEmbedding.forward_cuda, SiluAndMul.forward_cuda, the v1
FlashAttentionImpl.forward, PagedAttention.write_to_paged_cache and the `_C::silu_and_mul` kernel.  The
reference also replaces the MLA decode, two MoE routing kernels and the FA3 scheduler-metadata op; those are
not operators of this package and stay on vLLM's own kernels.
"""
from typing import Optional, Tuple

import torch

from .patch_util import patch_module_method, patch_vllm_lib

# what apply_gems_patches_to_vllm() leaves alone, for its report
_LEFT_ON_VLLM = (
    "TritonMLAImpl._forward_decode",
    "torch.ops._moe_C.moe_align_block_size",
    "torch.ops._moe_C.topk_softmax",
    "torch.ops._vllm_fa3_C.get_scheduler_metadata",
)


def custom_gems_rms_forward_cuda(self, x, residual=None):
    """RMSNorm.forward_cuda: plain norm, or residual add + norm returning (normed, new residual)."""
    from ..modules.normalization import gems_rms_forward

    return gems_rms_forward(x, residual, self.weight, self.variance_epsilon)


def custom_gems_rope_forward_cuda(
    self,
    positions: torch.Tensor,
    query: torch.Tensor,
    key: torch.Tensor,
    offsets: Optional[torch.Tensor] = None,
) -> Tuple[torch.Tensor, torch.Tensor]:
    """RotaryEmbedding.forward_cuda: rotate the first rotary_dim features of every head in place, by the
    layer's [max_position, rotary_dim] table whose halves are cos and sin."""
    from ..modules.rotary_embedding import gems_rope_forward

    self.cos_sin_cache = self.cos_sin_cache.to(positions.device)
    pos = (positions if offsets is None else positions + offsets).flatten()
    tokens = pos.shape[0]
    q_shape, k_shape = query.shape, key.shape
    q = query.view(tokens, -1, self.head_size)
    k = key.view(tokens, -1, self.head_size)
    partial = self.rotary_dim < self.head_size
    cos, sin = self.cos_sin_cache.chunk(2, dim=-1)
    q_rot, k_rot = gems_rope_forward(
        q[..., : self.rotary_dim], k[..., : self.rotary_dim], cos, sin, position_ids=pos,
        rotary_interleaved=not self.is_neox_style, inplace=True,
    )
    if partial:
        q_rot = torch.cat((q_rot, q[..., self.rotary_dim:]), dim=-1)
        k_rot = torch.cat((k_rot, k[..., self.rotary_dim:]), dim=-1)
    return q_rot.reshape(q_shape), k_rot.reshape(k_shape)


def custom_gems_silu_and_mul(self, x: torch.Tensor) -> torch.Tensor:
    """SiluAndMul.forward_cuda: silu(x[..., :d]) * x[..., d:]."""
    from ..modules.activation import gems_silu_and_mul

    d = x.shape[-1] // 2
    return gems_silu_and_mul(x[..., :d], x[..., d:])


def custom_silu_and_mul(out: torch.Tensor, input: torch.Tensor):
    """torch.ops._C.silu_and_mul(out, input)."""
    from ..fused.silu_and_mul import silu_and_mul_out

    d = input.size(-1) // 2
    silu_and_mul_out(input[..., :d], input[..., d:], out)


def custom_gems_write_to_paged_cache(key, value, key_cache, value_cache, slot_mapping, kv_cache_dtype, k_scale, v_scale):
    """PagedAttention.write_to_paged_cache (a static method of the v0 backend): K/V rows into the
    [blocks, heads, head_size / x, block_size, x] / [blocks, heads, head_size, block_size] caches."""
    from ..fused.reshape_and_cache import reshape_and_cache

    reshape_and_cache(key, value, key_cache, value_cache, slot_mapping.flatten(), kv_cache_dtype, k_scale, v_scale)


def custom_gems_flash_attention_impl_forward(
    self,
    layer: torch.nn.Module,
    query: torch.Tensor,
    key: torch.Tensor,
    value: torch.Tensor,
    kv_cache: torch.Tensor,
    attn_metadata,
    output: Optional[torch.Tensor] = None,
    output_scale: Optional[torch.Tensor] = None,
) -> torch.Tensor:
    """v1 FlashAttentionImpl.forward: append this step's K/V to the paged cache, then attend over it.
    query [tokens, heads, d]; kv_cache [2, pages, page_size, kv_heads, d]; writes output[:num_actual_tokens]."""
    from ..fused.reshape_and_cache_flash import reshape_and_cache_flash
    from ..ops.attention import flash_attn_varlen_func

    assert output is not None, "Output tensor must be provided."
    if output_scale is not None:
        raise NotImplementedError("fused output quantization is not yet supported for FlashAttentionImpl")
    if attn_metadata is None:  # memory-profiling pass
        return output
    if self.kv_cache_dtype.startswith("fp8"):
        raise NotImplementedError("FP8 quantization is not yet supported for FlashAttentionImpl")

    n = attn_metadata.num_actual_tokens
    key_cache, value_cache = kv_cache.unbind(0)
    reshape_and_cache_flash(
        key, value, key_cache, value_cache, attn_metadata.slot_mapping, self.kv_cache_dtype,
        layer._k_scale, layer._v_scale,
    )

    local = getattr(attn_metadata, "local_attn_metadata", None) if self.use_irope else None
    if attn_metadata.use_cascade and local is None:
        raise NotImplementedError("Cascade attention is not implemented in flag_gems.")
    if local is not None:
        cu_q, used_k = local.local_query_start_loc, local.local_seqused_k
        max_q, max_k = local.local_max_query_len, local.local_max_seq_len
        table, sched = local.local_block_table, local.local_scheduler_metadata
    else:
        cu_q, used_k = attn_metadata.query_start_loc, attn_metadata.seq_lens
        max_q, max_k = attn_metadata.max_query_len, attn_metadata.max_seq_len
        table, sched = attn_metadata.block_table, attn_metadata.scheduler_metadata
    descale_shape = (cu_q.shape[0] - 1, key.shape[1])
    flash_attn_varlen_func(
        q=query[:n], k=key_cache, v=value_cache, out=output[:n],
        cu_seqlens_q=cu_q, max_seqlen_q=max_q, seqused_k=used_k, max_seqlen_k=max_k,
        softmax_scale=self.scale, causal=True, alibi_slopes=self.alibi_slopes, window_size=self.sliding_window,
        block_table=table, softcap=self.logits_soft_cap, scheduler_metadata=sched, fa_version=2,
        q_descale=layer._q_scale.expand(descale_shape), k_descale=layer._k_scale.expand(descale_shape),
        v_descale=layer._v_scale.expand(descale_shape),
    )
    return output


def apply_gems_patches_to_vllm(verbose=True):
    """Install the replacements above into an importable vLLM (raises ImportError without one)."""
    import vllm  # noqa: F401
    from vllm.attention.ops.paged_attn import PagedAttention
    from vllm.model_executor.layers.activation import SiluAndMul
    from vllm.model_executor.layers.layernorm import RMSNorm
    from vllm.model_executor.layers.rotary_embedding import RotaryEmbedding
    from vllm.v1.attention.backends.flash_attn import FlashAttentionImpl

    patch_module_method(RMSNorm, "forward_cuda", custom_gems_rms_forward_cuda, verbose)
    patch_module_method(RotaryEmbedding, "forward_cuda", custom_gems_rope_forward_cuda, verbose)
    patch_module_method(PagedAttention, "write_to_paged_cache", custom_gems_write_to_paged_cache, verbose)
    patch_module_method(SiluAndMul, "forward_cuda", custom_gems_silu_and_mul, verbose)
    patch_module_method(FlashAttentionImpl, "forward", custom_gems_flash_attention_impl_forward, verbose)
    patch_vllm_lib("_C", "silu_and_mul", custom_silu_and_mul, "CUDA", verbose)
    if verbose:
        for name in _LEFT_ON_VLLM:
            print(f"Left {name} on vLLM (not an operator of this package)")
