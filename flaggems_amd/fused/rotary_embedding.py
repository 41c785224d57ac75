"""Rotary position embedding (reference: src/flag_gems/fused/rotary_embedding.py:181-312)."""
import logging
from typing import Optional

import torch

from .. import _C

logger = logging.getLogger("flag_gems.fused.rotary_embedding")


def apply_rotary_pos_emb(
    q,
    k,
    cos,
    sin,
    position_ids: Optional[torch.IntTensor] = None,
    rotary_interleaved: bool = False,
    inplace: bool = False,
):
    """
    Apply rotary position embedding to q and k

    Args:
        q: (*, q_heads, head_dim)
        k: (*, k_heads, head_dim)
        cos: (max_seq_len, head_dim // 2)
        sin: (max_seq_len, head_dim // 2)
        position_ids: (*, ), optional, position ids for each token
        rotary_interleaved: whether the head_dim is rotated in an interleaved way
        inplace: rotate q and k in their own storage

    Returns:
        q_embed: (*, q_heads, head_dim)
        k_embed: (*, k_heads, head_dim)
    """
    logger.debug("GEMS ROTARY_POS_EMBEDDING")
    assert k.shape[-1] == q.shape[-1], f"q and k must have the same last dimension, got {q.shape} and {k.shape}"
    assert cos.shape[-1] == sin.shape[-1], f"cos and sin must have the same last dimension, got {cos.shape} and {sin.shape}"
    assert cos.shape[-1] * 2 == q.shape[-1], f"cos/sin dim must be half of q/k dim, got {cos.shape} and {q.shape}"
    assert cos.stride(-1) == 1, "cos must be contiguous at the last dimension"
    assert sin.stride(-1) == 1, "sin must be contiguous at the last dimension"
    assert q.dtype == k.dtype, "q and k must share a dtype"
    assert cos.dtype == sin.dtype, "cos and sin must share a dtype"

    q_shape = q.shape
    k_shape = k.shape
    assert q.shape[:-2] == k.shape[:-2], f"q and k must have the same length, got {q.shape[:-2]} and {k.shape[:-2]}"
    if position_ids is None:
        assert len(q.shape) == 4, f"q must have 4 dimensions if position_ids is not provided, got {q.shape}"
        seq_len = q.shape[-3]
    else:
        assert (
            position_ids.shape == q.shape[:-2]
        ), f"position_ids must have the same length as q, got {position_ids.shape} and {q.shape[:-2]}"
        assert position_ids.dtype in (torch.int64, torch.int32), "position_ids must be int64 or int32"
        position_ids = position_ids.reshape(-1)
        seq_len = 0

    flat = len(q_shape) == 3  # already (tokens, heads, head_dim), what a serving engine passes: no views to make
    if not flat:
        q = q.view(-1, q.shape[-2], q.shape[-1])
        k = k.view(-1, k.shape[-2], k.shape[-1])
    n_tokens, q_heads, head_dim = q.shape
    k_heads = k.shape[1]

    if inplace:
        q_embed, k_embed = q, k
    else:
        q_embed = torch.empty_like(q)
        k_embed = torch.empty_like(k)

    if n_tokens > 0 and head_dim > 0:
        I3 = _C.I64x3
        qs, ks = I3(*q.stride()), I3(*k.stride())
        with _C.device_guard(q.device):
            rc = _C.lib().fg_rope(
                q_embed.data_ptr(), k_embed.data_ptr(), q.data_ptr(), k.data_ptr(), cos.data_ptr(), sin.data_ptr(),
                position_ids.data_ptr() if position_ids is not None else None,
                1 if (position_ids is not None and position_ids.dtype == torch.int64) else 0,
                n_tokens, seq_len, q_heads, k_heads, head_dim,
                qs, ks, qs if inplace else I3(*q_embed.stride()), ks if inplace else I3(*k_embed.stride()),
                position_ids.stride(0) if position_ids is not None else 0,
                cos.stride(0) if cos.ndim > 1 else 0, sin.stride(0) if sin.ndim > 1 else 0, cos.shape[0],
                1 if rotary_interleaved else 0, _C.dtype_id(q.dtype), _C.dtype_id(cos.dtype),
                _C.current_stream(q.device),
            )
        _C.check(rc, "fg_rope")
    if flat:
        return q_embed, k_embed
    return q_embed.view(q_shape), k_embed.view(k_shape)
