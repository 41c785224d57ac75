"""Scatter of K/V rows into the paged cache of the older vLLM layout
(reference: src/flag_gems/fused/reshape_and_cache.py:70-112)."""
import logging

import torch

from .. import _C

logger = logging.getLogger("flag_gems.fused.reshape_and_cache")


def reshape_and_cache(
    key,  # [num_tokens, num_heads, head_size]
    value,  # [num_tokens, num_heads, head_size]
    key_cache,  # [num_blocks, num_heads, head_size/x, block_size, x]
    value_cache,  # [num_blocks, num_heads, head_size, block_size]
    slot_mapping,  # [num_tokens]
    kv_cache_dtype,
    k_scale,
    v_scale,
):
    """kv_cache_dtype, k_scale and v_scale are accepted and ignored, as in the reference (no fp8 cache).
    The caches must be contiguous; of key/value only the token stride is free."""
    logger.debug("GEMS RESHAPE_AND_CACHE")
    num_tokens = slot_mapping.size(0)
    num_heads = key.size(1)
    head_size = key.size(2)
    num_blocks = key_cache.size(0)
    block_size = key_cache.size(3)
    x = key_cache.size(4)
    assert tuple(key_cache.shape) == (num_blocks, num_heads, head_size // x, block_size, x) and head_size % x == 0, \
        "key_cache must be [num_blocks, num_heads, head_size / x, block_size, x]"
    assert tuple(value_cache.shape) == (num_blocks, num_heads, head_size, block_size), \
        "value_cache must be [num_blocks, num_heads, head_size, block_size]"
    assert key_cache.is_contiguous() and value_cache.is_contiguous(), "the caches must be contiguous"
    assert key.dtype == value.dtype == key_cache.dtype == value_cache.dtype, "key/value/cache dtypes must match"
    assert key.shape == value.shape and key.size(0) >= num_tokens
    assert key[0].is_contiguous() and value[0].is_contiguous() if num_tokens else True, \
        "the [num_heads, head_size] block of a token must be dense"
    assert slot_mapping.dtype in (torch.int64, torch.int32), "slot_mapping must be int64 or int32"
    assert slot_mapping.stride(0) == 1 or num_tokens <= 1, "slot_mapping must be contiguous"
    if num_tokens == 0:
        return
    with _C.device_guard(key.device):
        rc = _C.lib().fg_reshape_and_cache(
            key.data_ptr(), value.data_ptr(), key_cache.data_ptr(), value_cache.data_ptr(),
            slot_mapping.data_ptr(), 1 if slot_mapping.dtype == torch.int64 else 0,
            num_tokens, num_heads, head_size, block_size, x, num_blocks, key.stride(0), value.stride(0),
            key.element_size(), _C.current_stream(key.device),
        )
    _C.check(rc, "fg_reshape_and_cache")
