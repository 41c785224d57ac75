"""Scatter of K/V rows into the paged cache
(reference: src/flag_gems/fused/reshape_and_cache_flash.py:61-112)."""
import logging

import torch

from .. import _C

logger = logging.getLogger("flag_gems.fused.reshape_and_cache_flash")


def reshape_and_cache_flash(
    key,  # [num_tokens, num_heads, head_size]
    value,  # [num_tokens, num_heads, head_size]
    key_cache,  # [num_blocks, block_size, num_heads, head_size]
    value_cache,  # [num_blocks, block_size, num_heads, head_size]
    slot_mapping,  # [num_tokens]
    kv_cache_dtype,
    k_scale,
    v_scale,
):
    """kv_cache_dtype, k_scale and v_scale are accepted and ignored, as in the reference (no fp8
    cache).  Only the token stride of key/value and the page stride of the caches are consulted:
    the inner [heads, head_size] block of a token must be dense."""
    logger.debug("GEMS RESHAPE_AND_CACHE_FLASH")
    num_tokens = slot_mapping.size(0)
    num_heads = key.size(1)
    head_size = key.size(2)
    block_size = key_cache.size(1)
    assert key_cache.stride(0) == value_cache.stride(0)
    assert key.dtype == value.dtype == key_cache.dtype == value_cache.dtype, "key/value/cache dtypes must match"
    assert slot_mapping.dtype in (torch.int64, torch.int32), "slot_mapping must be int64 or int32"
    assert slot_mapping.stride(0) == 1 or num_tokens <= 1, "slot_mapping must be contiguous"
    if num_tokens == 0:
        return
    with _C.device_guard(key.device):
        rc = _C.lib().fg_reshape_and_cache_flash(
            key.data_ptr(), value.data_ptr(), key_cache.data_ptr(), value_cache.data_ptr(),
            slot_mapping.data_ptr(), 1 if slot_mapping.dtype == torch.int64 else 0,
            num_tokens, num_heads, head_size, block_size,
            key.stride(0), value.stride(0), key_cache.stride(0), key.element_size(),
            _C.current_stream(key.device),
        )
    _C.check(rc, "fg_reshape_and_cache_flash")
