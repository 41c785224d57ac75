"""flash_attn_varlen_func over a paged KV cache on the gfx950 attention kernel.

API shim: src/flag_gems/ops/attention.py:1118-1287.  Host checks and parameter preparation:
mha_varlan_fwd, src/flag_gems/ops/flash_api.py:230-569.
"""
import ctypes
import logging

import torch

from .. import _C

logger = logging.getLogger("flag_gems.ops.attention")


def maybe_contiguous(x):
    return x.contiguous() if x is not None and x.stride(-1) != 1 else x


def mha_varlan_fwd(
    q, k, v, out, cu_seqlens_q, cu_seqlens_k, seqused_k, leftpad_k, page_table, alibi_slopes,
    max_seqlen_q, max_seqlen_k, p_dropout, softmax_scale, zero_tensors, is_causal,
    window_size_left, window_size_right, softcap, return_softmax, gen,
):
    """Validation + launch.  Returns (out, q, k, v, lse, philox_args, unused, p) like the reference;
    the last three are placeholders because dropout is not part of the inference path."""
    assert q.is_cuda and k.is_cuda and v.is_cuda
    q_dtype = q.dtype
    assert q_dtype in (torch.float16, torch.bfloat16), "FlashAttention only support fp16 and bf16 data type"
    assert q_dtype == k.dtype
    assert q_dtype == v.dtype
    assert q.stride(-1) == 1, "Input tensor must have contiguous last dimension"
    assert k.stride(-1) == 1, "Input tensor must have contiguous last dimension"
    assert v.stride(-1) == 1, "Input tensor must have contiguous last dimension"
    assert cu_seqlens_q.dtype == torch.int32
    assert cu_seqlens_q.is_contiguous()
    assert cu_seqlens_k.dtype == torch.int32
    assert cu_seqlens_k.is_contiguous()
    assert page_table is not None
    assert page_table.dtype == torch.int32 and page_table.stride(-1) == 1

    total_q, num_heads, head_size = q.size()
    num_heads_k = k.size(2)
    batch_size = cu_seqlens_q.numel() - 1
    block_size = k.size(1)
    num_pages = k.size(0)

    assert k.size() == v.size()
    assert cu_seqlens_q.size() == (batch_size + 1,)
    assert cu_seqlens_k.size() == (batch_size + 1,)
    if out is not None:
        assert out.stride(-1) == 1
        assert out.dtype == q.dtype
        assert out.size() == (total_q, num_heads, head_size)
    assert seqused_k is not None, "the paged kernel takes key lengths from seqused_k"
    assert seqused_k.dtype == torch.int32
    assert seqused_k.is_contiguous()
    assert seqused_k.size() == (batch_size,)

    if max_seqlen_q == 1 and alibi_slopes is None:
        is_causal = False
    if is_causal:
        window_size_right = 0
    if window_size_left >= max_seqlen_k:
        window_size_left = -1
    if window_size_right >= max_seqlen_k:
        window_size_right = -1

    assert leftpad_k is None, "leftpad_k is not supported."
    assert head_size <= 256, "FlashAttention forward only supports head dimension at most 256"
    assert head_size % 8 == 0, "head_size must be a multiple of 8, this is ensured by padding!"
    assert num_heads % num_heads_k == 0, "Number of heads in key/value must divide number of heads in query"
    assert k.shape == (num_pages, block_size, num_heads_k, head_size)
    assert k.stride() == v.stride()
    assert p_dropout == 0, "dropout is not implemented on this path (inference only)"
    assert not return_softmax, "return_softmax needs dropout, which is not implemented"

    if alibi_slopes is not None:
        assert alibi_slopes.device == q.device
        assert alibi_slopes.dtype in (torch.float,)
        assert alibi_slopes.stride(-1) == 1
        assert alibi_slopes.shape == (num_heads,) or alibi_slopes.shape == (batch_size, num_heads)
        alibi_batch_stride = alibi_slopes.stride(0) if alibi_slopes.ndim == 2 else 0
    else:
        alibi_batch_stride = 0

    with _C.device_guard(q.device):
        if out is None:
            out = torch.empty_like(q, dtype=v.dtype)
        lse = torch.empty((num_heads, total_q), dtype=torch.float, device=q.device)
        if zero_tensors:
            out.zero_()
            lse.fill_(float("-inf"))
        if total_q > 0 and batch_size > 0:
            p = _C.FgFlashParams()
            p.q, p.k_cache, p.v_cache, p.out, p.lse = q.data_ptr(), k.data_ptr(), v.data_ptr(), out.data_ptr(), lse.data_ptr()
            p.cu_seqlens_q = cu_seqlens_q.data_ptr()
            p.seqused_k = seqused_k.data_ptr()
            p.block_table = page_table.data_ptr()
            p.alibi_slopes = alibi_slopes.data_ptr() if alibi_slopes is not None else None
            p.q_row_stride, p.q_head_stride = q.stride(0), q.stride(1)
            p.o_row_stride, p.o_head_stride = out.stride(0), out.stride(1)
            p.k_page_stride, p.k_row_stride, p.k_head_stride = k.stride(0), k.stride(1), k.stride(2)
            p.v_page_stride, p.v_row_stride, p.v_head_stride = v.stride(0), v.stride(1), v.stride(2)
            p.block_table_stride = page_table.stride(0)
            p.alibi_batch_stride = alibi_batch_stride
            p.total_q = total_q
            p.batch, p.Hq, p.Hk, p.D, p.page_size = batch_size, num_heads, num_heads_k, head_size, block_size
            p.max_seqlen_q, p.max_seqlen_k = int(max_seqlen_q), int(max_seqlen_k)
            p.is_causal = 1 if is_causal else 0
            p.window_left, p.window_right = int(window_size_left), int(window_size_right)
            p.softmax_scale = float(softmax_scale)
            p.softcap = float(softcap)
            p.dtype = _C.dtype_id(q.dtype)
            # single-token queries: scratch for the partial results of split key ranges (the reference's
            # out_accum / softmax_lse_accum); the library says how much it wants, zero for prefill shapes
            ws_bytes = _C.lib().fg_flash_attn_workspace_bytes(ctypes.byref(p), q.device.index or 0)
            if ws_bytes > 0:
                ws = torch.empty(ws_bytes, dtype=torch.uint8, device=q.device)
                p.workspace, p.workspace_bytes = ws.data_ptr(), ws_bytes
            rc = _C.lib().fg_flash_attn_varlen_fwd(ctypes.byref(p), _C.current_stream(q.device))
            _C.check(rc, "fg_flash_attn_varlen_fwd")
        philox_args = torch.empty((2,), dtype=torch.int64, device=q.device)
        unused = torch.empty((), dtype=torch.int64, device=q.device)
        probs = torch.empty((), device=q.device)
    return out, q, k, v, lse, philox_args, unused, probs


def flash_attn_varlen_func(
    q,
    k,
    v,
    max_seqlen_q,
    cu_seqlens_q,
    max_seqlen_k,
    cu_seqlens_k=None,  # only used for non-paged prefill
    seqused_k=None,
    q_v=None,
    dropout_p=0.0,
    softmax_scale=None,
    causal=False,
    window_size=None,
    softcap=0.0,  # 0.0 means deactivated
    alibi_slopes=None,
    deterministic=False,
    return_attn_probs=False,
    block_table=None,
    return_softmax_lse=False,
    out=None,
    # Dummy FA3 arguments
    scheduler_metadata=None,
    q_descale=None,
    k_descale=None,
    v_descale=None,
    num_splits: int = 0,
    fa_version: int = 2,
):
    """Variable-length attention forward with FA2 semantics over a paged KV cache.

    q: (total_q, nheads, headdim); k, v: (num_pages, page_size, nheads_k, headdim);
    cu_seqlens_q: (batch + 1,) int32; seqused_k: (batch,) int32; block_table: (batch, pages) int32.
    The causal mask is aligned to the bottom right corner; GQA/MQA by head mapping
    (query head h reads KV head h // (nheads // nheads_k)); window_size = (left, right) gives
    sliding-window attention; softcap > 0 applies softcap * tanh(score / softcap); alibi_slopes
    (nheads,) or (batch, nheads) fp32 adds -slope * |i + seqlen_k - seqlen_q - j|.
    Returns out (total_q, nheads, headdim), and the fp32 log-sum-exp (nheads, total_q) as well
    when return_softmax_lse is set.  q_v, deterministic, return_attn_probs, scheduler_metadata
    and the descale arguments are accepted and ignored, as in the reference.
    """
    logger.debug("GEMS FLASH_ATTN_VARLEN_FUNC")
    assert cu_seqlens_k is not None or seqused_k is not None, "cu_seqlens_k or seqused_k must be provided"
    assert cu_seqlens_k is None or seqused_k is None, "cu_seqlens_k and seqused_k cannot be provided at the same time"
    assert block_table is None or seqused_k is not None, "seqused_k must be provided if block_table is provided"
    if softmax_scale is None:
        softmax_scale = q.shape[-1] ** (-0.5)
    if window_size is None:
        real_window_size = (-1, -1)
    else:
        assert len(window_size) == 2
        real_window_size = (window_size[0], window_size[1])
    q, k, v = [maybe_contiguous(x) for x in (q, k, v)]
    dummy_cu_seqlens_k = torch.empty_like(cu_seqlens_q)
    if fa_version != 2:
        raise RuntimeError("Only FA2 is implemented.")
    if num_splits > 0:
        raise RuntimeError("num_splits > 0 is not implemented in GEMS.")
    max_seqlen_q = max_seqlen_q.item() if hasattr(max_seqlen_q, "item") else max_seqlen_q
    max_seqlen_k = max_seqlen_k.item() if hasattr(max_seqlen_k, "item") else max_seqlen_k
    out, q, k, v, softmax_lse, *_ = mha_varlan_fwd(
        q, k, v, out, cu_seqlens_q,
        dummy_cu_seqlens_k if cu_seqlens_k is None else cu_seqlens_k,
        seqused_k, None, block_table, alibi_slopes, max_seqlen_q, max_seqlen_k, dropout_p,
        softmax_scale, False, causal, real_window_size[0], real_window_size[1], softcap,
        return_softmax_lse and dropout_p > 0, None,
    )
    return (out, softmax_lse) if return_softmax_lse else out
