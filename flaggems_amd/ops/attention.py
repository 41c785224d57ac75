"""flash_attn_varlen_func over a paged KV cache on the gfx950 attention kernel, and the dense
entry points (flash_attention_forward / scaled_dot_product_attention) mapped onto the same kernel.

API shims: src/flag_gems/ops/attention.py:1118-1287 (varlen), :1028-1110 (flash_attention_forward),
:749-769 (scaled_dot_product_attention).  Host checks and parameter preparation: mha_varlan_fwd and
mha_fwd, src/flag_gems/ops/flash_api.py:230-569 and :26-227.
"""
import ctypes
import logging

import torch

from .. import _C

logger = logging.getLogger("flag_gems.ops.attention")


def maybe_contiguous(x):
    return x.contiguous() if x is not None and x.stride(-1) != 1 else x


# The reference's forward returns three tensors that only dropout gives a meaning (philox state, an unused slot, the
# attention probabilities).  Dropout is not part of this path, so they are placeholders: made once per device and
# handed out again, instead of three allocations on every call.
_placeholders = {}


def _dropout_placeholders(device):
    hit = _placeholders.get(device)
    if hit is None:
        hit = _placeholders[device] = (torch.empty((2,), dtype=torch.int64, device=device),
                                       torch.empty((), dtype=torch.int64, device=device),
                                       torch.empty((), device=device))
    return hit


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
            p.q_row_stride, p.q_head_stride, _ = q.stride()
            p.o_row_stride, p.o_head_stride, _ = out.stride()
            p.k_page_stride, p.k_row_stride, p.k_head_stride, _ = k.stride()
            p.v_page_stride, p.v_row_stride, p.v_head_stride, _ = v.stride()
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
        philox_args, unused, probs = _dropout_placeholders(q.device)
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
    q, k, v = maybe_contiguous(q), maybe_contiguous(k), maybe_contiguous(v)
    if fa_version != 2:
        raise RuntimeError("Only FA2 is implemented.")
    if num_splits > 0:
        raise RuntimeError("num_splits > 0 is not implemented in GEMS.")
    max_seqlen_q = max_seqlen_q.item() if hasattr(max_seqlen_q, "item") else max_seqlen_q
    max_seqlen_k = max_seqlen_k.item() if hasattr(max_seqlen_k, "item") else max_seqlen_k
    out, q, k, v, softmax_lse, *_ = mha_varlan_fwd(
        q, k, v, out, cu_seqlens_q,
        # (the reference passes an uninitialised tensor shaped like cu_seqlens_q here; only its shape and dtype are
        # looked at, so cu_seqlens_q itself serves without an allocation)
        cu_seqlens_q if cu_seqlens_k is None else cu_seqlens_k,
        seqused_k, None, block_table, alibi_slopes, max_seqlen_q, max_seqlen_k, dropout_p,
        softmax_scale, False, causal, real_window_size[0], real_window_size[1], softcap,
        return_softmax_lse and dropout_p > 0, None,
    )
    return (out, softmax_lse) if return_softmax_lse else out


# ---- dense attention on the paged kernel ---------------------------------------------------------------
# A dense K (batch, seqlen_k, heads_k, head_dim) with arbitrary batch / row / head strides IS a paged cache:
# cut every sequence into virtual pages of `page` consecutive rows; page j of sequence b is page number
# b * pages_per_batch_stride + j of a cache whose page stride is page * row_stride.  No byte is copied; the
# kernel never reads a key row at or past seqlen_k, so a last, partial page is fine.  The page size is the
# largest power of two (16..256) that divides the batch stride measured in rows; when there is none
# (a sequence length like 1030) the whole sequence is one page, which the general kernel handles.
_dense_meta = {}


def _page_rows(k, batch):
    """Virtual page size for a dense K, or None when the batch stride is not a whole number of pages."""
    if batch == 1:
        return 64  # no batch stride to respect
    row_stride, batch_stride = k.stride(1), k.stride(0)
    if row_stride <= 0 or batch_stride % row_stride != 0:
        return None
    rows = batch_stride // row_stride
    for page in (256, 128, 64, 32, 16):
        if rows % page == 0:
            return page
    return None


def _dense_tables(device, batch, seqlen_q, seqlen_k, page, pages_per_batch):
    """cu_seqlens_q, seqused_k and the virtual block table of a dense batch (cached per shape)."""
    key = (device.index, batch, seqlen_q, seqlen_k, page, pages_per_batch)
    hit = _dense_meta.get(key)
    if hit is None:
        if len(_dense_meta) > 256:
            _dense_meta.clear()
        cu = torch.arange(batch + 1, dtype=torch.int32, device=device) * seqlen_q
        used = torch.full((batch,), seqlen_k, dtype=torch.int32, device=device)
        npages = max(1, (seqlen_k + page - 1) // page)
        table = (torch.arange(batch, dtype=torch.int32, device=device)[:, None] * pages_per_batch
                 + torch.arange(npages, dtype=torch.int32, device=device)[None, :]).contiguous()
        hit = (cu, used, table)
        _dense_meta[key] = hit
    return hit


def mha_fwd(q, k, v, out, alibi_slopes, p_dropout, softmax_scale, is_causal, window_size_left, window_size_right,
            softcap, return_softmax, disable_splitkv=False):
    """Dense forward, q (batch, seqlen_q, heads, d), k / v (batch, seqlen_k, heads_k, d), any strides with a
    contiguous last dimension (reference: mha_fwd, src/flag_gems/ops/flash_api.py:26-227).  Returns
    (out, q, k, v, lse (batch, heads, seqlen_q) fp32, philox_seed, philox_offset, p) with placeholders for the
    dropout outputs."""
    assert q.is_cuda and k.is_cuda and v.is_cuda
    assert q.dtype in (torch.float16, torch.bfloat16), "FlashAttention only support fp16 and bf16 data type"
    assert q.dtype == k.dtype and q.dtype == v.dtype
    assert q.stride(-1) == 1 and k.stride(-1) == 1 and v.stride(-1) == 1, "Input tensor must have contiguous last dimension"
    batch, seqlen_q, num_heads, head_size = q.shape
    seqlen_k, num_heads_k = k.shape[1], k.shape[2]
    assert k.shape == (batch, seqlen_k, num_heads_k, head_size) and v.shape == k.shape
    assert head_size <= 256 and head_size % 8 == 0, "head dimension must be a multiple of 8 and at most 256"
    assert num_heads % num_heads_k == 0, "Number of heads in key/value must divide number of heads in query"
    assert p_dropout == 0, "dropout is not implemented on this path (inference only)"
    assert not return_softmax, "return_softmax needs dropout, which is not implemented"
    if seqlen_q == 1 and alibi_slopes is None:
        is_causal = False
    if is_causal:
        window_size_right = 0
    if window_size_left >= seqlen_k:
        window_size_left = -1
    if window_size_right >= seqlen_k:
        window_size_right = -1
    if alibi_slopes is not None:
        assert alibi_slopes.dtype == torch.float and alibi_slopes.stride(-1) == 1
        assert alibi_slopes.shape == (num_heads,) or alibi_slopes.shape == (batch, num_heads)
    with _C.device_guard(q.device):
        # rows of q must be equally spaced over the whole batch (row b * seqlen_q + s)
        if batch > 1 and q.stride(0) != seqlen_q * q.stride(1):
            q = q.contiguous()
        # K and V share one virtual block table, so they must share their strides
        if k.stride() != v.stride():
            k, v = k.contiguous(), v.contiguous()
        page = _page_rows(k, batch)
        if page is None:
            page, pages_per_batch, page_stride = max(seqlen_k, 1), 1, k.stride(0)  # one page per sequence
        else:
            pages_per_batch = k.stride(0) // (page * k.stride(1)) if batch > 1 else 0
            page_stride = page * k.stride(1)
        cu, used, table = _dense_tables(q.device, batch, seqlen_q, seqlen_k, page, pages_per_batch)
        if out is None:
            out = torch.empty((batch, seqlen_q, num_heads, head_size), dtype=q.dtype, device=q.device)
        else:
            assert out.shape == (batch, seqlen_q, num_heads, head_size) and out.dtype == q.dtype and out.stride(-1) == 1
            assert batch == 1 or out.stride(0) == seqlen_q * out.stride(1), "out rows must be equally spaced over the batch"
        total_q = batch * seqlen_q
        lse = torch.empty((num_heads, total_q), dtype=torch.float, device=q.device)
        if total_q > 0 and seqlen_k >= 0:
            p = _C.FgFlashParams()
            p.q, p.k_cache, p.v_cache, p.out, p.lse = q.data_ptr(), k.data_ptr(), v.data_ptr(), out.data_ptr(), lse.data_ptr()
            p.cu_seqlens_q, p.seqused_k, p.block_table = cu.data_ptr(), used.data_ptr(), table.data_ptr()
            p.alibi_slopes = alibi_slopes.data_ptr() if alibi_slopes is not None else None
            p.q_row_stride, p.q_head_stride = q.stride(1), q.stride(2)
            p.o_row_stride, p.o_head_stride = out.stride(1), out.stride(2)
            p.k_page_stride, p.k_row_stride, p.k_head_stride = page_stride, k.stride(1), k.stride(2)
            p.v_page_stride, p.v_row_stride, p.v_head_stride = page_stride, v.stride(1), v.stride(2)
            p.block_table_stride = table.stride(0)
            p.alibi_batch_stride = alibi_slopes.stride(0) if alibi_slopes is not None and alibi_slopes.ndim == 2 else 0
            p.total_q = total_q
            p.batch, p.Hq, p.Hk, p.D, p.page_size = batch, num_heads, num_heads_k, head_size, page
            p.max_seqlen_q, p.max_seqlen_k = seqlen_q, seqlen_k
            p.is_causal = 1 if is_causal else 0
            p.window_left, p.window_right = int(window_size_left), int(window_size_right)
            p.softmax_scale = float(softmax_scale)
            p.softcap = float(softcap)
            p.dtype = _C.dtype_id(q.dtype)
            ws_bytes = _C.lib().fg_flash_attn_workspace_bytes(ctypes.byref(p), q.device.index or 0)
            if ws_bytes > 0:
                ws = torch.empty(ws_bytes, dtype=torch.uint8, device=q.device)
                p.workspace, p.workspace_bytes = ws.data_ptr(), ws_bytes
            rc = _C.lib().fg_flash_attn_varlen_fwd(ctypes.byref(p), _C.current_stream(q.device))
            _C.check(rc, "fg_flash_attn_varlen_fwd")
        philox_seed = torch.empty((), dtype=torch.int64, device=q.device)
        philox_offset = torch.empty((), dtype=torch.int64, device=q.device)
        probs = torch.empty((), device=q.device)
    return out, q, k, v, lse.view(num_heads, batch, seqlen_q).permute(1, 0, 2), philox_seed, philox_offset, probs


def flash_attention_forward(
    query, key, value, cumulative_sequence_length_q, cumulative_sequence_length_k, max_q, max_k, dropout_p, is_causal,
    return_debug_mask, *, scale=None, softcap=0.0, window_size_left=None, window_size_right=None, seqused_k=None,
    alibi_slopes=None, disable_splitkv=False,
):
    """aten::_flash_attention_forward for dense batches: query (batch, seqlen_q, heads, d), key / value
    (batch, seqlen_k, heads_k, d); FA2 semantics (causal mask aligned to the bottom right corner).
    Returns (out, lse (batch, heads, seqlen_q), philox_seed, philox_offset, debug_mask)."""
    logger.debug("GEMS FLASH_ATTENTION_FORWARD")
    assert cumulative_sequence_length_q is None and cumulative_sequence_length_k is None, "varlen is not supported yet."
    head_dim_q, head_dim_k, head_dim_v = query.shape[-1], key.shape[-1], value.shape[-1]
    assert head_dim_q == head_dim_k and head_dim_k == head_dim_v
    assert head_dim_k in {16, 32, 64, 96, 128, 192, 256}
    softmax_scale = scale or 1.0 / (head_dim_k ** 0.5)
    left = window_size_left if window_size_left is not None else -1
    right = window_size_right if window_size_right is not None else -1
    out, _, _, _, lse, philox_seed, philox_offset, p = mha_fwd(
        query, key, value, None, alibi_slopes, dropout_p, softmax_scale, is_causal, left, right, softcap,
        return_debug_mask, disable_splitkv=disable_splitkv,
    )
    return out, lse, philox_seed, philox_offset, p


def scaled_dot_product_attention(query, key, value, attn_mask=None, dropout_p=0.0, is_causal=False, scale=None,
                                 enable_gqa=False):
    """torch.nn.functional.scaled_dot_product_attention for (batch, heads, seqlen, d) inputs, forward only.
    Calls with an attention mask, with inputs that require a gradient, or causal with seqlen_q != seqlen_k (where
    torch aligns the mask to the top left corner) go to torch's own implementation."""
    logger.debug("GEMS SCALED DOT PRODUCT ATTENTION")
    head_dim_q, head_dim_k, head_dim_v = query.shape[-1], key.shape[-1], value.shape[-1]
    assert head_dim_q == head_dim_k and head_dim_k == head_dim_v
    assert dropout_p == 0.0, "Currenty only support dropout_p=0.0"
    q_heads, kv_heads = query.shape[1], key.shape[1]
    assert enable_gqa or q_heads == kv_heads, (
        f"q_head_num {q_heads} != kv_head_num {kv_heads}, enable_gqa must be True to support different head numbers."
    )
    needs_grad = torch.is_grad_enabled() and (query.requires_grad or key.requires_grad or value.requires_grad)
    covered = (
        query.dim() == 4 and attn_mask is None and not needs_grad and query.dtype in (torch.float16, torch.bfloat16)
        and head_dim_k % 8 == 0 and head_dim_k <= 256 and (not is_causal or query.shape[2] == key.shape[2])
        and query.is_cuda
    )
    if not covered:
        return torch.nn.functional.scaled_dot_product_attention(
            query, key, value, attn_mask=attn_mask, dropout_p=dropout_p, is_causal=is_causal, scale=scale,
            enable_gqa=enable_gqa,
        )
    sm_scale = scale if scale is not None else 1.0 / (head_dim_k ** 0.5)
    q, k, v = (maybe_contiguous(x).transpose(1, 2) for x in (query, key, value))
    out, *_ = mha_fwd(q, k, v, None, None, 0.0, sm_scale, is_causal, -1, -1, 0.0, False)
    return out.transpose(1, 2)
