"""silu(A) * B (reference: src/flag_gems/fused/silu_and_mul.py:12-53)."""
import logging

import torch

from .. import _C

logger = logging.getLogger("flag_gems.fused.silu_and_mul")


def _rows_view(t):
    """(rows, cols, row_stride) when t is a stack of unit-stride rows with one uniform row stride
    (contiguous tensors, and the halves of a gate-up projection, qualify); otherwise None."""
    if t.ndim == 2:  # the usual case, spelled out: one stride() call instead of a walk over the dims
        row_stride, col_stride = t.stride()
        rows, cols = t.shape
        if (col_stride == 1 or cols == 1) and row_stride >= cols:
            return rows, cols, row_stride
        return None
    if t.ndim == 0:
        return 1, 1, 1
    if t.stride(-1) != 1 and t.shape[-1] != 1:
        return None
    cols = t.shape[-1]
    if t.ndim == 1:
        return 1, cols, cols
    row_stride = t.stride(-2)
    expect = row_stride * t.shape[-2]
    for d in range(t.ndim - 3, -1, -1):  # leading dims must collapse onto the row stride
        if t.shape[d] != 1 and t.stride(d) != expect:
            return None
        expect *= t.shape[d]
    if row_stride < cols:
        return None
    rows = t.numel() // cols if cols else 0
    return rows, cols, row_stride


def _launch(A, B, out):
    va, vb, vo = _rows_view(A), _rows_view(B), _rows_view(out)
    if va is None:
        A = A.contiguous()
        va = _rows_view(A)
    if vb is None:
        B = B.contiguous()
        vb = _rows_view(B)
    assert vo is not None, "silu_and_mul: out must be made of unit-stride rows"
    rows, cols, _ = vo
    if rows * cols == 0:
        return out
    with _C.device_guard(out.device):
        rc = _C.lib().fg_silu_and_mul(
            A.data_ptr(), B.data_ptr(), out.data_ptr(), rows, cols, va[2], vb[2], vo[2],
            _C.dtype_id(out.dtype), _C.current_stream(out.device),
        )
    _C.check(rc, "fg_silu_and_mul")
    return out


def silu_and_mul(A, B):
    logger.debug("GEMS SILU AND MUL FORWARD")
    if A.shape != B.shape:
        A, B = torch.broadcast_tensors(A, B)
    dtype = torch.promote_types(A.dtype, B.dtype)
    if A.dtype != dtype:
        A = A.to(dtype)
    if B.dtype != dtype:
        B = B.to(dtype)
    if not _C.supported_dtype(dtype):
        return torch.nn.functional.silu(A) * B
    out = torch.empty(A.shape, dtype=dtype, device=A.device)
    return _launch(A, B, out)


def silu_and_mul_out(A, B, out):
    assert A.shape == B.shape == out.shape, "silu_and_mul_out: shapes must match"
    assert A.dtype == B.dtype == out.dtype, "silu_and_mul_out: dtypes must match"
    _launch(A, B, out)
    return out
