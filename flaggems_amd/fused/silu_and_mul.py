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


_FG_ERR_UNSUPPORTED = -2
_grad_kernel_built = None   # whether the loaded library holds the gradient kernel; learnt from its first answer


def _grads(A, B, grad):
    """(grad_A, grad_B) of silu(A) * B.  The library's kernel where the build holds it; a build without it answers
    FG_ERR_UNSUPPORTED once, and from then on the vendor's elementwise kernels do the arithmetic (fp32, as the
    reference's silu_and_mul_grad_kernel, src/flag_gems/fused/silu_and_mul.py:20-31)."""
    global _grad_kernel_built
    if _grad_kernel_built is not False and grad.numel() > 0:
        va, vb = _rows_view(A), _rows_view(B)
        if va is None:
            A = A.contiguous()
            va = _rows_view(A)
        if vb is None:
            B = B.contiguous()
            vb = _rows_view(B)
        vg = _rows_view(grad)
        if vg is None:
            grad = grad.contiguous()
            vg = _rows_view(grad)
        dA, dB = torch.empty(A.shape, dtype=A.dtype, device=A.device), torch.empty(A.shape, dtype=A.dtype, device=A.device)
        vo = _rows_view(dA)
        rows, cols, _ = vo
        with _C.device_guard(A.device):
            rc = _C.lib().fg_silu_and_mul_backward(
                A.data_ptr(), B.data_ptr(), grad.data_ptr(), dA.data_ptr(), dB.data_ptr(), rows, cols,
                va[2], vb[2], vg[2], vo[2], vo[2], _C.dtype_id(A.dtype), _C.current_stream(A.device),
            )
        if rc == 0:
            _grad_kernel_built = True
            return dA, dB
        if rc != _FG_ERR_UNSUPPORTED or _grad_kernel_built:
            _C.check(rc, "fg_silu_and_mul_backward")
        _grad_kernel_built = False
    x, y, g = A.float(), B.float(), grad.float()
    sig = torch.sigmoid(x)
    return (sig * (1.0 + x * (1.0 - sig)) * g * y).to(A.dtype), (g * (x * sig)).to(A.dtype)


class SiluAndMul(torch.autograd.Function):
    """silu(A) * B with its gradient (reference: class SiluAndMul, src/flag_gems/fused/silu_and_mul.py:34-44)."""

    @staticmethod
    def forward(ctx, A, B):
        ctx.save_for_backward(A, B)
        return _launch(A, B, torch.empty(A.shape, dtype=A.dtype, device=A.device))

    @staticmethod
    def backward(ctx, grad_output):
        A, B = ctx.saved_tensors
        logger.debug("GEMS SILU AND MUL BACKWARD")
        return _grads(A, B, grad_output.to(A.dtype))


def silu_and_mul(A, B):
    logger.debug("GEMS SILU AND MUL FORWARD")
    # broadcasting and type promotion stay outside the autograd function, as differentiable torch operations: the
    # function itself then sees two tensors of one shape and dtype, and so do its gradients
    if A.shape != B.shape:
        A, B = torch.broadcast_tensors(A, B)
    dtype = torch.promote_types(A.dtype, B.dtype)
    if A.dtype != dtype:
        A = A.to(dtype)
    if B.dtype != dtype:
        B = B.to(dtype)
    if not _C.supported_dtype(dtype):
        return torch.nn.functional.silu(A) * B
    if torch.is_grad_enabled() and (A.requires_grad or B.requires_grad):
        return SiluAndMul.apply(A, B)
    return _launch(A, B, torch.empty(A.shape, dtype=dtype, device=A.device))


def silu_and_mul_out(A, B, out):
    assert A.shape == B.shape == out.shape, "silu_and_mul_out: shapes must match"
    assert A.dtype == B.dtype == out.dtype, "silu_and_mul_out: dtypes must match"
    _launch(A, B, out)
    return out
