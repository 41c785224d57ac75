"""aten::rms_norm on the gfx950 kernels, forward and backward
(reference: src/flag_gems/ops/rms_norm.py:149-222)."""
import logging
import math

import torch

from .. import _C

logger = logging.getLogger("flag_gems.ops.rms_norm")

def _composite(x, normalized_shape, weight, eps):
    # plain tensor math: used when the dtype has no kernel
    dims = tuple(range(x.ndim - len(normalized_shape), x.ndim))
    if eps is None:
        eps = torch.finfo(x.dtype).eps
    xf = x.float() if x.dtype in (torch.float16, torch.bfloat16) else x
    y = xf * torch.rsqrt(xf.pow(2).mean(dim=dims, keepdim=True) + eps)
    if weight is not None:
        y = y * weight
    return y.to(x.dtype)


def _forward(x, normalized_shape, weight, eps, want_inv_rms):
    """(y, inv_rms or None, x as the kernel read it): one launch."""
    dim = x.ndim - len(normalized_shape)
    assert tuple(x.shape[dim:]) == normalized_shape, "normalized_shape does not match the trailing dims of x"
    M = math.prod(x.shape[:dim])
    N = math.prod(normalized_shape)
    x = x.contiguous()
    w = weight.contiguous() if weight is not None else None
    y = torch.empty_like(x)
    inv_rms = torch.empty((M,), device=x.device, dtype=torch.float32) if want_inv_rms else None
    if M == 0 or N == 0:
        return y, inv_rms, x
    with _C.device_guard(x.device):
        rc = _C.lib().fg_rms_norm(
            x.data_ptr(), w.data_ptr() if w is not None else None, y.data_ptr(),
            inv_rms.data_ptr() if inv_rms is not None else None,
            M, N, N, N, eps, _C.dtype_id(x.dtype), _C.current_stream(x.device),
        )
    _C.check(rc, "fg_rms_norm")
    return y, inv_rms, x


class RmsNorm(torch.autograd.Function):
    """Forward saves x and the per-row 1/rms; backward is one kernel that writes dx and, when the weight needs
    a gradient, fp32 partial column sums (one row per group of rows) that a second small kernel adds up (the reference
    uses a kernel per gradient, src/flag_gems/ops/rms_norm.py:149-218)."""

    @staticmethod
    def forward(ctx, x, normalized_shape, weight, eps):
        logger.debug("GEMS LAYERNORM FORWARD")
        y, inv_rms, xc = _forward(x, normalized_shape, weight, eps, True)
        ctx.save_for_backward(xc, inv_rms, weight)
        ctx.normalized_shape = normalized_shape
        return y

    @staticmethod
    def backward(ctx, dy):
        logger.debug("GEMS LAYERNORM BACKWARD")
        x, inv_rms, weight = ctx.saved_tensors
        normalized_shape = ctx.normalized_shape
        dim = x.ndim - len(normalized_shape)
        M = math.prod(x.shape[:dim])
        N = math.prod(normalized_shape)
        dy = dy.contiguous()
        if dy.dtype != x.dtype:
            dy = dy.to(x.dtype)
        w = weight.contiguous() if weight is not None else None
        dx = torch.empty_like(x)
        want_dw = weight is not None and ctx.needs_input_grad[2]
        if M == 0 or N == 0:
            return dx, None, (torch.zeros_like(weight) if want_dw else None), None
        partial, partial_rows = None, 0
        lib = _C.lib()
        if want_dw:
            partial_rows = lib.fg_rms_norm_backward_partial_rows(M, N, _C.dtype_id(x.dtype), x.device.index or 0)
            partial = torch.empty((partial_rows, N), dtype=torch.float32, device=x.device)
        with _C.device_guard(x.device):
            rc = lib.fg_rms_norm_backward(
                x.data_ptr(), dy.data_ptr(), inv_rms.data_ptr(), w.data_ptr() if w is not None else None,
                dx.data_ptr(), partial.data_ptr() if partial is not None else None, partial_rows,
                M, N, _C.dtype_id(x.dtype), _C.current_stream(x.device),
            )
            _C.check(rc, "fg_rms_norm_backward")
            dw = None
            if want_dw:
                # added up in fp32 and rounded once (the reference rounds the partial rows to x.dtype first)
                dw = torch.empty(weight.shape, dtype=x.dtype, device=x.device)
                rc = lib.fg_rms_norm_backward_dw(
                    partial.data_ptr(), partial_rows, N, dw.data_ptr(), _C.dtype_id(x.dtype), _C.current_stream(x.device)
                )
                _C.check(rc, "fg_rms_norm_backward_dw")
        return dx, None, dw, None


def rms_norm(x, normalized_shape, weight=None, eps=1e-5):
    """y = x * rsqrt(mean(x^2 over normalized_shape) + eps) * weight.

    `weight=None` (ones) and `eps=None` (machine epsilon of x.dtype) follow the ATen schema.  When
    autograd needs a graph through this call it goes through RmsNorm (kernels for both directions);
    otherwise the forward kernel alone runs.
    """
    normalized_shape = tuple(normalized_shape)
    if not _C.supported_dtype(x.dtype) or (weight is not None and weight.dtype != x.dtype):
        logger.debug("GEMS LAYERNORM FORWARD")
        return _composite(x, normalized_shape, weight, eps)
    if eps is None:
        eps = torch.finfo(x.dtype).eps
    needs_grad = torch.is_grad_enabled() and (
        x.requires_grad or (weight is not None and weight.requires_grad)
    )
    if needs_grad:
        return RmsNorm.apply(x, normalized_shape, weight, eps)
    logger.debug("GEMS LAYERNORM FORWARD")
    return _forward(x, normalized_shape, weight, eps, False)[0]
