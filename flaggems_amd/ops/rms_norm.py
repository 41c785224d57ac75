"""aten::rms_norm forward on the gfx950 kernel (reference: src/flag_gems/ops/rms_norm.py:149-222)."""
import logging
import math

import torch

from .. import _C

logger = logging.getLogger("flag_gems.ops.rms_norm")


def _composite(x, normalized_shape, weight, eps):
    # plain tensor math: used when autograd must see the computation or the dtype has no kernel
    dims = tuple(range(x.ndim - len(normalized_shape), x.ndim))
    if eps is None:
        eps = torch.finfo(x.dtype).eps
    xf = x.float() if x.dtype in (torch.float16, torch.bfloat16) else x
    y = xf * torch.rsqrt(xf.pow(2).mean(dim=dims, keepdim=True) + eps)
    if weight is not None:
        y = y * weight
    return y.to(x.dtype)


def rms_norm(x, normalized_shape, weight=None, eps=1e-5):
    """y = x * rsqrt(mean(x^2 over normalized_shape) + eps) * weight.

    `weight=None` (ones) and `eps=None` (machine epsilon of x.dtype) follow the ATen schema.  The
    kernel is forward-only: when autograd needs a graph through this call the composite tensor
    formula is used instead, which autograd differentiates by itself.
    """
    logger.debug("GEMS LAYERNORM FORWARD")
    normalized_shape = tuple(normalized_shape)
    needs_grad = torch.is_grad_enabled() and (
        x.requires_grad or (weight is not None and weight.requires_grad)
    )
    if needs_grad or not _C.supported_dtype(x.dtype) or (weight is not None and weight.dtype != x.dtype):
        return _composite(x, normalized_shape, weight, eps)
    if eps is None:
        eps = torch.finfo(x.dtype).eps
    dim = x.ndim - len(normalized_shape)
    assert tuple(x.shape[dim:]) == normalized_shape, "normalized_shape does not match the trailing dims of x"
    M = math.prod(x.shape[:dim])
    N = math.prod(normalized_shape)
    x = x.contiguous()
    w = weight.contiguous() if weight is not None else None
    y = torch.empty_like(x)
    if M == 0 or N == 0:
        return y
    with _C.device_guard(x.device):
        rc = _C.lib().fg_rms_norm(
            x.data_ptr(), w.data_ptr() if w is not None else None, y.data_ptr(), None,
            M, N, N, N, eps, _C.dtype_id(x.dtype), _C.current_stream(x.device),
        )
    _C.check(rc, "fg_rms_norm")
    return y
