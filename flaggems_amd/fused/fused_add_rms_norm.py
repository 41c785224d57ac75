"""In-place residual add + RMS norm (reference: src/flag_gems/fused/fused_add_rms_norm.py:57-82)."""
import logging
import math

from .. import _C

logger = logging.getLogger("flag_gems.fused.fused_add_rms_norm")


def fused_add_rms_norm(x, residual, normalized_shape, weight, eps=1e-5):
    """residual += x; x = rmsnorm(residual) * weight.  Both tensors are modified in place and
    returned.  As in the reference, non-contiguous arguments are made contiguous first, in which
    case the update lands in the returned copies."""
    logger.debug(
        "GEMS FUSED_ADD_RMS_NORM FORWARD, [input shape]: %s, [residual shape]: %s, [weight shape]: %s",
        x.size(), residual.size(), weight.size(),
    )
    dim = x.ndim - len(normalized_shape)
    M = math.prod(x.shape[:dim])
    N = math.prod(normalized_shape)
    assert x.shape == residual.shape, "x and residual must have the same shape"
    assert x.dtype == residual.dtype == weight.dtype, "x, residual and weight must share a dtype"
    x = x.contiguous()
    residual = residual.contiguous()
    weight = weight.contiguous()
    if M == 0 or N == 0:
        return x, residual
    with _C.device_guard(x.device):
        rc = _C.lib().fg_fused_add_rms_norm(
            x.data_ptr(), residual.data_ptr(), weight.data_ptr(), M, N, N, N, eps,
            _C.dtype_id(x.dtype), _C.current_stream(x.device),
        )
    _C.check(rc, "fg_fused_add_rms_norm")
    return x, residual
