"""aten::_log_softmax and aten::_log_softmax_backward_data on the gfx950 kernels
(reference: src/flag_gems/ops/log_softmax.py:98-160)."""
import logging

import torch

from .. import _C
from .softmax import _backward

logger = logging.getLogger("flag_gems.ops.log_softmax")


def log_softmax(self, dim, half_to_float=False):
    logger.debug("GEMS LOG_SOFTMAX")
    assert dim >= -self.ndim and dim < self.ndim, "Invalid dim"
    if not _C.supported_dtype(self.dtype):
        # the .out overload is a separate ATen kernel that stays on the vendor library
        out = torch.empty_like(self, memory_format=torch.contiguous_format)
        return torch.ops.aten._log_softmax.out(self, dim, half_to_float, out=out)
    dim = dim % self.ndim
    M = 1
    N = self.shape[dim]
    for i in range(dim):
        M *= self.shape[i]
    inp = self.contiguous()
    dtype = torch.float32 if half_to_float else self.dtype
    out = torch.empty_like(inp, dtype=dtype)
    if inp.numel() == 0:
        return out
    K = inp.numel() // M // N
    with _C.device_guard(inp.device):
        rc = _C.lib().fg_log_softmax(
            inp.data_ptr(), out.data_ptr(), M, N, K, _C.dtype_id(inp.dtype), _C.dtype_id(dtype),
            _C.current_stream(inp.device),
        )
    _C.check(rc, "fg_log_softmax")
    return out


def log_softmax_backward(grad_output, output, dim, input_dtype):
    logger.debug("GEMS LOG_SOFTMAX VJP")
    return _backward("_log_softmax_backward_data", "out", "fg_log_softmax_backward", grad_output, output, dim, input_dtype)
