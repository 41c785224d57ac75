"""aten::_softmax and aten::_softmax_backward_data on the gfx950 kernels
(reference: src/flag_gems/ops/softmax.py:283-355)."""
import logging

import torch

from .. import _C

logger = logging.getLogger("flag_gems.ops.softmax")


def softmax(self, dim, half_to_float=False):
    logger.debug("GEMS SOFTMAX")
    assert dim >= -self.ndim and dim < self.ndim, "Invalid dim"
    if not _C.supported_dtype(self.dtype):
        # the .out overload is a separate ATen kernel that stays on the vendor library
        out = torch.empty_like(self, memory_format=torch.contiguous_format)
        return torch.ops.aten._softmax.out(self, dim, half_to_float, out=out)
    dim = dim % self.ndim
    M = 1
    N = self.shape[dim]
    for i in range(dim):
        M *= self.shape[i]
    self = self.contiguous()
    dtype = torch.float32 if half_to_float else self.dtype
    out = torch.empty_like(self, dtype=dtype)
    if self.numel() == 0:
        return out
    K = self.numel() // M // N
    with _C.device_guard(self.device):
        rc = _C.lib().fg_softmax(
            self.data_ptr(), out.data_ptr(), M, N, K, _C.dtype_id(self.dtype), _C.dtype_id(dtype),
            _C.current_stream(self.device),
        )
    _C.check(rc, "fg_softmax")
    return out


def _backward(name, out_kw, entry, grad_output, output, dim, input_dtype):
    """Shared host half of the softmax / log_softmax backward: grad_input from (grad_output, output)."""
    assert dim >= -output.ndim and dim < output.ndim, "Invalid dim"
    covered = (
        _C.supported_dtype(output.dtype) and grad_output.dtype == output.dtype
        and (input_dtype == output.dtype or (output.dtype == torch.float32 and _C.supported_dtype(input_dtype)))
    )
    if not covered:
        # the .out overload is a separate ATen kernel that stays on the vendor library
        in_grad = torch.empty_like(output, dtype=input_dtype, memory_format=torch.contiguous_format)
        return getattr(torch.ops.aten, name).out(grad_output, output, dim, input_dtype, **{out_kw: in_grad})
    dim = dim % output.ndim
    M = 1
    N = output.shape[dim]
    for i in range(dim):
        M *= output.shape[i]
    output = output.contiguous()
    grad_output = grad_output.contiguous()
    in_grad = torch.empty_like(output, dtype=input_dtype)
    if output.numel() == 0:
        return in_grad
    K = output.numel() // M // N
    with _C.device_guard(output.device):
        rc = getattr(_C.lib(), entry)(
            output.data_ptr(), grad_output.data_ptr(), in_grad.data_ptr(), M, N, K, _C.dtype_id(output.dtype),
            _C.dtype_id(input_dtype), _C.current_stream(output.device),
        )
    _C.check(rc, entry)
    return in_grad


def softmax_backward(grad_output, output, dim, input_dtype):
    logger.debug("GEMS SOFTMAX VJP")
    return _backward("_softmax_backward_data", "grad_input", "fg_softmax_backward", grad_output, output, dim, input_dtype)
