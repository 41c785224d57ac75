"""aten::mm / aten::mm.out on the gfx950 MFMA GEMM (reference: src/flag_gems/ops/mm.py:137-237)."""
import logging

import torch

from .. import _C
from ._gemm import gemm, get_higher_dtype  # noqa: F401

logger = logging.getLogger("flag_gems.ops.mm")


def _prepare(a, b):
    # same contiguity rule as the reference: copy only when both strides exceed one
    sa0, sa1 = a.stride()
    sb0, sb1 = b.stride()
    if sa0 > 1 and sa1 > 1:
        a = a.contiguous()
    if sb0 > 1 and sb1 > 1:
        b = b.contiguous()
    assert a.shape[1] == b.shape[0], "incompatible dimensions"
    if sa1 == 1:
        return a, b  # A is contiguous along K already (the usual case): nothing below applies
    # A column-major A (the X^T of a weight gradient) misses the direct-to-LDS and skinny kernels, which want
    # A contiguous along K; one transposing copy of A (the library's own kernel) costs far less than the
    # slower main loop once the output is 256 columns wide, or 64 when A has few rows.  Measured, bf16:
    # 4096^3 209 -> 127 us, 65 x 4096 x 4096 195 -> 29 us, 16384 x 4096 x 11008 1954 -> 1393 us.
    wide = b.shape[1] >= 256 or (b.shape[1] >= 64 and a.shape[0] <= 1024)
    if (a.stride(0) == 1 and a.stride(1) > 1 and a.shape[0] > 1 and wide and a.is_cuda
            and a.element_size() in (2, 4) and _C.supported_dtype(a.dtype)):
        a = _transposed_copy(a)
    return a, b


def _transposed_copy(a):
    """Row-major copy of a column-major [M, K] matrix (memory [K, M]) with the library's transpose kernel."""
    M, K = a.shape
    out = torch.empty((M, K), dtype=a.dtype, device=a.device)
    with _C.device_guard(a.device):
        rc = _C.lib().fg_transpose2d(a.data_ptr(), out.data_ptr(), K, M, a.stride(1), K, a.element_size(),
                                     _C.current_stream(a.device))
    _C.check(rc, "fg_transpose2d")
    return out


def _kernel_covers(a, b):
    return a.dim() == 2 and b.dim() == 2 and _C.supported_dtype(a.dtype) and _C.supported_dtype(b.dtype)


def _vendor_mm(a, b, out=None):
    # bmm.out is a separate ATen kernel that is never overridden, so this cannot re-enter
    r = torch.empty((1, a.shape[0], b.shape[1]), dtype=torch.result_type(a, b), device=a.device)
    r = torch.ops.aten.bmm.out(a.unsqueeze(0), b.unsqueeze(0), out=r).squeeze(0)
    if out is None:
        return r
    out.copy_(r)
    return out


def _run(a, b, c):
    M, K = a.shape
    N = b.shape[1]
    if logger.isEnabledFor(logging.DEBUG):
        logger.debug(
            "GEMS MM, [shape info]: [-, %s, %s, %s](batch, M, N, K), [A column-major]: %s, [B column-major]: %s",
            M, N, K, a.stride(0) == 1, b.stride(0) == 1,
        )
    if M == 0 or N == 0:
        return c
    if K == 0:
        return c.zero_()
    if a.dtype != b.dtype:
        # the reference casts inside the kernel to the higher of the two dtypes
        hi = get_higher_dtype(a.dtype, b.dtype)
        a, b = a.to(hi), b.to(hi)
    return gemm(a, b, None, c, 1.0, 0.0)


def mm(a, b):
    if not _kernel_covers(a, b):
        return _vendor_mm(a, b)
    a, b = _prepare(a, b)
    M, _ = a.shape
    N = b.shape[1]
    c = torch.empty((M, N), device=a.device, dtype=get_higher_dtype(a.dtype, b.dtype))
    return _run(a, b, c)


def mm_out(a, b, *, out):
    if not _kernel_covers(a, b) or not _C.supported_dtype(out.dtype):
        return _vendor_mm(a, b, out)
    a, b = _prepare(a, b)
    assert out.shape == (a.shape[0], b.shape[1]), "incompatible output shape"
    return _run(a, b, out)
