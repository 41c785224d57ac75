"""aten::addmm / aten::addmm.out (reference: src/flag_gems/ops/addmm.py:83-181)."""
import logging

import torch

from .. import _C
from ._gemm import gemm, get_higher_dtype

logger = logging.getLogger("flag_gems.ops.addmm")


def broadcastable_to(s1, s2):
    """True when shape s1 broadcasts to shape s2
    (semantics of src/flag_gems/utils/shape_utils.py:70-86)."""
    r1, r2 = len(s1), len(s2)
    if r1 == 0:
        return True
    if r2 == 0:
        return False
    if r1 > r2:
        return False
    d = r2 - r1
    for i in range(r1):
        if s1[i] != 1 and s1[i] != s2[d + i]:
            return False
    return True


def _covers(bias, mat1, mat2):
    return (
        mat1.dim() == 2 and mat2.dim() == 2
        and _C.supported_dtype(bias.dtype) and _C.supported_dtype(mat1.dtype) and _C.supported_dtype(mat2.dtype)
    )


def _vendor_addmm(bias, mat1, mat2, beta, alpha, out=None):
    M, N = mat1.shape[0], mat2.shape[1]
    r = torch.baddbmm(
        bias.broadcast_to((M, N)).unsqueeze(0), mat1.unsqueeze(0), mat2.unsqueeze(0), beta=beta, alpha=alpha
    ).squeeze(0)
    if out is None:
        return r
    out.copy_(r)
    return out


def _run(bias, mat1, mat2, beta, alpha, out):
    M, K = mat1.shape
    N = mat2.shape[1]
    if logger.isEnabledFor(logging.DEBUG):
        logger.debug(
            "GEMS ADDMM, [shape info]: [-, %s, %s, %s](batch, M, N, K), "
            "[A column-major]: %s, [B column-major]: %s, [bias column-major]: %s",
            M, N, K, mat1.stride(0) == 1, mat2.stride(0) == 1, bias.stride(0) == 1 if bias.dim() else True,
        )
    if M == 0 or N == 0:
        return out
    mat1 = mat1.contiguous()
    if mat2.stride(0) > 1 and mat2.stride(1) > 1:
        mat2 = mat2.contiguous()
    bias = bias.broadcast_to((M, N))
    if mat1.dtype != mat2.dtype:
        hi = get_higher_dtype(mat1.dtype, mat2.dtype)
        mat1, mat2 = mat1.to(hi), mat2.to(hi)
    if K == 0:
        out.copy_(bias * beta)
        return out
    return gemm(mat1, mat2, bias, out, float(alpha), float(beta))


def addmm(bias, mat1, mat2, *, beta=1, alpha=1):
    assert mat1.shape[1] == mat2.shape[0], "Incompatible dimensions"
    assert broadcastable_to(bias.shape, (mat1.shape[0], mat2.shape[1])), "Incompatible input shape"
    if not _covers(bias, mat1, mat2):
        return _vendor_addmm(bias, mat1, mat2, beta, alpha)
    M, N = mat1.shape[0], mat2.shape[1]
    # The reference allocates in mat1's dtype and stores values cast to the bias dtype
    # (src/flag_gems/ops/addmm.py:79,103); both are the same dtype on every path torch allows.
    out = torch.empty((M, N), device=mat1.device, dtype=mat1.dtype)
    return _run(bias, mat1, mat2, beta, alpha, out)


def addmm_out(bias, mat1, mat2, *, beta=1, alpha=1, out=None):
    assert mat1.shape[1] == mat2.shape[0], "Incompatible dimensions"
    assert broadcastable_to(bias.shape, (mat1.shape[0], mat2.shape[1])), "Incompatible input shape"
    M, N = mat1.shape[0], mat2.shape[1]
    if out is None:
        out = torch.empty((M, N), device=mat1.device, dtype=mat1.dtype)
    else:
        assert out.shape == (M, N), "Incompatible output shape"
    if not _covers(bias, mat1, mat2) or not _C.supported_dtype(out.dtype):
        return _vendor_addmm(bias, mat1, mat2, beta, alpha, out)
    return _run(bias, mat1, mat2, beta, alpha, out)
