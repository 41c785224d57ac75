"""aten::bmm on the gfx950 MFMA GEMM, one launch per matrix (reference: src/flag_gems/ops/bmm.py:121-136)."""
import logging

import torch

from .. import _C
from ._gemm import gemm

logger = logging.getLogger("flag_gems.ops.bmm")


def _vendor_bmm(A, B):
    # the .out overload is a separate ATen kernel that stays on the vendor library
    out = torch.empty((A.shape[0], A.shape[1], B.shape[2]), dtype=A.dtype, device=A.device)
    return torch.ops.aten.bmm.out(A, B, out=out)


def _addressable(t):
    # the kernels take any strides, but load fast only when one of the two matrix dims is contiguous
    if t.stride(1) != 1 and t.stride(2) != 1:
        return t.contiguous()
    return t


# Largest batch the per-matrix launches are verified on: 16 matrices and 2^24 output elements in all.  A call
# beyond that (32 x 2048 x 2048 x 128 bf16, timed in a loop next to the vendor kernel) once ended in a GPU memory
# fault whose cause was not found in the kernels' address arithmetic; until it is, larger batches stay on the
# vendor kernel.
_MAX_BATCH = 16
_MAX_OUT_ELEMS = 1 << 24


def _within_verified_envelope(batch, M, N):
    return batch <= _MAX_BATCH and batch * M * N <= _MAX_OUT_ELEMS


def bmm(A, B):
    logger.debug("GEMS BMM")
    assert A.dim() == 3 and B.dim() == 3, "batch1 and batch2 must be 3D tensors"
    batch, M, K = A.shape
    assert B.shape[0] == batch and B.shape[1] == K, "incompatible dimensions"
    N = B.shape[2]
    if A.dtype != B.dtype or not _C.supported_dtype(A.dtype):
        return _vendor_bmm(A, B)
    if batch > 1 and not _within_verified_envelope(batch, M, N):
        return _vendor_bmm(A, B)
    out = torch.empty((batch, M, N), dtype=A.dtype, device=A.device)
    if batch == 0 or M == 0 or N == 0:
        return out
    if K == 0:
        return out.zero_()
    A = _addressable(A)
    B = _addressable(B)
    if batch == 1:
        # a single matrix has the skinny and stream-K schedules of mm at its disposal
        gemm(A[0], B[0], None, out[0])
        return out
    with _C.device_guard(out.device):
        rc = _C.lib().fg_bmm(
            A.data_ptr(), B.data_ptr(), out.data_ptr(), batch, M, N, K,
            A.stride(0), A.stride(1), A.stride(2), B.stride(0), B.stride(1), B.stride(2),
            out.stride(0), out.stride(1), out.stride(2), _C.dtype_id(A.dtype), _C.current_stream(out.device),
        )
    _C.check(rc, "fg_bmm")
    return out
