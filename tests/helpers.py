"""Shared helpers of the parity tests: the reference's comparison rule plus error reporting."""
import torch

from flaggems_amd.testing import RESOLUTION


def gems_assert_close(res, ref, dtype, equal_nan=False, reduce_dim=1, atol=1e-4):
    """tests/accuracy_utils.py:196-200 of the reference: the result is brought to the host, the
    reference cast to the result dtype, atol = 1e-4 * reduce_dim, rtol = RESOLUTION[dtype]."""
    res = res.detach().to("cpu")
    assert res.dtype == dtype, f"result dtype {res.dtype} != {dtype}"
    ref = ref.to(dtype)
    torch.testing.assert_close(res, ref, atol=atol * reduce_dim, rtol=RESOLUTION[dtype], equal_nan=equal_nan)


def gems_assert_equal(res, ref, equal_nan=False):
    torch.testing.assert_close(res.detach().to("cpu"), ref, atol=0, rtol=0, equal_nan=equal_nan)


def err_stats(res, ref):
    res = res.detach().to("cpu").double()
    ref = ref.double()
    d = (res - ref).abs()
    fin = torch.isfinite(ref)
    rel = d[fin] / ref[fin].abs().clamp_min(1e-30)
    return float(d[fin].max()) if fin.any() else 0.0, float(rel.max()) if fin.any() else 0.0


FLOAT_DTYPES = [torch.float16, torch.float32, torch.bfloat16]
SCALARS = [0.001, -0.999, 100.001, -111.999]  # tests/accuracy_utils.py:169
MNK_SHAPES = [(1, 1, 32), (15, 160, 1024), (495, 5333, 71)]  # tests/test_blas_ops.py:17-20
REDUCTION_SHAPES = [(1, 2), (4096, 256), (200, 40999)]  # tests/accuracy_utils.py:70 (2-d part)
SOFTMAX_SHAPES = [(1, 256), (4096, 256), (200, 2560, 3)]
