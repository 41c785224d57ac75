"""GPU parity of the backward kernels (softmax, log_softmax, rms_norm) against the CPU oracle.
Shapes and value ranges follow tests/test_reduction_ops.py:483-557 and tests/test_norm_ops.py:516-559 of the
reference."""
import numpy as np
import pytest
import torch

import flag_gems
from oracle import torch_ref as O

from helpers import FLOAT_DTYPES, REDUCTION_SHAPES, SOFTMAX_SHAPES, gems_assert_close

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("dtype", FLOAT_DTYPES)
@pytest.mark.parametrize("shape", SOFTMAX_SHAPES + [(16, 2048), (7, 40999), (5, 33), (3, 16392), (64, 8192), (3, 70000), (2, 131072),
                                                    (9, 1001), (4, 1500), (6, 100), (4, 300), (3, 500)])
@pytest.mark.parametrize("neg_inf", [False, True])
def test_softmax_backward(gpu, shape, dtype, neg_inf):
    torch.manual_seed(0)
    for dim in range(len(shape)):
        grad = torch.randn(shape, dtype=dtype, device=gpu)
        if neg_inf:
            grad = torch.where(grad < 0.0, float("-inf"), grad)
        out = torch.randn_like(grad)  # as in the reference test: any tensor stands for the forward's output
        ref = O.softmax_backward(grad, out, dim)
        with flag_gems.use_gems():
            res = torch.ops.aten._softmax_backward_data(grad, out, dim, dtype)
        gems_assert_close(res, ref, dtype, reduce_dim=shape[dim], equal_nan=True)


@pytest.mark.parametrize("dtype", FLOAT_DTYPES)
@pytest.mark.parametrize("shape", REDUCTION_SHAPES + [(200, 2560, 3), (16, 2048), (5, 33), (8, 32000), (3, 70001), (2, 151936),
                                                      (9, 1001)])
def test_log_softmax_backward(gpu, shape, dtype):
    torch.manual_seed(0)
    for dim in range(len(shape)):
        grad = torch.randn(shape, dtype=dtype, device=gpu)
        out = torch.randn_like(grad)
        ref = O.log_softmax_backward(grad, out, dim)
        with flag_gems.use_gems():
            res = torch.ops.aten._log_softmax_backward_data(grad, out, dim, dtype)
        gems_assert_close(res, ref, dtype, reduce_dim=shape[dim])


def test_softmax_backward_through_autograd(gpu):
    """softmax / log_softmax of real rows, differentiated under the override: forward and backward kernels
    of this package on both sides; fp16 input with an fp32 result exercises the narrowing gradient."""
    torch.manual_seed(1)
    x = torch.randn(33, 1000, device=gpu)
    dy = torch.randn(33, 1000, device=gpu)
    for fn, ofwd, obwd in ((torch.softmax, O.softmax, O.softmax_backward),
                           (torch.log_softmax, O.log_softmax, O.log_softmax_backward)):
        xg = x.clone().requires_grad_(True)
        with flag_gems.use_gems():
            y = fn(xg, -1)
            (gx,) = torch.autograd.grad(y, xg, dy)
        gems_assert_close(gx, obwd(dy, ofwd(x, -1), 1), torch.float32, reduce_dim=1000)
        xh = x.half().requires_grad_(True)
        with flag_gems.use_gems():
            y = fn(xh, -1, dtype=torch.float32)  # half_to_float forward
            (gh,) = torch.autograd.grad(y, xh, dy)
        assert y.dtype == torch.float32 and gh.dtype == torch.float16
        gems_assert_close(gh, obwd(dy, ofwd(x.half(), -1), 1), torch.float16, reduce_dim=1000)
    # empty tensors and dtypes without a kernel
    e = torch.empty(0, 7, device=gpu)
    assert flag_gems.softmax_backward(e, e, 1, torch.float32).shape == (0, 7)
    yd = torch.softmax(x.double(), -1); gd = dy.double()
    with flag_gems.use_gems():
        rd = torch.ops.aten._softmax_backward_data(gd, yd, 1, torch.float64)
    assert rd.dtype == torch.float64 and torch.allclose(rd.cpu(), O.softmax_backward(gd, yd, 1), atol=1e-12)


@pytest.mark.parametrize("dtype", FLOAT_DTYPES)
@pytest.mark.parametrize("shape", REDUCTION_SHAPES + [(64, 4096), (3, 5, 1024), (17, 8200), (130, 16392), (1000, 33), (5, 40999),
                                                      (3, 70000)])
def test_rms_norm_backward(gpu, shape, dtype):
    np.random.seed(0)
    n = shape[-1]
    x = torch.from_numpy(np.random.uniform(-0.1, 0.1, shape).astype(np.float32)).to(dtype).to(gpu).requires_grad_(True)
    dy = torch.from_numpy(np.random.uniform(-0.01, 0.01, shape).astype(np.float32)).to(dtype).to(gpu)
    w = torch.from_numpy(np.random.uniform(-0.1, 0.1, (n,)).astype(np.float32)).to(dtype).to(gpu).requires_grad_(True)
    y = flag_gems.rms_norm(x, [n], w, 1e-5)
    gems_assert_close(y, O.rms_norm(x, w, 1e-5), dtype)
    dx, dw = torch.autograd.grad(y, (x, w), dy)
    ref_dx, ref_dw = O.rms_norm_grads(x.detach().view(-1, n), w.detach(), 1e-5, dy.view(-1, n))
    rows = x.numel() // n
    gems_assert_close(dx, ref_dx.view(shape), dtype)
    # rows terms of magnitude ~1e-3 are added per column, the last step rounding to dtype
    gems_assert_close(dw, ref_dw, dtype, reduce_dim=max(1, rows // 64))
    # input gradient alone (no weight gradient wanted: the column-sum kernel is skipped)
    x2 = x.detach().clone().requires_grad_(True)
    (dx2,) = torch.autograd.grad(flag_gems.rms_norm(x2, [n], w.detach(), 1e-5), x2, dy)
    assert torch.equal(dx2, dx)


def test_rms_norm_backward_variants(gpu):
    torch.manual_seed(3)
    x = torch.randn(37, 96, device=gpu, requires_grad=True)
    dy = torch.randn(37, 96, device=gpu)
    # no weight; two trailing dims; a non-contiguous upstream gradient
    y = flag_gems.rms_norm(x, [96], None, 1e-6)
    (dx,) = torch.autograd.grad(y, x, dy)
    ref_dx, _ = O.rms_norm_grads(x.detach(), torch.ones(96), 1e-6, dy)
    gems_assert_close(dx, ref_dx, torch.float32)
    w = torch.randn(4, 24, device=gpu, requires_grad=True)
    y = flag_gems.rms_norm(x.view(37, 4, 24), [4, 24], w, 1e-5)
    gt = torch.randn(24, 4, 37, device=gpu).permute(2, 1, 0)
    dx, dw = torch.autograd.grad(y, (x, w), gt)
    ref_dx, ref_dw = O.rms_norm_grads(x.detach(), w.detach().view(96), 1e-5, gt.reshape(37, 96))
    gems_assert_close(dx, ref_dx, torch.float32)
    gems_assert_close(dw, ref_dw.view(4, 24), torch.float32, reduce_dim=37)
    # without a graph the forward kernel alone runs and nothing is saved
    with torch.no_grad():
        assert not flag_gems.rms_norm(x, [96], None, 1e-6).requires_grad


@pytest.mark.parametrize("dtype", FLOAT_DTYPES)
@pytest.mark.parametrize("rows,N", [(1, 32), (7, 33), (32, 4096), (100, 1000), (1024, 4096), (513, 8200), (0, 64)])
def test_rms_norm_backward_dw_column_sum(gpu, rows, N, dtype):
    """fg_rms_norm_backward_dw through the C ABI: fp32 column sums of the partial rows, rounded once to the
    output dtype, identical from call to call."""
    from flaggems_amd import _C

    torch.manual_seed(rows + N)
    partial = torch.randn(rows, N, dtype=torch.float32, device=gpu) * 3.0
    lib = _C.lib()
    outs = []
    for _ in range(3):
        dw = torch.full((N,), float("nan"), dtype=dtype, device=gpu)
        rc = lib.fg_rms_norm_backward_dw(partial.data_ptr() if rows else None, rows, N, dw.data_ptr(), _C.dtype_id(dtype),
                                         _C.current_stream(dw.device))
        assert rc == 0, _C.last_error()
        outs.append(dw)
    ref = partial.double().sum(0).cpu()
    # fp32 accumulation of `rows` terms of size ~3, then one rounding to dtype
    eps = {torch.float16: 1e-3, torch.bfloat16: 7.8e-3, torch.float32: 1.2e-7}[dtype]
    err = (outs[0].double().cpu() - ref).abs()
    bound = ref.abs() * eps + 1e-5 * max(rows, 1)
    assert bool((err <= bound).all()), float((err - bound).max())
    assert torch.equal(outs[0], outs[1]) and torch.equal(outs[0], outs[2])
