"""fg_gemm_skinny_static (the entry point that allocates nothing: its stream-K scratch is a static device array)
against fg_gemm with a caller-provided workspace, through the C ABI: bit-identical results on two calls in a row,
the second on a smaller problem, for both B layouts and row counts on either side of 16; plus its error paths."""
import ctypes

import pytest
import torch

from flaggems_amd import _C
from oracle import torch_ref as O

pytestmark = pytest.mark.gpu


def _call(entry, a, b, bias, out, alpha, beta, ws=None):
    lib = _C.lib()
    stream = _C.current_stream(out.device)
    head = (a.data_ptr(), b.data_ptr(), bias.data_ptr() if bias is not None else None, out.data_ptr(),
            a.shape[0], b.shape[1], a.shape[1], a.stride(0), a.stride(1), b.stride(0), b.stride(1),
            0 if bias is None else bias.stride(0), 0 if bias is None else bias.stride(1), out.stride(0), out.stride(1),
            alpha, beta, _C.dtype_id(a.dtype), _C.dtype_id(out.dtype), _C.dtype_id(a.dtype))
    if entry == "static":
        return lib.fg_gemm_skinny_static(*head, stream)
    used = ctypes.c_int(0)
    rc = lib.fg_gemm(*head, _C.SCHED_STREAM_K, ws.data_ptr(), ws.numel(), ctypes.byref(used), stream)
    assert used.value == _C.SCHED_STREAM_K
    return rc


def _problem(dev, M, N, K, dtype, b_kc, seed, with_bias):
    g = torch.Generator(device="cpu").manual_seed(seed)
    a = (torch.randn(M, K, generator=g) / K ** 0.5).to(dtype).to(dev)
    b = (torch.randn(N, K, generator=g).to(dtype).to(dev).t() if b_kc else torch.randn(K, N, generator=g).to(dtype).to(dev))
    bias = torch.randn(M, N, generator=g).to(dtype).to(dev) if with_bias else None
    return a, b, bias


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("b_kc", [True, False])
def test_static_scratch_gemm_matches_workspace_gemm(gpu, dtype, b_kc):
    lib = _C.lib()
    total, header = ctypes.c_size_t(0), ctypes.c_size_t(0)
    assert lib.fg_gemm_workspace_layout(gpu.index, ctypes.byref(total), ctypes.byref(header)) == 0
    ws = torch.zeros(total.value, dtype=torch.uint8, device=gpu)
    # two calls in a row, the second smaller; then more shapes (ragged N, a tile split over many workgroups, bias)
    shapes = [(16, 4096, 14336, False), (5, 520, 2048, False), (1, 4096, 4096, True), (16, 136, 8192, True)]
    if b_kc:
        shapes += [(48, 1024, 4096, False), (17, 4096, 1024, True)]
    for i, (M, N, K, with_bias) in enumerate(shapes):
        a, b, bias = _problem(gpu, M, N, K, dtype, b_kc, 100 + i, with_bias)
        want = torch.empty(M, N, dtype=dtype, device=gpu)
        got = torch.full((M, N), float("nan"), dtype=dtype, device=gpu)
        alpha, beta = (0.5, 2.0) if with_bias else (1.0, 0.0)
        assert _call("workspace", a, b, bias, want, alpha, beta, ws) == 0, _C.last_error()
        assert _call("static", a, b, bias, got, alpha, beta) == 0, _C.last_error()
        torch.cuda.synchronize()
        assert torch.equal(got, want), (M, N, K)
        ref = O.addmm(bias, a, b, alpha=alpha, beta=beta) if with_bias else O.mm(a, b)
        torch.testing.assert_close(got.cpu().double(), ref.double(), atol=1e-4 * K, rtol=1.6e-2)


def test_static_scratch_gemm_back_to_back_and_in_a_graph(gpu):
    """Calls queued back to back on one stream share the array without a host synchronisation in between, and a
    call recorded into a HIP graph (where nothing may be allocated) replays to the same bits."""
    dtype = torch.bfloat16
    probs = [_problem(gpu, 8, 4096, 4096, dtype, True, 7, False), _problem(gpu, 3, 264, 1024, dtype, True, 8, False)]
    wants = [torch.empty(a.shape[0], b.shape[1], dtype=dtype, device=gpu) for a, b, _ in probs]
    total, header = ctypes.c_size_t(0), ctypes.c_size_t(0)
    _C.lib().fg_gemm_workspace_layout(gpu.index, ctypes.byref(total), ctypes.byref(header))
    ws = torch.zeros(total.value, dtype=torch.uint8, device=gpu)
    for (a, b, _), w in zip(probs, wants):
        assert _call("workspace", a, b, None, w, 1.0, 0.0, ws) == 0
    gots = [torch.zeros_like(w) for w in wants]
    for _ in range(4):
        for (a, b, _), g in zip(probs, gots):
            assert _call("static", a, b, None, g, 1.0, 0.0) == 0
    torch.cuda.synchronize()
    for g, w in zip(gots, wants):
        assert torch.equal(g, w)
    side = torch.cuda.Stream()
    graph = torch.cuda.CUDAGraph()
    outs = [torch.zeros_like(w) for w in wants]
    with torch.cuda.graph(graph, stream=side):
        for (a, b, _), o in zip(probs, outs):
            assert _call("static", a, b, None, o, 1.0, 0.0) == 0
    for _ in range(3):
        for o in outs:
            o.zero_()
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        for o, w in zip(outs, wants):
            assert torch.equal(o, w)


def test_static_scratch_gemm_rejects_what_it_cannot_hold(gpu):
    dtype = torch.bfloat16
    a, b, _ = _problem(gpu, 65, 512, 2048, dtype, True, 1, False)
    out = torch.empty(65, 512, dtype=dtype, device=gpu)
    assert _call("static", a, b, None, out, 1.0, 0.0) == -2
    assert "exceed the maximum of 64" in _C.last_error()
    a, b, _ = _problem(gpu, 8, 512, 512, dtype, True, 2, False)  # K too shallow for the stream-K kernels
    out = torch.empty(8, 512, dtype=dtype, device=gpu)
    assert _call("static", a, b, None, out, 1.0, 0.0) == -2
    assert "use fg_gemm" in _C.last_error()
    a32 = torch.randn(8, 2048, device=gpu)
    b32 = torch.randn(2048, 512, device=gpu)
    out = torch.empty(8, 512, device=gpu)
    assert _call("static", a32, b32, None, out, 1.0, 0.0) == -2


_FIRST_CALL_UNDER_CAPTURE = r"""
import ctypes, os, sys
import torch
sys.path.insert(0, os.path.join(os.getcwd(), "tests"))
import test_zz_no_alloc as T
from flaggems_amd import _C

lib = _C.lib()
dev = torch.device("cuda:0")
a, b, _ = T._problem(dev, 8, 4096, 4096, torch.bfloat16, True, 7, False)
total, header = ctypes.c_size_t(0), ctypes.c_size_t(0)
assert lib.fg_gemm_workspace_layout(0, ctypes.byref(total), ctypes.byref(header)) == 0
ws = torch.zeros(total.value, dtype=torch.uint8, device=dev)
want = torch.empty(8, 4096, dtype=torch.bfloat16, device=dev)
assert T._call("workspace", a, b, None, want, 1.0, 0.0, ws) == 0
out = torch.zeros_like(want)
torch.cuda.synchronize()
side = torch.cuda.Stream()
g1 = torch.cuda.CUDAGraph()
with torch.cuda.graph(g1, stream=side):
    out.zero_()                                              # (a fill kernel: the captured graph is not empty)
    rc = T._call("static", a, b, None, out, 1.0, 0.0)       # the process's first call: refused, capture intact
    msg = _C.last_error()
assert rc == -2 and "under stream capture" in msg, (rc, msg)
g1.replay()                                                  # the capture the refused call sat in is a working graph
torch.cuda.synchronize()
n = ctypes.c_int(0)
assert lib.fg_device_info(0, ctypes.byref(n), None, None) == 0 and n.value > 0
g2 = torch.cuda.CUDAGraph()
with torch.cuda.graph(g2, stream=side):
    assert T._call("static", a, b, None, out, 1.0, 0.0) == 0, _C.last_error()
for _ in range(2):
    out.zero_()
    torch.cuda.synchronize()
    g2.replay()
    torch.cuda.synchronize()
    assert torch.equal(out, want)
print("FIRST-CALL-UNDER-CAPTURE OK")
"""


def test_first_call_under_capture_is_refused_until_the_device_is_primed(gpu):
    """In a fresh process: the entry point's first call on a device, made under stream capture, returns
    FG_ERR_UNSUPPORTED and leaves the capture usable; after fg_device_info for that device the same call is recorded
    and replays to fg_gemm's bits.  (A child process, because this process has long made its first call.)"""
    import os
    import subprocess
    import sys

    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    p = subprocess.run([sys.executable, "-c", _FIRST_CALL_UNDER_CAPTURE], cwd=root, capture_output=True, text=True,
                       timeout=300)
    assert p.returncode == 0 and "FIRST-CALL-UNDER-CAPTURE OK" in p.stdout, (p.stdout[-2000:], p.stderr[-4000:])
