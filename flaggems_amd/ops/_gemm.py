"""Shared host half of mm / addmm: one fg_gemm call, plus the cached stream-K scratch buffer."""
import ctypes

import torch

from .. import _C

_ORDERED = [torch.float16, torch.bfloat16, torch.float32]


def get_higher_dtype(a, b):
    """Result dtype of a mixed-dtype mm, ordered fp16 < bf16 < fp32
    (reference: src/flag_gems/ops/mm.py:137-151)."""
    if a is b:
        return a
    assert a in _ORDERED
    assert b in _ORDERED
    for d in _ORDERED:
        if a is d:
            return b
        if b is d:
            return a


# One scratch buffer per (device, stream): stream-K partial tiles and their flags.  The reference
# allocates these per call (src/flag_gems/ops/mm_streamk.py:488-491); launches on one stream are
# ordered, so a buffer per stream can be reused without a hazard.
_workspaces = {}


def _workspace(device, stream, nbytes):
    key = (device.index, stream)
    buf = _workspaces.get(key)
    if buf is None or buf.numel() < nbytes:
        # zero-filled once: the kernels return their ticket counters to zero after every launch
        buf = torch.zeros(max(nbytes, 1 << 20), dtype=torch.uint8, device=device)
        _workspaces[key] = buf
    return buf


_last_schedule = ctypes.c_int(0)


def last_schedule():
    """Schedule the most recent gemm call on this process used (1 data-parallel, 2 stream-K)."""
    return _last_schedule.value


def gemm(a, b, bias, c, alpha=1.0, beta=0.0, schedule=_C.SCHED_AUTO):
    """c = alpha * a @ b + beta * bias, with every operand addressed through its strides."""
    M, K = a.shape
    N = b.shape[1]
    lib = _C.lib()
    dev = c.device
    with _C.device_guard(dev):
        stream = _C.current_stream(dev)
        ab = _C.dtype_id(a.dtype)
        ws_bytes = lib.fg_gemm_workspace_bytes(M, N, K, ab, schedule, dev.index)
        ws = _workspace(dev, stream, ws_bytes) if ws_bytes else None
        if bias is not None:
            bptr, sim, sin_, bdt = bias.data_ptr(), bias.stride(0), bias.stride(1), _C.dtype_id(bias.dtype)
        else:
            bptr, sim, sin_, bdt = None, 0, 0, ab
        rc = lib.fg_gemm(
            a.data_ptr(), b.data_ptr(), bptr, c.data_ptr(), M, N, K,
            a.stride(0), a.stride(1), b.stride(0), b.stride(1), sim, sin_, c.stride(0), c.stride(1),
            alpha, beta, ab, _C.dtype_id(c.dtype), bdt, schedule,
            ws.data_ptr() if ws is not None else None, ws.numel() if ws is not None else 0,
            ctypes.byref(_last_schedule), stream,
        )
    _C.check(rc, "fg_gemm")
    return c
