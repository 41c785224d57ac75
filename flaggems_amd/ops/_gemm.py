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


# One scratch buffer per (device, stream): stream-K partial tiles behind a header of ticket counters.  The
# reference allocates these per call (src/flag_gems/ops/mm_streamk.py:488-491); launches on one stream are
# ordered, so a buffer per stream is reused without a hazard.  The buffer has the largest size any problem can
# ask for on the device and is never replaced: a HIP graph that recorded its address stays valid whatever runs
# later.  Only the header has to read zero when a launch starts, and the kernels return it to zero.  It is
# cleared when the buffer is made and, once per graph capture that uses the buffer, by a fill kernel recorded
# into that graph, so that every replay starts from a cleared header whichever graph of the stream ran (or was
# only recorded) before it.  A buffer whose first use falls inside a capture has only a recorded clear; its first
# eager use clears it for real.
_workspaces = {}
_layouts = {}
_capture_id = ctypes.c_ulonglong(0)


def _workspace(device, stream):
    lib = _C.lib()
    key = (device.index, stream)
    entry = _workspaces.get(key)
    _C.check(lib.fg_stream_capture_id(stream, ctypes.byref(_capture_id)), "fg_stream_capture_id")
    capture = _capture_id.value
    if entry is None:
        layout = _layouts.get(device.index)
        if layout is None:
            total, header = ctypes.c_size_t(0), ctypes.c_size_t(0)
            _C.check(lib.fg_gemm_workspace_layout(device.index, ctypes.byref(total), ctypes.byref(header)),
                     "fg_gemm_workspace_layout")
            layout = _layouts[device.index] = (total.value, header.value)
        buf = torch.empty(layout[0], dtype=torch.uint8, device=device)
        buf[:layout[1]].zero_()
        # entry: buffer, capture id last seen, header bytes, whether a clear has ever RUN (one issued under capture
        # is only recorded into that graph)
        entry = _workspaces[key] = [buf, capture, layout[1], capture == 0]
    elif capture != entry[1]:
        if capture != 0:
            entry[0][:entry[2]].zero_()
        elif not entry[3]:
            # the buffer was made under capture and this is its first eager use: no clear has run yet unless that
            # graph was replayed, so the header may hold whatever the allocation held
            entry[0][:entry[2]].zero_()
            entry[3] = True
        entry[1] = capture
    return entry[0]


_last_schedule = ctypes.c_int(0)
_last_schedule_ref = ctypes.byref(_last_schedule)


def last_schedule():
    """Schedule the most recent gemm call on this process used (1 data-parallel, 2 stream-K)."""
    return _last_schedule.value


# fg_gemm_workspace_bytes is a pure function of its arguments (shape, dtype, schedule and the device's CU count):
# its answers are kept, so that a decode-size call pays for one transition into the library, not two.
_ws_need = {}


def gemm(a, b, bias, c, alpha=1.0, beta=0.0, schedule=_C.SCHED_AUTO):
    """c = alpha * a @ b + beta * bias, with every operand addressed through its strides."""
    M, K = a.shape
    N = b.shape[1]
    lib = _C.lib()
    dev = c.device
    with _C.device_guard(dev):
        stream = _C.current_stream(dev)
        ab = _C.dtype_id(a.dtype)
        key = (M, N, K, ab, schedule, dev.index)
        ws_bytes = _ws_need.get(key)
        if ws_bytes is None:
            if len(_ws_need) > 4096:
                _ws_need.clear()
            ws_bytes = _ws_need[key] = lib.fg_gemm_workspace_bytes(M, N, K, ab, schedule, dev.index)
        if ws_bytes:
            ws = _workspace(dev, stream)
            wptr, wlen = ws.data_ptr(), ws.numel()
        else:
            wptr, wlen = None, 0
        if bias is not None:
            (sim, sin_), bptr, bdt = bias.stride(), bias.data_ptr(), _C.dtype_id(bias.dtype)
        else:
            bptr, sim, sin_, bdt = None, 0, 0, ab
        sam, sak = a.stride()
        sbk, sbn = b.stride()
        scm, scn = c.stride()
        rc = lib.fg_gemm(
            a.data_ptr(), b.data_ptr(), bptr, c.data_ptr(), M, N, K, sam, sak, sbk, sbn, sim, sin_, scm, scn,
            alpha, beta, ab, _C.dtype_id(c.dtype), bdt, schedule, wptr, wlen, _last_schedule_ref, stream,
        )
    if rc != 0:
        _C.check(rc, "fg_gemm")
    return c
