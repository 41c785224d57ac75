"""ctypes binding of libfg_mi355.so, the C-ABI library that holds every gfx950 kernel.

The library links the HIP runtime by soname; torch is imported first so that the runtime torch
already mapped is the one the kernels launch on (two HIP runtimes in one process would not share
streams or allocations).  Nothing here falls back to another implementation: when the library is
missing, or a call fails, the caller gets an exception.
"""
import ctypes
import os
import threading

import torch

_HERE = os.path.dirname(os.path.abspath(__file__))
# FG_LIB_PATH names another build of the same library (csrc/build.py --variant ... --tag TAG: kernel variants on trial)
LIB_PATH = os.environ.get("FG_LIB_PATH") or os.path.join(_HERE, "libfg_mi355.so")

FG_F16, FG_BF16, FG_F32 = 0, 1, 2
SCHED_AUTO, SCHED_DATA_PARALLEL, SCHED_STREAM_K = 0, 1, 2

_DTYPE_ID = {torch.float16: FG_F16, torch.bfloat16: FG_BF16, torch.float32: FG_F32}

c_i64 = ctypes.c_int64
c_int = ctypes.c_int
c_vp = ctypes.c_void_p
c_f32 = ctypes.c_float
I64x3 = c_i64 * 3


class FgFlashParams(ctypes.Structure):
    """Mirror of struct FgFlashParams in include/fg_mi355.h (field order and widths must match)."""

    _fields_ = [
        ("q", c_vp),
        ("k_cache", c_vp),
        ("v_cache", c_vp),
        ("out", c_vp),
        ("lse", c_vp),
        ("cu_seqlens_q", c_vp),
        ("seqused_k", c_vp),
        ("block_table", c_vp),
        ("alibi_slopes", c_vp),
        ("q_row_stride", c_i64),
        ("q_head_stride", c_i64),
        ("o_row_stride", c_i64),
        ("o_head_stride", c_i64),
        ("k_page_stride", c_i64),
        ("k_row_stride", c_i64),
        ("k_head_stride", c_i64),
        ("v_page_stride", c_i64),
        ("v_row_stride", c_i64),
        ("v_head_stride", c_i64),
        ("block_table_stride", c_i64),
        ("alibi_batch_stride", c_i64),
        ("total_q", c_i64),
        ("batch", ctypes.c_int32),
        ("Hq", ctypes.c_int32),
        ("Hk", ctypes.c_int32),
        ("D", ctypes.c_int32),
        ("page_size", ctypes.c_int32),
        ("max_seqlen_q", ctypes.c_int32),
        ("max_seqlen_k", ctypes.c_int32),
        ("is_causal", ctypes.c_int32),
        ("window_left", ctypes.c_int32),
        ("window_right", ctypes.c_int32),
        ("softmax_scale", c_f32),
        ("softcap", c_f32),
        ("dtype", ctypes.c_int32),
        ("workspace", c_vp),
        ("workspace_bytes", c_i64),
    ]


_SIGNATURES = {
    "fg_last_error": (ctypes.c_char_p, []),
    "fg_abi_version": (c_int, []),
    "fg_device_info": (c_int, [c_int, ctypes.POINTER(c_int), ctypes.POINTER(c_int), ctypes.POINTER(c_int)]),
    "fg_mfma_probe": (c_int, [c_vp, c_vp, c_int, c_int, ctypes.POINTER(ctypes.c_double), c_vp]),
    "fg_rms_norm": (c_int, [c_vp, c_vp, c_vp, c_vp, c_i64, c_i64, c_i64, c_i64, c_f32, c_int, c_vp]),
    "fg_fused_add_rms_norm": (c_int, [c_vp, c_vp, c_vp, c_i64, c_i64, c_i64, c_i64, c_f32, c_int, c_vp]),
    "fg_softmax": (c_int, [c_vp, c_vp, c_i64, c_i64, c_i64, c_int, c_int, c_vp]),
    "fg_log_softmax": (c_int, [c_vp, c_vp, c_i64, c_i64, c_i64, c_int, c_int, c_vp]),
    "fg_rope": (
        c_int,
        [c_vp, c_vp, c_vp, c_vp, c_vp, c_vp, c_vp, c_int, c_i64, c_i64, c_int, c_int, c_int,
         ctypes.POINTER(c_i64), ctypes.POINTER(c_i64), ctypes.POINTER(c_i64), ctypes.POINTER(c_i64),
         c_i64, c_i64, c_i64, c_i64, c_int, c_int, c_int, c_vp],
    ),
    "fg_reshape_and_cache_flash": (
        c_int,
        [c_vp, c_vp, c_vp, c_vp, c_vp, c_int, c_i64, c_int, c_int, c_int, c_i64, c_i64, c_i64, c_int, c_vp],
    ),
    "fg_reshape_and_cache": (
        c_int,
        [c_vp, c_vp, c_vp, c_vp, c_vp, c_int, c_i64, c_int, c_int, c_int, c_int, c_i64, c_i64, c_i64, c_int, c_vp],
    ),
    "fg_silu_and_mul": (c_int, [c_vp, c_vp, c_vp, c_i64, c_i64, c_i64, c_i64, c_i64, c_int, c_vp]),
    "fg_silu_and_mul_backward": (c_int, [c_vp, c_vp, c_vp, c_vp, c_vp, c_i64, c_i64, c_i64, c_i64, c_i64, c_i64, c_i64,
                                         c_int, c_vp]),
    "fg_softmax_backward": (c_int, [c_vp, c_vp, c_vp, c_i64, c_i64, c_i64, c_int, c_int, c_vp]),
    "fg_log_softmax_backward": (c_int, [c_vp, c_vp, c_vp, c_i64, c_i64, c_i64, c_int, c_int, c_vp]),
    "fg_rms_norm_backward_partial_rows": (c_i64, [c_i64, c_i64, c_int, c_int]),
    "fg_rms_norm_backward": (c_int, [c_vp, c_vp, c_vp, c_vp, c_vp, c_vp, c_i64, c_i64, c_i64, c_int, c_vp]),
    "fg_rms_norm_backward_dw": (c_int, [c_vp, c_i64, c_i64, c_vp, c_int, c_vp]),
    "fg_transpose2d": (c_int, [c_vp, c_vp, c_i64, c_i64, c_i64, c_i64, c_int, c_vp]),
    "fg_reload_options": (None, []),
    "fg_gemm_workspace_layout": (c_int, [c_int, ctypes.POINTER(ctypes.c_size_t), ctypes.POINTER(ctypes.c_size_t)]),
    "fg_stream_capture_id": (c_int, [c_vp, ctypes.POINTER(ctypes.c_ulonglong)]),
    "fg_gemm_workspace_bytes": (ctypes.c_size_t, [c_i64, c_i64, c_i64, c_int, c_int, c_int]),
    "fg_gemm": (
        c_int,
        [c_vp, c_vp, c_vp, c_vp, c_i64, c_i64, c_i64, c_i64, c_i64, c_i64, c_i64, c_i64, c_i64, c_i64, c_i64,
         c_f32, c_f32, c_int, c_int, c_int, c_int, c_vp, ctypes.c_size_t, ctypes.POINTER(c_int), c_vp],
    ),
    "fg_gemm_skinny_static": (
        c_int,
        [c_vp, c_vp, c_vp, c_vp, c_i64, c_i64, c_i64, c_i64, c_i64, c_i64, c_i64, c_i64, c_i64, c_i64, c_i64,
         c_f32, c_f32, c_int, c_int, c_int, c_vp],
    ),
    "fg_bmm": (
        c_int,
        [c_vp, c_vp, c_vp, c_i64, c_i64, c_i64, c_i64, c_i64, c_i64, c_i64, c_i64, c_i64, c_i64, c_i64, c_i64, c_i64,
         c_int, c_vp],
    ),
    "fg_gemm_tile_order": (c_int, [c_int, c_int, c_int, ctypes.POINTER(c_int), ctypes.POINTER(c_int)]),
    "fg_gemm_plan": (
        c_int,
        [c_i64, c_i64, c_i64, c_int, ctypes.POINTER(c_int), ctypes.POINTER(c_int), ctypes.POINTER(ctypes.c_double),
         ctypes.POINTER(c_int), ctypes.POINTER(ctypes.c_double), ctypes.POINTER(c_int)],
    ),
    "fg_streamk_partition": (
        c_int,
        [c_i64, c_i64, c_i64, ctypes.POINTER(c_i64), ctypes.POINTER(c_i64), ctypes.POINTER(c_i64)],
    ),
    "fg_flash_attn_varlen_fwd": (c_int, [ctypes.POINTER(FgFlashParams), c_vp]),
    "fg_flash_attn_workspace_bytes": (ctypes.c_size_t, [ctypes.POINTER(FgFlashParams), c_int]),
}

_lib = None
_lock = threading.Lock()


class ExtensionMissing(RuntimeError):
    pass


def lib():
    """The loaded library (loads on first use)."""
    global _lib
    if _lib is not None:
        return _lib
    with _lock:
        if _lib is not None:
            return _lib
        if not os.path.exists(LIB_PATH):
            raise ExtensionMissing(
                "libfg_mi355.so is not built (%s). Build it with `python flaggems_amd/csrc/build.py`; "
                "there is no fallback implementation." % LIB_PATH
            )
        # torch's bundled HIP runtime must already be mapped (import torch above does that); load it
        # by its file name as well so the soname lookup below resolves to the same object.
        hip_rt = os.path.join(os.path.dirname(torch.__file__), "lib", "libamdhip64.so")
        if os.path.exists(hip_rt):
            ctypes.CDLL(hip_rt, mode=ctypes.RTLD_GLOBAL)
        handle = ctypes.CDLL(LIB_PATH)
        for name, (res, args) in _SIGNATURES.items():
            fn = getattr(handle, name)  # AttributeError here means header and library disagree
            fn.restype = res
            fn.argtypes = args
        _lib = handle
    return _lib


def exported_symbols():
    return list(_SIGNATURES)


def last_error():
    return lib().fg_last_error().decode("utf-8", "replace")


def check(rc, what):
    if rc != 0:
        raise RuntimeError("%s failed (code %d): %s" % (what, rc, last_error()))


def dtype_id(dtype):
    try:
        return _DTYPE_ID[dtype]
    except KeyError:
        raise TypeError("dtype %s is not supported by the gfx950 kernels (fp16, bf16, fp32 only)" % dtype)


def supported_dtype(dtype):
    return dtype in _DTYPE_ID


def current_stream(device):
    """Raw handle of torch's current stream on `device` (the launches of this library go there)."""
    index = device.index
    if index is None:
        index = torch.cuda.current_device()
    return torch._C._cuda_getCurrentRawStream(index)


class _NoGuard:
    def __enter__(self):
        return None

    def __exit__(self, *exc):
        return False


_NO_GUARD = _NoGuard()


def device_guard(device):
    """Context that makes `device` current for the library call.  Switching devices costs several
    microseconds per call, as much as a small kernel runs; when the device is current already (the
    usual case) nothing is switched."""
    index = device.index
    if index is None or index == torch.cuda.current_device():
        return _NO_GUARD
    return torch.cuda.device(device)


_dev_info = {}


def device_info(index):
    """(num_cu, lds_bytes, gcn_arch) of a device, cached."""
    if index not in _dev_info:
        a, b, c = c_int(), c_int(), c_int()
        check(lib().fg_device_info(index, ctypes.byref(a), ctypes.byref(b), ctypes.byref(c)), "fg_device_info")
        _dev_info[index] = (a.value, b.value, c.value)
    return _dev_info[index]
