"""ctypes binding of the plain-C oracle (oracle/kv_oracle.c).  Test infrastructure only."""
import ctypes
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB = os.path.join(_HERE, "liboracle.so")
_lib = None


def build(force=False):
    if force or not os.path.exists(_LIB) or os.path.getmtime(_LIB) < os.path.getmtime(os.path.join(_HERE, "kv_oracle.c")):
        subprocess.run(["make", "-s", "-C", _HERE, "-B" if force else "-s", "liboracle.so"], check=True)
    return _LIB


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(_LIB):
            build()
        h = ctypes.CDLL(_LIB)
        vp, i64 = ctypes.c_void_p, ctypes.c_int64
        h.oracle_reshape_and_cache_flash.argtypes = [vp, vp, vp, vp, vp, i64, i64, i64, i64, i64, i64, ctypes.c_int]
        h.oracle_reshape_and_cache_flash.restype = None
        h.oracle_virtual_to_cache.argtypes = [i64, vp, i64, i64]
        h.oracle_virtual_to_cache.restype = i64
        h.oracle_streamk_partition.argtypes = [i64, i64, i64, vp, vp]
        h.oracle_streamk_partition.restype = i64
        h.oracle_fused_add_rms_norm_f32.argtypes = [vp, vp, vp, i64, i64, ctypes.c_float]
        h.oracle_fused_add_rms_norm_f32.restype = None
        _lib = h
    return _lib


def reshape_and_cache_flash(key, value, key_cache, value_cache, slot_mapping, key_stride, value_stride, block_stride):
    """key/value: flat numpy arrays (any dtype) holding the token rows at the given element strides;
    key_cache/value_cache: numpy arrays [num_blocks*...] updated in place; slot_mapping int64."""
    n = key_cache.shape[2] * key_cache.shape[3]
    block_size = key_cache.shape[1]
    slots = np.ascontiguousarray(slot_mapping, dtype=np.int64)
    lib().oracle_reshape_and_cache_flash(
        key.ctypes.data, value.ctypes.data, key_cache.ctypes.data, value_cache.ctypes.data, slots.ctypes.data,
        len(slots), n, block_size, key_stride, value_stride, block_stride, key_cache.itemsize,
    )


def virtual_to_cache(virt, page_table, block_size, k_row_stride):
    pt = np.ascontiguousarray(page_table, dtype=np.int32)
    return lib().oracle_virtual_to_cache(virt, pt.ctypes.data, block_size, k_row_stride)


def streamk_partition(tiles, iters_per_tile, workers):
    b = np.zeros(workers, dtype=np.int64)
    e = np.zeros(workers, dtype=np.int64)
    coop = lib().oracle_streamk_partition(tiles, iters_per_tile, workers, b.ctypes.data, e.ctypes.data)
    return coop, b, e


def fused_add_rms_norm_f32(x, residual, w, eps):
    """In place on float32 C-contiguous numpy arrays x, residual [M, N]; w [N]."""
    M, N = x.shape
    lib().oracle_fused_add_rms_norm_f32(x.ctypes.data, residual.ctypes.data, w.ctypes.data, M, N, eps)
