"""fg_gemm_plan: the host-only query of the automatic GEMM schedule (workgroup tile of the data-parallel launch,
stream-K or not), on a 256-CU device.  No GPU: the entry is arithmetic on the sizes.  The pinned choices are the
ones timed fastest on MI355X for these shapes; a change of the duration model that flips one of them must come with
a new measurement."""
import ctypes

import pytest

from flaggems_amd import _C


def plan(M, N, K, cu=256):
    bm, bn, w, ch = ctypes.c_int(), ctypes.c_int(), ctypes.c_int(), ctypes.c_int()
    dp, sk = ctypes.c_double(), ctypes.c_double()
    rc = _C.lib().fg_gemm_plan(M, N, K, cu, ctypes.byref(bm), ctypes.byref(bn), ctypes.byref(dp), ctypes.byref(w),
                               ctypes.byref(sk), ctypes.byref(ch))
    assert rc == 0, _C.lib().fg_last_error()
    return dict(tile=(bm.value, bn.value), dp_us=dp.value, workers=w.value, sk_us=sk.value, streamk=bool(ch.value))


@pytest.mark.parametrize("shape,tile", [
    ((8192, 8192, 8192), (256, 256)),      # the square benchmark product: 4 full rounds of 256 tiles
    ((4096, 11008, 4096), (256, 256)),     # the FFN projection with bias
    ((16384, 6144, 4096), (256, 256)),     # decoder layer: fused QKV projection
    ((16384, 4096, 4096), (256, 256)),     # ... output projection
    ((16384, 22016, 4096), (256, 256)),    # ... gate-up projection
    ((16384, 4096, 11008), (256, 256)),    # ... down projection
    ((2048, 4096, 4096), (256, 128)),      # 128 big tiles would leave half the CUs idle
    ((3072, 3072, 3072), (192, 256)),      # 144 big tiles: 16 x 12 of the 192-row tile use 192 CUs
])
def test_data_parallel_tile_of_large_products(shape, tile):
    p = plan(*shape)
    assert p["tile"] == tile and not p["streamk"] and p["workers"] == 0


@pytest.mark.parametrize("shape", [(512, 4096, 4096), (256, 4096, 4096), (128, 4096, 4096), (1024, 1024, 8192),
                                   (256, 256, 16384)])
def test_few_tiles_and_a_deep_k_take_stream_k(shape):
    p = plan(*shape)
    assert p["streamk"] and 0 < p["workers"] <= 256 and p["sk_us"] < p["dp_us"]


def test_stream_k_needs_four_k_steps_per_cu_and_no_more_tiles_than_cus():
    assert plan(128, 128, 1024)["workers"] == 0      # 16 K steps in all: nothing to share
    assert plan(4096, 4096, 4096)["workers"] == 0    # 1024 tiles of 128 x 128
    assert plan(2048, 2048, 4096)["workers"] > 0     # 256 tiles: exactly one per CU


def test_modelled_duration_is_linear_in_k_and_never_falls_with_more_rows():
    a, b = plan(8192, 8192, 4096), plan(8192, 8192, 8192)
    assert a["tile"] == b["tile"] and b["dp_us"] == pytest.approx(2 * a["dp_us"])
    prev = 0.0
    for m in range(256, 8193, 256):
        d = plan(m, 8192, 4096)["dp_us"]
        assert d >= prev * 0.999, m   # the best tile's duration, so a finer tile may take over but never slower
        prev = d


def test_smaller_devices_choose_smaller_grids():
    # 64 CUs: 2048 x 4096 is already two full rounds of big tiles
    assert plan(2048, 4096, 4096, cu=64)["tile"] == (256, 256)


def test_errors():
    lib = _C.lib()
    assert lib.fg_gemm_plan(0, 8, 64, 256, None, None, None, None, None, None) < 0
    assert lib.fg_gemm_plan(128, 128, 100, 256, None, None, None, None, None, None) < 0
    assert b"multiple of 64" in lib.fg_last_error()
    assert lib.fg_gemm_plan(128, 128, 128, 256, None, None, None, None, None, None) == 0  # every output optional
