"""The order in which the GEMM kernels walk their grid of workgroup tiles (tile_coords, flaggems_amd/csrc/gemm_tile.h),
through the host-only entry fg_gemm_tile_order, which calls the function the kernels call.  A tile that no workgroup
computes is a hole in the output and a tile computed twice means another one is missing, so the map must be a
bijection on every grid; on the grids the L2-sharing layout applies to, the 32 workgroups an XCD runs together must
form one 8 x 4 sub-block."""
import ctypes

import numpy as np
import pytest

from flaggems_amd import _C


def order(tiles_m, tiles_n, b_kc):
    n = tiles_m * tiles_n
    tm = (ctypes.c_int * n)()
    tn = (ctypes.c_int * n)()
    assert _C.lib().fg_gemm_tile_order(tiles_m, tiles_n, int(b_kc), tm, tn) == 0, _C.lib().fg_last_error()
    return np.frombuffer(tm, dtype=np.int32).copy(), np.frombuffer(tn, dtype=np.int32).copy()


@pytest.mark.parametrize("b_kc", [True, False])
def test_every_tile_is_visited_exactly_once_on_every_grid(b_kc):
    for tiles_m in list(range(1, 41)) + [48, 56, 64, 72, 96, 128]:
        for tiles_n in list(range(1, 41)) + [44, 48, 64, 86, 172]:
            tm, tn = order(tiles_m, tiles_n, b_kc)
            assert tm.min() >= 0 and tm.max() < tiles_m and tn.min() >= 0 and tn.max() < tiles_n, (tiles_m, tiles_n)
            seen = np.zeros((tiles_m, tiles_n), np.int32)
            np.add.at(seen, (tm, tn), 1)
            assert (seen == 1).all(), (tiles_m, tiles_n)


@pytest.mark.parametrize("b_kc", [True, False])
@pytest.mark.parametrize("grid", [(32, 32), (64, 16), (16, 44), (64, 86 * 2), (8, 4), (24, 12), (40, 20)])
def test_an_xcd_round_is_one_sub_block_of_8_by_4_tiles(grid, b_kc):
    tiles_m, tiles_n = grid
    tm, tn = order(tiles_m, tiles_n, b_kc)
    ids = np.arange(tiles_m * tiles_n)
    xcd, turn = ids % 8, ids // 8
    full_rounds = (tiles_m // 8) * (tiles_n // 4) // 8   # rounds in which every XCD has a sub-block of its own
    for x in range(8):
        for rnd in range(full_rounds):
            sel = (xcd == x) & (turn // 32 == rnd)
            assert sel.sum() == 32
            assert len(set(tm[sel] // 8)) == 1 and len(set(tn[sel] // 4)) == 1, (grid, x, rnd)
    # what is left over (fewer than 8 sub-blocks) is split evenly: every XCD still gets the same number of tiles
    counts = np.bincount(xcd, minlength=8)
    assert counts.max() - counts.min() == 0


def test_consecutive_rounds_share_operand_panels():
    """On 64 x 16 tiles with B = W^T (the decoder layer's down projection) a round of the chip (8 sub-blocks) spans 16
    tile rows, not all 64: A is streamed once, not once per round."""
    tm, tn = order(64, 16, True)
    for rnd in range(4):
        rows = set(tm[rnd * 256:(rnd + 1) * 256] // 8)
        assert len(rows) == 2, rows


def test_errors():
    lib = _C.lib()
    one = (ctypes.c_int * 1)()
    assert lib.fg_gemm_tile_order(0, 4, 1, one, one) < 0
    assert lib.fg_gemm_tile_order(1, 1, 1, None, one) < 0
    assert lib.fg_gemm_tile_order(1, 1, 1, one, one) == 0 and one[0] == 0
