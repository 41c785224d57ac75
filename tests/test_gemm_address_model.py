"""Host-side model of every global address the direct-to-LDS GEMM kernels generate (flaggems_amd/csrc/gemm_dma.h):
the tile copies of every K step, prologue and peeled steps included, the zero-padded last K step of a ragged K, and
the epilogue's stores and bias loads.  The model restates the kernel's address arithmetic (lane offsets, scalar
bases biased by 3072 bytes, instruction immediates, row clamps) with numpy over all lanes and asserts that every
16-byte access stays inside its operand, for the shapes the parity tests run on the GPU and for the batched shape
(32 x 2048 x 2048 x 128, one launch per matrix) whose GPU run once ended in a memory fault that was never explained.
It cannot prove the kernel correct (it is a second statement of the same arithmetic), but it pins the invariants a
change to the offsets must keep: 32-bit lane offsets never wrap, clamped rows stay inside, nothing is read past K."""
import itertools

import numpy as np
import pytest

ROWB, BK = 128, 64  # bytes of K per stage row, K step


def _tile_copy_addresses(M, N, K, sam, sbk, sbn, bm, bn, ns, tm, tn, a_base, b_base, zeros_base):
    """Yield (operand, byte address array [lanes], valid mask) for every copy instruction of tile (tm, tn)."""
    b_kc = sbk == 1
    nk = -(-K // BK)
    ragged = K % BK
    na, nb = bm // 32, bn // 32
    rbb = bn * 2
    cprb, rpi = rbb // 16, 1024 // rbb
    lane = np.arange(64)
    row0, col0 = tm * bm, tn * bn
    b_step = ROWB if b_kc else sbk * BK * 2
    for wave in range(4):
        for j in range(na):
            r = (wave * na + j) * 8 + (lane >> 3)
            c = (lane & 7) ^ ((r >> 1) & 7)
            ra = np.minimum(row0 + r, M - 1) - row0
            off = (ra * sam + c * 8) * 2 + 3072 - (j & 3) * 1024
            assert (off >= 0).all() and (off < 2 ** 32).all()
            sbase = a_base + row0 * sam * 2 - 3072
            for kk in range(nk):
                valid = np.ones(64, bool) if not (ragged and kk == nk - 1) else (c * 8 < ragged)
                addr = np.where(valid, sbase + kk * ROWB + off + (j & 3) * 1024, zeros_base + (j & 3) * 1024)
                yield "A", addr, valid
        for j in range(nb):
            if b_kc:
                r = (wave * nb + j) * 8 + (lane >> 3)
                c = (lane & 7) ^ ((r >> 1) & 7)
                rb = np.minimum(col0 + r, N - 1) - col0
                off = (rb * sbn + c * 8) * 2 + 3072 - (j & 3) * 1024
                sbase = b_base + row0 * 0 + col0 * sbn * 2 - 3072
                lane_valid = (c * 8 < ragged) if ragged else None
            else:
                k = (wave * nb + j) * rpi + lane // cprb
                c = (lane % cprb) ^ (((k & 3) << 2) | (((k >> 3) & 1) << 1))
                cb = col0 + c * 8
                cb = np.where(cb + 8 <= N, cb, N - 8) - col0
                off = (k * sbk + cb) * 2 + 3072 - (j & 3) * 1024
                sbase = b_base + col0 * 2 - 3072
                lane_valid = (k < ragged) if ragged else None
            assert (off >= 0).all() and (off < 2 ** 32).all()
            for kk in range(nk):
                valid = np.ones(64, bool) if not (ragged and kk == nk - 1) else lane_valid
                addr = np.where(valid, sbase + kk * b_step + off + (j & 3) * 1024, zeros_base + (j & 3) * 1024)
                yield "B", addr, valid


def _check_problem(M, N, K, b_kc, bm, bn, ns, sam=None, ldb=None):
    sam = K if sam is None else sam
    if b_kc:
        sbn, sbk = (K if ldb is None else ldb), 1
        b_extent = ((N - 1) * sbn + K) * 2
    else:
        sbk, sbn = (N if ldb is None else ldb), 1
        b_extent = ((K - 1) * sbk + N) * 2
    a_extent = ((M - 1) * sam + K) * 2
    a_base, b_base, zeros = 1 << 40, 1 << 41, 1 << 42
    tiles_m, tiles_n = -(-M // bm), -(-N // bn)
    corner = {(0, 0), (tiles_m - 1, 0), (0, tiles_n - 1), (tiles_m - 1, tiles_n - 1), (tiles_m // 2, tiles_n // 2)}
    for tm, tn in corner:
        for op, addr, valid in _tile_copy_addresses(M, N, K, sam, sbk, sbn, bm, bn, ns, tm, tn, a_base, b_base, zeros):
            base, extent = (a_base, a_extent) if op == "A" else (b_base, b_extent)
            v = addr[valid]
            assert (v >= base).all() and (v + 16 <= base + extent).all(), (op, tm, tn, M, N, K)
            z = addr[~valid]
            assert (z >= zeros).all() and (z + 16 <= zeros + 4096).all()
    # epilogue: lane (r = lane % 16, g = lane / 16) of sub-tile pair (i, jp) stores 16 bytes at row 16 i + r,
    # column (2 jp + (g & 1)) * 16 + (g & 2) * 4 of its wave tile, when row < M and column < N (N % 8 == 0)
    lane = np.arange(64)
    lr, lg = lane & 15, lane >> 4
    for (tm, tn), wave in itertools.product(corner, range(4)):
        wm, wn = wave >> 1, wave & 1
        for i in range(bm // 32):
            r = tm * bm + wm * (bm // 2) + i * 16 + lr
            for jp in range(bn // 64):
                c = tn * bn + wn * (bn // 2) + (2 * jp + (lg & 1)) * 16 + (lg & 2) * 4
                ok = (r < M) & (c < N)
                assert (c[ok] + 8 <= N).all()


DMA_TILES = [(256, 256, 2), (192, 256, 2), (256, 128, 3), (128, 256, 3), (128, 128, 4)]


@pytest.mark.parametrize("b_kc", [False, True])
@pytest.mark.parametrize("bm,bn,ns", DMA_TILES)
def test_tile_copies_stay_inside_their_operands(bm, bn, ns, b_kc):
    for M, N, K in [(1024, 4096, 128), (1100, 4104, 64), (2040, 4104, 256), (1537, 2824, 192), (1100, 2824, 1088),
                    (2048, 2048, 128), (1, 8, 64), (255, 264, 4096), (8192, 8192, 8192), (4096, 11008, 4096)]:
        _check_problem(M, N, K, b_kc, bm, bn, ns)
    # padded leading dimensions, and the largest the host admits (tile-local offsets just below 4 GiB)
    _check_problem(3000, 4104, 1024, b_kc, bm, bn, ns, sam=1024 + 64, ldb=(1024 if b_kc else 4104) + 24)
    _check_problem(300, 520, 256, b_kc, bm, bn, ns, sam=(1 << 22) + 8)


@pytest.mark.parametrize("b_kc", [False, True])
@pytest.mark.parametrize("bm,bn,ns", [(256, 256, 2), (128, 128, 4)])
def test_ragged_last_k_step_reads_zeros_past_k(bm, bn, ns, b_kc):
    for M, N, K in [(300, 520, 72), (1100, 2824, 136), (2040, 1032, 1000), (513, 4104, 2744), (4100, 4104, 200)]:
        _check_problem(M, N, K, b_kc, bm, bn, ns)


@pytest.mark.parametrize("b_kc", [False, True])
def test_batched_attention_sized_matrices_one_launch_each(b_kc):
    """32 matrices of 2048 x 2048 x 128, bases 2048*128*2 (A, B) bytes apart: every launch of the per-matrix loop
    on its own pointers, on both tiles the host can pick for it."""
    for bm, bn, ns in [(256, 256, 2), (128, 128, 4)]:
        _check_problem(2048, 2048, 128, b_kc, bm, bn, ns)
