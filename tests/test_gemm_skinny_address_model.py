"""Host-side model of the skinny stream-K GEMM kernels (flaggems_amd/csrc/gemm_skinny.hip): the partition of the
(tile, k-step) units over the persistent workgroups, and every global address the two kernels form from it: the A and B
loads of every k-step of every wave (the row-major kernel's guarded loads, the K-contiguous kernel's clamped rows, its
rotated walk over a wave's share and the steps past the end of the share that re-read the last one), the partial
tiles in the workspace, the ticket counters, and the stores of C with the bias loads beside them.

It restates the kernels' index arithmetic with numpy over the lanes of a wave and asserts that the units are covered
exactly once, that a split tile's contributors and slots are the ones its finisher reads, and that every access stays
inside its operand or its share of the workspace (as skinny_workspace_bytes sizes it).  A second statement of the same
arithmetic, not a proof; shapes: the benchmark's 16 x 4096 x 14336 in both B layouts, ragged N, one to 64 rows, and the
host's conditions for taking these kernels (K and N multiples of 8, 16-byte aligned rows)."""
import numpy as np
import pytest

TILE_N, STEP_K, WAVES, BLOCK = 128, 32, 8, 512
TILE_ELEMS = 16 * TILE_N
KC_STEP = 64
MAX_WORKERS = 1024
TICKET_OFF, PARTIAL_OFF = 256, 256 + MAX_WORKERS * 4
LANES = np.arange(64)


def inside(off, width, nbytes, what):
    off = np.asarray(off, dtype=np.int64)
    assert (off >= 0).all() and (off + width <= nbytes).all(), "%s leaves its operand by %d bytes" % (
        what, int(max((off + width).max() - nbytes, -off.min())))


def range_begin(per, rem, w):
    return w * per + min(w, rem)


def worker_of(per, rem, u):
    big = rem * (per + 1)
    return u // (per + 1) if u < big else rem + (u - big) // per


def plan(M, N, K, kc, num_cu=256, force_tile=0):
    kc_tile = 32 if N >= 32 * num_cu else 16
    if force_tile:
        kc_tile = force_tile
    if M > 32:
        kc_tile = 32
    tn = kc_tile if kc else TILE_N
    tiles_n = -(-N // tn)
    ksteps = -(-K // (KC_STEP if kc else STEP_K))
    units = tiles_n * ksteps
    workers = min(units, min(num_cu, MAX_WORKERS))
    return tn, tiles_n, ksteps, workers, units // workers, units % workers


def segments(w, per, rem, ksteps):
    """(tile, ks0, ks1, slot) of workgroup w, in the order it walks them."""
    u, u_begin, u_end = range_begin(per, rem, w), range_begin(per, rem, w), range_begin(per, rem, w + 1)
    while u < u_end:
        tile = u // ksteps
        tb = tile * ksteps
        ks0, ks1 = u - tb, min(u_end, tb + ksteps) - tb
        yield tile, ks0, ks1, (1 if u_begin < tb else 0)
        u = tb + ks1


def check_partition(tiles_n, ksteps, workers, per, rem, tile_elems, ws_bytes):
    seen = np.zeros(tiles_n * ksteps, dtype=np.int64)
    contrib = {}
    for w in range(workers):
        slots = set()
        for tile, ks0, ks1, slot in segments(w, per, rem, ksteps):
            seen[tile * ksteps + ks0:tile * ksteps + ks1] += 1
            if not (ks0 == 0 and ks1 == ksteps):
                assert slot not in slots, "a workgroup writes one partial slot twice"
                slots.add(slot)
                contrib.setdefault(tile, []).append((w, slot))
                off = PARTIAL_OFF + ((w * 2 + slot) * tile_elems) * 4
                assert off + tile_elems * 4 <= ws_bytes, "partial tile outside the workspace"
    assert (seen == 1).all(), "a (tile, k-step) unit is covered %s times" % sorted(set(seen.tolist()))
    for tile, who in contrib.items():
        tb, te = tile * ksteps, tile * ksteps + ksteps
        w_first, w_last = worker_of(per, rem, tb), worker_of(per, rem, te - 1)
        assert 0 <= w_first < MAX_WORKERS
        # the finisher reads, for every workgroup from the first to the last of the tile, the slot that workgroup wrote
        assert [w for w, _ in who] == list(range(w_first, w_last + 1))
        for w2, slot in who:
            assert slot == (1 if range_begin(per, rem, w2) < tb else 0)
        assert len(who) == w_last - w_first + 1 >= 2


def check_store(M, N, n_of_elem, m_of_elem, valid, scm, c_bytes, sim, sin_, bias_bytes):
    ok = valid & (m_of_elem < M) & (n_of_elem < N)
    inside((m_of_elem[ok] * scm + n_of_elem[ok]) * 2, 2, c_bytes, "C store")
    if bias_bytes:
        inside((m_of_elem[ok] * sim + n_of_elem[ok] * sin_) * 2, 2, bias_bytes, "bias load")


def check_rowmajor(M, N, K, b_rowmajor=True, num_cu=256, sam=None, ldb=None, bias=None):
    """gemm_skinny_kernel<T, B_ROWMAJOR>."""
    assert M <= 16 and K % 8 == 0 and K >= 1024
    sam = K if sam is None else sam
    if b_rowmajor:
        assert N % 8 == 0
        sbk, sbn = (N if ldb is None else ldb), 1
        b_bytes = ((K - 1) * sbk + N) * 2
    else:
        sbn, sbk = (K if ldb is None else ldb), 1
        b_bytes = ((N - 1) * sbn + K) * 2
    a_bytes, c_bytes = ((M - 1) * sam + K) * 2, M * N * 2
    tn, tiles_n, ksteps, workers, per, rem = plan(M, N, K, False, num_cu)
    ws_bytes = PARTIAL_OFF + num_cu * 2 * TILE_ELEMS * 4
    check_partition(tiles_n, ksteps, workers, per, rem, TILE_ELEMS, ws_bytes)
    m, grp = LANES & 15, LANES >> 4
    sim, sin_, bias_bytes = (0, 0, 0) if bias is None else bias
    for w in {0, 1, workers // 2, workers - 1}:
        for tile, ks0, ks1, _ in segments(w, per, rem, ksteps):
            n0 = tile * TILE_N
            share = -(-(ks1 - ks0) // WAVES)
            for wave in range(WAVES):
                my0 = ks0 + wave * share
                my1 = min(my0 + share, ks1)
                for ks in range(my0, my1):
                    k0 = ks * STEP_K
                    ka = k0 + grp * 8
                    ok = (m < M) & (ka < K)
                    inside(((m * sam + ka) * 2)[ok], 16, a_bytes, "A load")
                    if b_rowmajor:
                        n = n0 + m * 8
                        for j in range(8):
                            k = k0 + grp * 8 + j
                            okb = (k < K) & (n < N)
                            inside(((k * sbk + n) * 2)[okb], 16, b_bytes, "B load")
                    else:
                        for c in range(8):
                            n = n0 + 16 * c + m
                            okb = (ka < K) & (n < N)
                            inside(((n * sbn + ka) * 2)[okb], 16, b_bytes, "B load")
            # epilogue: element e = tid + 512 j of the tile
            e = np.arange(TILE_ELEMS)
            el, ci = e & 63, e >> 6
            em, eg, c, i = el & 15, el >> 4, ci >> 2, ci & 3
            n = n0 + (8 * (4 * eg + i) + c if b_rowmajor else 16 * c + 4 * eg + i)
            check_store(M, N, n, em, np.ones_like(e, bool), N, c_bytes, sim, sin_, bias_bytes)


def check_kc(M, N, K, num_cu=256, sam=None, ldb=None, force_tile=0, bias=None):
    """gemm_skinny_kc_kernel<T, TN, RING, A_LINES, MB>."""
    assert M <= 64 and K % KC_STEP == 0 and K >= 1024
    sam = K if sam is None else sam
    sbn = K if ldb is None else ldb
    a_bytes, b_bytes, c_bytes = ((M - 1) * sam + K) * 2, ((N - 1) * sbn + K) * 2, M * N * 2
    tn, tiles_n, ksteps, workers, per, rem = plan(M, N, K, True, num_cu, force_tile)
    MB = 4 if M > 32 else (2 if M > 16 else 1)
    a_lines = M > 8
    ring = 4 if tn == 32 else 8
    ndma, nal = tn // 8, 2 * MB
    assert (ndma + nal) * (ring - 1) < 64, "the wait count exceeds the counter"
    tile_elems = 16 * MB * tn
    assert tile_elems <= TILE_ELEMS and tile_elems * 4 <= ring * tn * KC_STEP * 2
    ws_bytes = PARTIAL_OFF + num_cu * 2 * TILE_ELEMS * 4
    check_partition(tiles_n, ksteps, workers, per, rem, tile_elems, ws_bytes)
    m, grp = LANES & 15, LANES >> 4
    sim, sin_, bias_bytes = (0, 0, 0) if bias is None else bias
    for w in {0, 1, workers // 2, workers - 1}:
        for tile, ks0, ks1, _ in segments(w, per, rem, ksteps):
            n0 = tile * tn
            share = -(-(ks1 - ks0) // WAVES)
            for wave in range(WAVES):
                my0 = ks0 + wave * share
                my1 = min(my0 + share, ks1)
                nmine = my1 - my0
                if nmine <= 0:
                    continue
                rot = (w * 13 + wave * 5) % nmine
                # the steps the ring issues: nmine real ones and up to ring - 1 past the end, which re-read the last
                total_issued = nmine + ring - 1
                ksteps_read = set()
                for step in range(total_issued):
                    sidx = min(step, nmine - 1)
                    kidx = sidx + rot
                    kidx = kidx - nmine if kidx >= nmine else kidx
                    assert 0 <= kidx < nmine
                    ksteps_read.add(my0 + kidx)
                assert ksteps_read == set(range(my0, my1)), "the rotated walk misses a k-step of the share"
                for kstep in (my0, my1 - 1):
                    koff = kstep * KC_STEP * 2
                    for i in range(ndma):
                        r = 8 * i + (LANES >> 3)
                        c = (LANES & 7) ^ (r & 7)
                        n = np.minimum(n0 + r, N - 1)
                        # (the kernel biases the pointer by -1024 i and the instruction adds it back)
                        inside((n * sbn + c * 8) * 2 - i * 1024 + i * 1024 + koff, 16, b_bytes, "B copy")
                    for j in range(nal):
                        fr = np.minimum(8 * j + (LANES >> 3) if a_lines else m, M - 1)
                        col = (LANES & 7) if a_lines else 4 * j + grp
                        inside((fr * sam + col * 8) * 2 + koff, 16, a_bytes, "A load")
            e = np.arange(-(-tile_elems // BLOCK) * BLOCK)
            ncb = tn // 16
            el, i, blk = e & 63, (e >> 6) & 3, e >> 8
            cb, rb = blk % ncb, blk // ncb
            em, eg = 16 * rb + (el & 15), el >> 4
            n = n0 + 16 * cb + 4 * eg + i
            check_store(M, N, n, em, e < tile_elems, N, c_bytes, sim, sin_, bias_bytes)


@pytest.mark.parametrize("b_rowmajor", [True, False])
def test_benchmark_shape_row_kernel(b_rowmajor):
    check_rowmajor(16, 4096, 14336, b_rowmajor)


def test_benchmark_shape_kc_kernel_has_nothing_to_fix_up():
    check_kc(16, 4096, 14336)
    tn, tiles_n, ksteps, workers, per, rem = plan(16, 4096, 14336, True)
    assert (tn, tiles_n, workers, rem) == (16, 256, 256, 0) and per == ksteps   # one whole tile per CU


@pytest.mark.parametrize("M", [1, 5, 8, 9, 16])
@pytest.mark.parametrize("N,K", [(520, 2048), (136, 8192), (4096, 4096), (264, 1024), (32000, 4096), (8, 65536)])
def test_row_kernel_shapes(M, N, K):
    check_rowmajor(M, N, K, True)
    check_rowmajor(M, N, K, False)
    check_rowmajor(M, N, K, True, sam=K + 64, ldb=N + 8, bias=(N, 1, M * N * 2))
    check_rowmajor(M, N, K, False, ldb=K + 8, bias=(0, 1, N * 2))


@pytest.mark.parametrize("M", [1, 8, 9, 16, 17, 32, 33, 48, 64])
@pytest.mark.parametrize("N,K", [(520, 2048), (136, 8192), (4096, 4096), (1024, 4096), (4096, 1024), (12288, 4096), (16, 65536)])
def test_kc_kernel_shapes(M, N, K):
    check_kc(M, N, K)
    check_kc(M, N, K, sam=K + 64, ldb=K + 8, bias=(N, 1, M * N * 2))
    check_kc(M, N, K, force_tile=32 if M <= 32 else 0, bias=(0, 1, N * 2))


@pytest.mark.parametrize("num_cu", [1, 3, 104, 256, 304, 1024, 2000])
def test_other_device_sizes(num_cu):
    cu = min(num_cu, MAX_WORKERS)
    check_rowmajor(16, 4096, 14336, True, num_cu=cu)
    check_kc(16, 4096, 14336, num_cu=cu)
    check_kc(64, 1024, 4096, num_cu=cu)


def test_the_model_notices_a_short_operand():
    with pytest.raises(AssertionError, match="leaves its operand"):
        inside(np.array([0, 16]), 16, 31, "probe")
    # a B whose last row is shorter than K by one pack: the last k-step of the last column reads past it
    M, N, K = 16, 136, 2048
    tn, tiles_n, ksteps, workers, per, rem = plan(M, N, K, True)
    with pytest.raises(AssertionError, match="B copy"):
        lanes_r = 8 * (tn // 8 - 1) + (LANES >> 3)
        n = np.minimum((tiles_n - 1) * tn + lanes_r, N - 1)
        inside((n * K + ((LANES & 7) ^ (lanes_r & 7)) * 8) * 2 + (ksteps - 1) * KC_STEP * 2, 16, ((N - 1) * K + K - 8) * 2, "B copy")
