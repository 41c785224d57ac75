"""Host-side model of the global addresses of the two attention kernels that serve the benchmark configurations:
the lean paged prefill kernel (flaggems_amd/csrc/attn_pipe.h) and the single-token kernel with split key ranges
(flaggems_amd/csrc/attn_decode.h), together with the host arithmetic that plans their launches (decode_plan,
decode_range_tiles, the workgroup re-numbering per XCD).

The model restates the kernels' index arithmetic with numpy over all 64 lanes of every wave: query rows, block-table
reads (the windows of page ids a wave keeps in registers, with their clamps), the tile copies of full and partial
tiles, output, log-sum-exp and workspace stores.  It asserts that every access lies inside its operand, that the 32-bit
byte offsets never wrap, that a wave's 16 (or KPI) key rows of one copy never straddle a page, and that every page
index stays inside the register window it is read from.  Like the GEMM model it is a second statement of the same
arithmetic, not a proof: it pins the invariants a change to the addressing must keep, and it runs the variants that
load Q unconditionally (clamped addresses) through the same checks.  Shapes: the paged benchmark configurations, ragged
lengths around tile, page, window and key-range boundaries, every page size the kernels take, and dense K/V presented
as virtual pages (large row strides)."""
import itertools

import numpy as np
import pytest

BN = 64          # keys per tile of the prefill kernel
DEC_TILE = 32    # keys per wave tile of the single-token kernel
LANES = np.arange(64)


def swz(cpr, key):
    key = np.asarray(key)
    if cpr >= 16:
        return ((key & 3) << 2) | (((key >> 3) & 1) << 1) | ((key >> 2) & 1)
    return (((key >> 1) & 1) << 2) | (((key >> 2) & 1) << 1) | ((key >> 3) & 1)


def sampled(items, thin):
    """All of a short list; of a long one the first and last four and every fifth in between (thin=True)."""
    items = list(items)
    if not thin or len(items) <= 24:
        return items
    keep = set(range(4)) | set(range(len(items) - 4, len(items))) | set(range(0, len(items), 5))
    return [x for i, x in enumerate(items) if i in keep]


class Operand:
    """A device allocation at a made-up base: `check(offsets, nbytes)` asserts accesses of nbytes at byte offsets."""

    def __init__(self, name, nbytes, base):
        self.name, self.nbytes, self.base = name, int(nbytes), base

    def check(self, off, width, what=""):
        off = np.asarray(off, dtype=np.int64)
        assert (off >= 0).all(), "%s: %s reaches below the allocation" % (self.name, what)
        assert (off + width <= self.nbytes).all(), "%s: %s reaches %d bytes past the allocation" % (
            self.name, what, int((off + width).max() - self.nbytes))


class Case:
    """A paged (or virtually paged) attention problem in element units, as FgFlashParams describes it."""

    def __init__(self, qlens, klens, Hq, Hk, D, page, num_pages, rng, k_row_stride=None, k_head_stride=None,
                 k_page_stride=None, q_row_stride=None, table=None, max_k=None):
        self.qlens, self.klens = list(qlens), list(klens)
        self.B, self.Hq, self.Hk, self.D, self.page = len(qlens), Hq, Hk, D, page
        self.shift = page.bit_length() - 1
        assert 1 << self.shift == page
        self.cu = np.concatenate([[0], np.cumsum(qlens)]).astype(np.int64)
        self.total_q = int(self.cu[-1])
        self.max_q, self.max_k = max(qlens), (max(klens) if max_k is None else max_k)
        self.k_head_stride = D if k_head_stride is None else k_head_stride
        self.k_row_stride = Hk * D if k_row_stride is None else k_row_stride
        self.k_page_stride = page * self.k_row_stride if k_page_stride is None else k_page_stride
        self.q_row_stride = Hq * D if q_row_stride is None else q_row_stride
        self.q_head_stride = D
        self.table_w = max(1, -(-self.max_k // page))
        if table is None:
            table = rng.integers(0, num_pages, size=(self.B, self.table_w))
        self.table = np.asarray(table, dtype=np.int64)
        self.num_pages = num_pages
        # allocations (bytes): the cache ends with the last row of its last page
        cache_bytes = ((num_pages - 1) * self.k_page_stride + (page - 1) * self.k_row_stride
                       + (Hk - 1) * self.k_head_stride + D) * 2
        self.kc = Operand("k_cache", cache_bytes, 1 << 40)
        self.vc = Operand("v_cache", cache_bytes, 1 << 41)
        self.q = Operand("q", ((self.total_q - 1) * self.q_row_stride + (Hq - 1) * D + D) * 2 if self.total_q else 0, 1 << 42)
        self.out = Operand("out", self.total_q * Hq * D * 2, 1 << 43)
        self.lse = Operand("lse", Hq * self.total_q * 4, 1 << 44)
        self.bt = Operand("block_table", self.B * self.table_w * 4, 1 << 45)


# ----------------------------------------------------------------------------------------------------------------
# the lean prefill kernel
# ----------------------------------------------------------------------------------------------------------------
def check_prefill(c, causal=True, q_uncond=False, skip_single=False, window_left=-1, thin=False):
    D, page, shift = c.D, c.page, c.shift
    assert D in (64, 128) and shift >= 4
    RB = 2 * D
    CPR, KK = RB // 16, D // 32
    KPI = 1024 // RB
    IPW = BN // KPI // 4
    ratio = c.Hq // c.Hk
    hpb = 4 if ratio % 4 == 0 else (2 if ratio % 2 == 0 else 1)
    rows_per_block = 128 // hpb
    gx, gy, gz = -(-c.max_q // rows_per_block), c.B, c.Hq // hpb
    # host: 32-bit byte strides (use_fast conditions)
    for s in (c.k_page_stride, c.k_row_stride * page):
        assert 0 <= s < 1 << 30
    k_page_b, k_row_b = c.k_page_stride * 2, c.k_row_stride * 2
    assert k_page_b < 1 << 32 and KPI * k_row_b >= 1024
    # the XCD re-numbering is a permutation of the grid
    total = gx * gy * gz
    per = total // 8
    lin = np.arange(total)
    idx = np.where(lin < per * 8, (lin % 8) * per + lin // 8, lin)
    assert sorted(idx.tolist()) == list(range(total))
    g_, c_ = LANES >> 4, LANES & 15
    lane_key, lane_pos = LANES // CPR, LANES % CPR
    for b, hgroup, bx in itertools.product(range(gy), sampled(range(gz), thin), sampled(range(gx), thin)):
        m_block = (gx - 1 - bx + b * 5 + hgroup * 3) % gx
        q_bos, q_len, k_len = int(c.cu[b]), c.qlens[b], c.klens[b]
        block_row0 = m_block * rows_per_block
        if block_row0 >= q_len or (skip_single and q_len == 1):
            continue
        shift_qk = k_len - q_len
        n_max = -(-k_len // BN)
        if causal:
            last = block_row0 + rows_per_block + shift_qk
            n_max = min(n_max, 0 if last <= 0 else -(-last // BN))
        n_min = 0
        if window_left >= 0:
            first = block_row0 + shift_qk - window_left
            n_min = 0 if first <= 0 else first // BN
        T_ = max(n_max - n_min, 0)
        last_page = (k_len - 1) >> shift if k_len > 0 else 0
        for wave in range(4):
            wph = 4 // hpb
            head = hgroup * hpb + wave // wph
            row0 = block_row0 + (wave % wph) * 32
            kv_head = head // ratio
            assert 0 <= head < c.Hq and 0 <= kv_head < c.Hk
            # ---- Q: two column tiles of 16 rows, KK loads of 16 bytes per lane
            for qt in range(2):
                qrow = row0 + qt * 16 + c_
                row_ok = qrow < q_len
                rows = q_bos + np.where(row_ok, qrow, 0)
                for kk in range(KK):
                    off = (rows * c.q_row_stride + head * c.q_head_stride + kk * 32 + g_ * 8) * 2
                    c.q.check(off if q_uncond else off[row_ok], 16, "Q fragment")
                # ---- out and lse stores of the rows that exist
                orow = q_bos + qrow[row_ok]
                for dt in range(D // 16):
                    c.out.check((orow[:, None] * c.Hq * D + head * D + dt * 16 + np.arange(4)[None, :] * 4) * 2, 8, "O store")
                c.lse.check((head * c.total_q + orow) * 4, 4, "lse store")
            if T_ == 0:
                continue
            # ---- page-id windows and tile copies
            lane_c0 = (lane_pos ^ swz(CPR, wave * IPW * KPI + lane_key)) * 16
            lane_row = lane_key * k_row_b
            assert (lane_row < 1 << 32).all()
            wave_key0 = wave * IPW * KPI

            def window(first_tile):
                pg0 = ((n_min + first_tile + LANES) * BN + wave_key0) >> shift
                pg1 = ((n_min + first_tile + 64 + LANES) * BN + wave_key0) >> shift
                pg0, pg1 = np.minimum(pg0, last_page), np.minimum(pg1, last_page)
                c.bt.check((b * c.table_w + np.concatenate([pg0, pg1])) * 4, 4, "page-id window")
                return first_tile, np.concatenate([c.table[b, pg0], c.table[b, pg1]])

            pg_base, pg_cache = window(0)
            # the tiles in the order the kernel requests them: K(0), V(0), K(1), then V(t+1) / K(t+2) per step
            order = [0, 0] + ([1] if T_ > 1 else [])
            for t in range(T_):
                if t + 1 < T_:
                    order.append(t + 1)
                if t + 2 < T_:
                    order.append(t + 2)
            # (a thinned walk keeps the tiles around every reload of the window, which happens at tile 128 and then
            # every 127 tiles: where the window stands depends on the walk)
            for t in order if not thin else [t for i, t in enumerate(order) if i < 6 or i + 6 >= len(order) or i % 5 == 0
                                             or (t >= 127 and (t - 128) % 127 in (0, 1, 126))]:
                nb = n_min + t
                if nb * BN + BN <= k_len:
                    if t - pg_base >= 128:
                        pg_base, pg_cache = window(t - 1)
                    tl = t - pg_base
                    assert 0 <= tl < 128, "tile outside the page-id window"
                    pageid = int(pg_cache[tl])
                    first_key = nb * BN + wave_key0
                    assert pageid == c.table[b, first_key >> shift]
                    slot = first_key & (page - 1)
                    assert slot + IPW * KPI <= page, "a wave's key rows straddle a page"
                    assert slot * k_row_b < 1 << 32
                    step_b = KPI * k_row_b - 1024
                    for j in range(IPW):
                        voff = lane_row + (lane_c0 ^ (j * 16))
                        assert (voff < 1 << 32).all() and j * step_b < 1 << 32
                        off = pageid * k_page_b + slot * k_row_b + j * step_b + voff + j * 1024 + kv_head * c.k_head_stride * 2
                        # the row and column the access resolves to
                        want_row = slot + j * KPI + lane_key
                        col = off - (pageid * k_page_b + want_row * k_row_b + kv_head * c.k_head_stride * 2)
                        assert ((col >= 0) & (col + 16 <= RB)).all(), "chunk outside its key row"
                        c.kc.check(off, 16, "K tile copy")
                        c.vc.check(off, 16, "V tile copy")
                else:
                    for j in range(IPW):
                        key = nb * BN + (wave * IPW + j) * KPI + lane_key
                        key = np.minimum(key, k_len - 1)
                        assert (key >= 0).all()
                        c.bt.check((b * c.table_w + (key >> shift)) * 4, 4, "page id of a partial tile")
                        pageid = c.table[b, key >> shift]
                        slot = key & (page - 1)
                        assert (slot * k_row_b + (lane_c0 ^ (j * 16)) < 1 << 32).all()
                        off = pageid * k_page_b + slot * k_row_b + (lane_c0 ^ (j * 16)) + kv_head * c.k_head_stride * 2
                        c.kc.check(off, 16, "K partial-tile copy")
                        c.vc.check(off, 16, "V partial-tile copy")


# ----------------------------------------------------------------------------------------------------------------
# the single-token kernel and its launch plan
# ----------------------------------------------------------------------------------------------------------------
def decode_plan(max_k, shift, batch, Hk, num_cu=256, per_cu=2):
    cdiv = lambda a, b: -(-a // b)  # noqa: E731
    max_k = max(max_k, 1)
    range_cap = min(256 << shift, 4096)
    need = cdiv(max_k, range_cap)
    wgs = batch * Hk
    want = min(cdiv(per_cu * num_cu, max(wgs, 1)), max(max_k // 512, 1))
    s = max(need, want)
    tps = cdiv(cdiv(max_k, DEC_TILE), s)
    tps = (tps + 3) // 4 * 4
    s = cdiv(cdiv(max_k, DEC_TILE), tps)
    return max(s, 1), tps


def range_tiles(tiles_total, splits, tps, min_tiles=16):
    t = -(-tiles_total // splits)
    t = (t + 3) & ~3
    t = max(t, min_tiles)
    return min(t, tps)


def check_decode(c, q_early=False, min_tiles=16, num_cu=256, thin=False):
    D, page, shift = c.D, c.page, c.shift
    assert D in (64, 128) and shift >= 4 and c.Hq // c.Hk <= 32
    RB = 2 * D
    CPR, KS = RB // 16, D // 16
    KPI = 1024 // RB
    NI = DEC_TILE // KPI
    G = c.Hq // c.Hk
    splits, tps = decode_plan(c.max_k, shift, c.B, c.Hk, num_cu)
    assert tps % 4 == 0 and tps * DEC_TILE <= 4096 and splits * tps * DEC_TILE >= c.max_k
    ws = Operand("workspace", splits * c.B * c.Hq * (D + 2) * 4 if splits > 1 else 0, 1 << 46)
    half, ql = LANES >> 5, LANES & 31
    lane_key, lane_pos = LANES // CPR, LANES % CPR
    k_row_b = c.k_row_stride * 2
    covered = {b: 0 for b in range(c.B)}
    for bx, b, kvh in itertools.product(range(splits), range(c.B), sampled(range(c.Hk), thin)):
        split = (bx + b * 5 + kvh * 3) % splits
        q_bos, q_len, k_len = int(c.cu[b]), c.qlens[b], c.klens[b]
        assert k_len <= c.max_k
        tiles_total = -(-k_len // DEC_TILE)
        rt = range_tiles(tiles_total, splits, tps, min_tiles)
        t_begin = split * rt
        t_end = min(t_begin + rt, tiles_total)
        if q_len != 1:
            continue
        if split > 0 and t_begin >= t_end:
            continue
        has_work = t_begin < t_end
        if kvh == 0:
            covered[b] += max(t_end - t_begin, 0)
        last_page = (k_len - 1) >> shift if k_len > 0 else 0
        pg_first = (t_begin * DEC_TILE) >> shift
        # ---- Q: row q_bos, head kvh*G + ql (clamped to the group's first head for the rows without one)
        row_ok = ql < G
        for ks in range(KS):
            off = (q_bos * c.q_row_stride + (kvh * G + np.where(row_ok, ql, 0)) * c.q_head_stride + ks * 16 + half * 8) * 2
            c.q.check(off if q_early else off[row_ok], 16, "Q fragment")
        if has_work:
            pg = np.minimum(pg_first + np.arange(4)[:, None] * 64 + LANES[None, :], last_page)
            c.bt.check((b * c.table_w + pg) * 4, 4, "page ids of the range")
            c.bt.check(np.array([(b * c.table_w + last_page) * 4]), 4, "last page id")
            pgc = c.table[b, pg].reshape(-1)
            last_row = (int(c.table[b, last_page]) * c.k_page_stride + ((k_len - 1) & (page - 1)) * c.k_row_stride) * 2
            for t in sampled(range(t_begin, t_end), thin):
                full = t * DEC_TILE + DEC_TILE <= k_len
                for j in range(NI):
                    key = t * DEC_TILE + j * KPI
                    pi = (key >> shift) - pg_first
                    valid = key + lane_key < k_len
                    if valid.any():
                        assert 0 <= pi < 256, "page index outside the 256-entry register window"
                        pageid = int(pgc[pi])
                        assert pageid == c.table[b, key >> shift]
                        slot = key & (page - 1)
                        assert slot + KPI <= page, "the key rows of one copy straddle a page"
                        c16 = (lane_pos ^ swz(CPR, j * KPI + lane_key)) * 16
                        assert ((c16 >= 0) & (c16 + 16 <= RB)).all()
                        assert (lane_key * k_row_b + c16 < 1 << 32).all()
                        off = (pageid * c.k_page_stride + slot * c.k_row_stride + kvh * c.k_head_stride) * 2 + lane_key * k_row_b + c16
                        sel = np.ones(64, bool) if full else valid
                        c.kc.check(off[sel], 16, "K tile copy")
                        c.vc.check(off[sel], 16, "V tile copy")
                    if not full:
                        c16 = (lane_pos ^ swz(CPR, j * KPI + lane_key)) * 16
                        off = last_row + kvh * c.k_head_stride * 2 + c16[~valid]
                        c.kc.check(off, 16, "K copy of the clamped last key")
                        c.vc.check(off, 16, "V copy of the clamped last key")
        # ---- results: out / lse, or the partial rows of the range
        heads = kvh * G + np.arange(G)
        if splits == 1:
            c.out.check(((q_bos * c.Hq + heads[:, None]) * D + np.arange(D)[None, :]) * 2, 2, "out store")
            c.lse.check((heads * c.total_q + q_bos) * 4, 4, "lse store")
        else:
            row = (split * c.B + b) * c.Hq + heads
            ws.check((row[:, None] * D + np.arange(D)[None, :]) * 4, 4, "partial out")
            ml0 = splits * c.B * c.Hq * D
            ws.check((ml0 + row * 2) * 4, 8, "partial (max, sum)")
    for b in range(c.B):
        if c.qlens[b] == 1:
            assert covered[b] == -(-c.klens[b] // DEC_TILE), "the key ranges of sequence %d do not cover its tiles" % b
    # ---- the merge kernel reads exactly the ranges that were written
    if splits > 1:
        for b in range(c.B):
            if c.qlens[b] != 1:
                continue
            tiles_total = -(-c.klens[b] // DEC_TILE)
            rt = range_tiles(tiles_total, splits, tps, min_tiles)
            ns = min(max(-(-tiles_total // rt), 1), splits)
            written = {s for s in range(splits) if s == 0 or s * rt < tiles_total}
            assert set(range(ns)) <= written


# ----------------------------------------------------------------------------------------------------------------
RNG = np.random.default_rng(0)
C4_LENS = [2641, 2501, 1405, 3002, 2670, 3056, 3789, 615, 2919, 1190, 3688, 538, 1358, 3566, 1260, 1648]


@pytest.mark.parametrize("q_uncond", [False, True])
def test_prefill_benchmark_shapes(q_uncond):
    # the GQA prefill configuration (16 sequences, 32 / 8 heads, head dim 128, pages of 16), two of its sequences
    c = Case(C4_LENS[6:8], C4_LENS[6:8], 32, 8, 128, 16, 1 << 12, RNG)
    check_prefill(c, q_uncond=q_uncond, thin=True)
    # the decoder layer's attention: 32 / 32 heads, 2048 tokens
    check_prefill(Case([2048], [2048], 32, 32, 128, 16, 256, RNG), q_uncond=q_uncond, thin=True)


@pytest.mark.parametrize("D,page", [(128, 16), (128, 32), (128, 256), (64, 16), (64, 64), (64, 128)])
@pytest.mark.parametrize("Hq,Hk", [(8, 2), (4, 4), (6, 2), (3, 1)])
def test_prefill_ragged_lengths(D, page, Hq, Hk):
    lens = [(1, 1328), (5, 18), (129, 463), (70, 70), (64, 64), (1, 1), (33, 8193), (130, 129), (3, 0)]
    c = Case([a for a, _ in lens], [b for _, b in lens], Hq, Hk, D, page, 700, RNG)
    check_prefill(c, q_uncond=True)   # (the unconditional Q loads touch a superset of the addresses of the checked ones)
    if (Hq, Hk) == (8, 2):
        check_prefill(c)
        check_prefill(c, causal=False)
        check_prefill(c, window_left=100)
        check_prefill(c, skip_single=True)


def test_prefill_page_window_is_reloaded_past_8192_keys():
    c = Case([40, 600, 3], [9000, 17000, 8193], 4, 2, 128, 16, 2048, RNG)
    check_prefill(c, thin=True)
    check_prefill(Case([257, 64], [12345, 64], 8, 8, 64, 128, 128, RNG), q_uncond=True, thin=True)


def test_prefill_dense_kv_as_virtual_pages():
    # (batch, heads, seq, d) K/V: row stride d, head stride seq*d, pages of 64 rows, page stride 64 rows, the last
    # batch ends with the allocation; and (batch, seq, heads, d): row stride heads*d
    B, H, S, D = 3, 8, 320, 64
    page, ppb = 64, 5
    table = np.arange(B)[:, None] * ppb + np.arange(ppb)[None, :]
    c = Case([S] * B, [S] * B, H, H, D, page, B * ppb, RNG, k_row_stride=D, k_head_stride=S * D, k_page_stride=page * D,
             q_row_stride=H * D, table=table)
    # the allocation really ends with the last row of the last head
    c.kc.nbytes = c.vc.nbytes = B * H * S * D * 2
    check_prefill(c)
    c2 = Case([17] * 4, [1040] * 4, 8, 2, 128, 16, 4 * 65, RNG, k_row_stride=2 * 128, k_head_stride=128,
              k_page_stride=16 * 2 * 128, table=np.arange(4)[:, None] * 65 + np.arange(65)[None, :])
    c2.kc.nbytes = c2.vc.nbytes = 4 * 1040 * 2 * 128 * 2
    check_prefill(c2, causal=False)
    check_prefill(c2, q_uncond=True)


@pytest.mark.parametrize("q_early", [False, True])
@pytest.mark.parametrize("D,page", [(128, 16), (128, 32), (128, 256), (64, 16), (64, 128)])
def test_decode_ragged_batches(D, page, q_early):
    klens = [1, 17, 32, 33, 0, 1000, 4095, 4097]
    check_decode(Case([1] * len(klens), klens, 32, 8, D, page, 1024, RNG), q_early=q_early)
    check_decode(Case([1], [9001], 32, 8, D, page, 1024, RNG), q_early=q_early)
    many = [100 + 37 * i for i in range(70)]
    check_decode(Case([1] * 70, many, 8, 2, D, page, 1024, RNG), q_early=q_early)
    # the reference's single-token grid
    check_decode(Case([1, 1, 1], [1328, 18, 463], 8, 2, D, page, 2048, RNG), q_early=q_early)


@pytest.mark.parametrize("max_k,min_tiles", [(4096, 16), (32768, 4), (32768, 64), (131072, 16)])
def test_decode_max_seqlen_k_above_the_lengths(max_k, min_tiles):
    klens = [2048, 1, 0, 31, 129, 511, 513, 2047, 2049, 3000, 4096, 640] + [700 + 61 * i for i in range(24)]
    c = Case([1] * len(klens), klens, 32, 8, 128, 16, 1024, RNG, max_k=max_k)
    check_decode(c, min_tiles=min_tiles, thin=True)
    long = Case([1] * 9, klens[:8] + [min(max_k, 32768)], 32, 8, 128, 16, 4096, RNG, max_k=max_k)
    check_decode(long, min_tiles=min_tiles, thin=True)


def test_decode_mixed_batch_and_benchmark_shape():
    # a mixed batch: the single-token kernel runs for the whole batch and leaves the longer queries alone
    c = Case([1, 512, 1, 1, 300], [3000, 512, 2000, 4000, 900], 32, 8, 128, 16, 1024, RNG)
    check_decode(c)
    check_prefill(c, skip_single=True)
    # 64 sequences x 4096 keys, 32 / 8 heads (the single-token benchmark workload)
    check_decode(Case([1] * 64, [4096] * 64, 32, 8, 128, 16, 64 * 256, RNG), thin=True)


def test_decode_plan_keeps_every_range_inside_the_register_window():
    for shift, batch, Hk, max_k in itertools.product((4, 5, 6, 8), (1, 3, 64, 256), (1, 8), list(range(1, 9000, 97)) + [
            4095, 4096, 4097, 8191, 8192, 8193, 32768, 131072, 1 << 20]):
        splits, tps = decode_plan(max_k, shift, batch, Hk)
        assert tps % 4 == 0 and 4 <= tps <= 128 and splits >= 1
        assert splits * tps * DEC_TILE >= max_k
        # pages one range can touch: its keys, plus one page when the range starts inside a page
        pages = (tps * DEC_TILE + (1 << shift) - 1) // (1 << shift) + (1 if (tps * DEC_TILE) % (1 << shift) else 0)
        assert pages <= 256


def test_the_model_notices_a_page_outside_the_cache_and_a_short_allocation():
    table = np.zeros((1, 13), dtype=np.int64)
    table[0, 7] = 64                                   # a page id one past the cache
    with pytest.raises(AssertionError, match="past the allocation"):
        check_prefill(Case([200], [200], 8, 2, 128, 16, 64, RNG, table=table))
    with pytest.raises(AssertionError, match="past the allocation"):
        check_decode(Case([1], [200], 8, 2, 128, 16, 64, RNG, table=table))
    c = Case([200], [200], 8, 2, 128, 16, 64, RNG, table=np.full((1, 13), 63))
    check_prefill(c)
    c.kc.nbytes -= 16                                   # the last chunk of the last row of the last page is read
    with pytest.raises(AssertionError, match="k_cache"):
        check_prefill(c)
    c = Case([200], [200], 8, 2, 128, 16, 64, RNG)
    c.q.nbytes -= 2                                     # ... and so is the last element of q
    with pytest.raises(AssertionError, match="Q fragment"):
        check_prefill(c)
