"""Host-side model of the copy / wait / barrier schedule of the direct-to-LDS GEMM main loop
(dma_tile_mainloop, flaggems_amd/csrc/gemm_dma.h): which copy instruction is issued in which quarter of which K step
into which LDS stage, how many copies each wait leaves in flight, and where the barriers stand.  It restates the
loop's control flow (prologue, steady state, the peeled last steps) as a list of events of one wave and asserts what
the kernel relies on, for every stage count, every split of a step's copies over the quarters and K lengths of
1 ... 40 steps:
  * every copy of every K step below nk is issued exactly once, none for a step at or past nk;
  * read after write: when a stage is first read for step k, all copies of step k had landed (by this wave's wait
    counts, copies retiring in issue order) before the last barrier (so every wave's copies had);
  * write after read: no copy is issued into a stage that was read, for an earlier step, since the last barrier;
  * the copies in flight never exceed what the 6-bit counter can express.
The split constants are taken from the header, so a change there is checked here before it reaches a GPU.  Like the
address model, this is a second statement of the same schedule: it guards the invariants, not the code generation.
"""
import os
import re

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HEADER = os.path.join(ROOT, "flaggems_amd", "csrc", "gemm_dma.h")


def program(nk, ns, ndma, c3, c0, c1):
    """Events of one wave in program order: ('dma', step, j, stage) | ('wait', copies left in flight) |
    ('barrier',) | ('read', stage, step)."""
    assert c3 + c0 + c1 == ndma
    ev = []

    def issue(step, j):
        ev.append(("dma", step, j, step % ns))

    for s in range(ns - 1):  # prologue: whole steps 0 .. ns-2, then the quarter-3 part of step ns-1
        if s < nk:
            for j in range(ndma):
                issue(s, j)
    if nk >= ns:
        for j in range(c3):
            issue(ns - 1, j)
        ev.append(("wait", ndma * (ns - 2) + c3))
    else:
        ev.append(("wait", 0))
    ev.append(("barrier",))
    ev.append(("read", 0, 0))

    def k_step(kb, tail, head, later):
        for qt in range(4):
            nxt = kb + (1 if qt == 3 else 0)  # quarter 3 already reads the next step's first fragments
            ev.append(("read", nxt % ns, nxt))
            if qt == 0 and tail:
                for j in range(c3, c3 + c0):
                    issue(kb + ns - 1, j)
            if qt == 1 and tail:
                for j in range(c3 + c0, ndma):
                    issue(kb + ns - 1, j)
            if qt == 3 and head:
                for j in range(c3):
                    issue(kb + ns, j)
            if qt == 2:
                ev.append(("wait", later))
                ev.append(("barrier",))

    kb = 0
    while kb + ns <= nk - ns:
        for s in range(ns):
            k_step(kb + s, 1, 1, ndma * (ns - 2))
        kb += ns
    for _ in range(ns - 1):
        if kb < nk - ns:
            k_step(kb, 1, 1, ndma * (ns - 2))
            kb += 1
    for ic in range(ns - 1):
        r = ns - 1 - ic
        if kb == nk - 1 - r:
            k_step(kb, 1 if r >= ns - 1 else 0, 0, ndma * min(ns - 2, r - 1))
            kb += 1
    k_step(kb, 0, 0, 0)
    return ev


def violations(nk, ns, ndma, c3, c0, c1, events=None):
    ev = program(nk, ns, ndma, c3, c0, c1) if events is None else events
    issued, order = {}, []
    landed = 0           # copies, in issue order, known complete by this wave's waits
    landed_at_barrier = 0
    read_since_barrier = {}  # stage -> step it was read for
    errs, max_in_flight = [], 0
    for e in ev:
        if e[0] == "dma":
            _, step, j, st = e
            if step >= nk:
                errs.append(("copy for a step past the end", step, j))
            if (step, j) in issued:
                errs.append(("issued twice", step, j))
            issued[(step, j)] = len(order)
            order.append((step, j))
            if st in read_since_barrier and read_since_barrier[st] != step:
                errs.append(("overwrites a stage still being read", step, j, st))
            max_in_flight = max(max_in_flight, len(order) - landed)
        elif e[0] == "wait":
            landed = max(landed, len(order) - e[1])
        elif e[0] == "barrier":
            read_since_barrier = {}
            landed_at_barrier = landed
        else:
            _, st, step = e
            if step < nk:  # the fragments read past the last step are never used
                for j in range(ndma):
                    if (step, j) not in issued or issued[(step, j)] >= landed_at_barrier:
                        errs.append(("reads a stage before its copies landed", step, j))
                        break
                read_since_barrier[st] = step
    for s in range(nk):
        for j in range(ndma):
            if (s, j) not in issued:
                errs.append(("never issued", s, j))
    if max_in_flight > 63:
        errs.append(("more copies in flight than the counter holds", max_in_flight))
    return errs


def header_splits():
    """(stages, copies per step, [(c3, c0, c1), ...]): every split the header can select for a tile it instantiates."""
    src = open(HEADER).read()
    q3 = re.search(r"constexpr int dma_split_q3\(int ndma, bool b_kc\) \{ return ndma == 16 \? \(b_kc \? (\d+) : (\d+)\) : "
                   r"ndma == 14 \? (\d+) : ndma == 12 \? (\d+) : (\d+); \}", src)
    q0 = re.search(r"constexpr int dma_split_q0\(int ndma\) \{ return ndma == 16 \? (\d+) : ndma == 14 \? (\d+) : "
                   r"ndma == 12 \? (\d+) : (\d+); \}", src)
    assert q3 and q0, "the copy split of dma_tile_mainloop is no longer written the way this test reads it"
    assert "constexpr int C3 = THREE_RUNS ? dma_split_q3(NDMA, B_KC) : NDMA / 2;" in src
    assert "constexpr int C0 = THREE_RUNS ? dma_split_q0(NDMA) : NDMA - C3;" in src
    assert "constexpr int C1 = NDMA - C3 - C0;" in src
    a, b, c14, c12, c8 = (int(x) for x in q3.groups())
    z16, z14, z12, z8 = (int(x) for x in q0.groups())
    three = {16: [(a, z16), (b, z16)], 14: [(c14, z14)], 12: [(c12, z12)], 8: [(c8, z8)]}
    # tiles and stage counts the launcher instantiates: copies per wave and step = (BM + BN) / 32
    tiles = [(256, 256, 2), (192, 256, 2), (256, 128, 3), (128, 256, 3), (128, 128, 4), (128, 128, 2)]
    out = []
    for bm, bn, ns in tiles:
        ndma = (bm + bn) // 32
        splits = [(ndma // 2, ndma - ndma // 2, 0)] + [(c3, c0, ndma - c3 - c0) for c3, c0 in three[ndma]]
        out.append((ns, ndma, splits))
    return out


@pytest.mark.parametrize("ns,ndma,splits", header_splits())
def test_schedule_invariants_hold_for_every_k_length(ns, ndma, splits):
    for c3, c0, c1 in splits:
        assert c0 > 0 and c1 >= 0
        for nk in range(1, 41):
            assert violations(nk, ns, ndma, c3, c0, c1) == [], (ns, ndma, (c3, c0, c1), nk)


def test_three_quarter_splits_generalise():
    """Splits the header does not use today, for the other stage counts: the control flow does not depend on them."""
    for ns, ndma, split in ((3, 12, (5, 4, 3)), (3, 12, (6, 4, 2)), (4, 8, (3, 3, 2)), (4, 8, (4, 3, 1)), (2, 14, (5, 4, 5))):
        for nk in range(1, 41):
            assert violations(nk, ns, ndma, *split) == []


def test_the_model_sees_a_broken_schedule():
    """Known-bad schedules must trip: a wait that leaves too many copies in flight, a missing barrier, a refill
    issued one quarter early (while its stage is still being read), a copy issued twice."""
    ns, ndma, c3, c0, c1 = 2, 16, 8, 8, 0
    good = program(8, ns, ndma, c3, c0, c1)
    assert violations(8, ns, ndma, c3, c0, c1, good) == []
    # 1. the wait of some step admits one copy more than it may
    i = [k for k, e in enumerate(good) if e[0] == "wait"][3]
    bad = list(good)
    bad[i] = ("wait", good[i][1] + 1)
    assert any(v[0].startswith("reads a stage before") for v in violations(8, ns, ndma, c3, c0, c1, bad))
    # 2. a barrier dropped: the next refill lands in a stage another wave may still read
    i = [k for k, e in enumerate(good) if e[0] == "barrier"][2]
    bad = good[:i] + good[i + 1:]
    assert any(v[0].startswith("overwrites") for v in violations(8, ns, ndma, c3, c0, c1, bad))
    # 3. the quarter-3 refill moved in front of quarter 2's barrier
    i = [k for k, e in enumerate(good) if e[0] == "barrier"][2]
    j = next(k for k in range(i, len(good)) if good[k][0] == "dma")
    bad = good[:i] + [good[j]] + good[i:j] + good[j + 1:]
    assert any(v[0].startswith("overwrites") for v in violations(8, ns, ndma, c3, c0, c1, bad))
    # 4. a copy issued twice, and so another one never
    j = [k for k, e in enumerate(good) if e[0] == "dma"][40]
    bad = list(good)
    bad[j + 1] = good[j]
    got = {v[0] for v in violations(8, ns, ndma, c3, c0, c1, bad)}
    assert "issued twice" in got and "never issued" in got
