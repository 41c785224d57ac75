"""Checks of the device assembly that the library's build runs on every HIP source: wait states around instructions
issued from inline asm, LDS reads issued from asm against the LDS counter, and no packed fp32 arithmetic.

gfx9 leaves these data hazards to software:
  * a vector instruction writes a scalar register (v_readfirstlane, v_readlane, a v_cmp with a scalar destination)
    and a vector-memory instruction reads that register: 5 wait states must lie between them;
  * a scalar instruction writes M0 and an LDS-direct load (global_load_lds_*, buffer_load_* ... lds) follows:
    1 wait state;
  * a matrix instruction writes its accumulator and an instruction other than a matrix instruction reads or
    writes one of those registers: number of passes + 3 wait states (4 passes for the 16x16x32 forms, 8 for
    32x32x16; the scan asks for 11).  Matrix instructions chained through the same accumulator are interlocked.
The compiler's hazard recognizer inserts s_nop for the instructions it selects itself, and recognizes the
producers by their opcode: a memory or matrix instruction written as asm is invisible to it on either side.  An asm statement
is opaque to it, so for the copies written as asm (gemm_dma.h, attn_pipe.h) the distance between, say, a
v_readfirstlane that produces a base address and the copy that reads it is whatever the scheduler happened to
leave: a copy issued too early takes the register's previous contents as its address.  build.py keeps the device
assembly of those sources and fails the build when this scan finds such a pair.

A fourth check (scan_lds_reads, further down) follows the LDS counter through the control-flow graph and reports uses
of a register whose LDS read, issued from asm with a hand-counted wait, may not have returned.

The scan of the three hazards above is textual: it walks each kernel's instructions in program order, counts every instruction as one wait
state (s_nop N as N + 1) and ignores control flow, which errs on the side of reporting (a pair split by a label
is still reported).
"""
import re
import sys

VALU_SGPR_TO_VMEM_WAIT = 5
M0_TO_LDS_DIRECT_WAIT = 1
MFMA_TO_OTHER_WAIT = 11

_VMEM_PREFIXES = ("global_load", "global_store", "global_atomic", "buffer_load", "buffer_store", "buffer_atomic",
                  "flat_load", "flat_store", "flat_atomic", "scratch_load", "scratch_store")
# a function runs from its own label to the .Lfunc_end label the compiler closes it with (it may hold several s_endpgm)
_KERNEL = re.compile(r"^([A-Za-z_]\w*):[^\n]*\n(.*?)^\.Lfunc_end\d+:", re.S | re.M)


def _sgprs(tok):
    """Scalar registers named by one operand: s7 -> {7}, s[6:7] -> {6, 7}, vcc -> {'vcc'}; anything else -> {}."""
    tok = tok.strip()
    m = re.match(r"^s\[(\d+):(\d+)\]$", tok)
    if m:
        return set(range(int(m.group(1)), int(m.group(2)) + 1))
    m = re.match(r"^s(\d+)$", tok)
    if m:
        return {int(m.group(1))}
    if tok in ("vcc", "vcc_lo", "vcc_hi"):
        return {"vcc"}
    return set()


def _acc_regs(tok):
    """Accumulator registers named by one operand: a3 -> {3}, a[0:3] -> {0, 1, 2, 3}."""
    tok = tok.strip()
    m = re.match(r"^a\[(\d+):(\d+)\]$", tok)
    if m:
        return set(range(int(m.group(1)), int(m.group(2)) + 1))
    m = re.match(r"^a(\d+)$", tok)
    return {int(m.group(1))} if m else set()


def _instructions(body):
    for line in body.splitlines():
        line = line.split(";")[0].split("//")[0].strip()
        if not line or line.startswith(".") or line.endswith(":"):
            continue
        parts = line.split(None, 1)
        ops = [a.strip() for a in parts[1].split(",")] if len(parts) > 1 else []
        yield parts[0], ops, line


def _is_vmem(op):
    return op.startswith(_VMEM_PREFIXES)


def _is_lds_direct(op, ops):
    return op.startswith("global_load_lds") or (op.startswith("buffer_load") and any(o.split()[-1:] == ["lds"] for o in ops))


def _valu_scalar_dst(op, ops):
    if not ops:
        return set()
    if op.startswith(("v_readfirstlane", "v_readlane")):
        return _sgprs(ops[0])
    if op.startswith("v_cmp") and not op.startswith("v_cmpx"):
        return _sgprs(ops[0])
    return set()


def scan(text):
    """All hazard pairs of an assembly text: a list of (kernel, instruction index, instruction, reason)."""
    hits = []
    for km in _KERNEL.finditer(text):
        kernel = km.group(1)
        pending = []  # [registers a vector instruction wrote, wait states since, the instruction]
        m0_age, m0_src = None, ""
        mfma = []  # [accumulator registers a matrix instruction wrote, wait states since, the instruction]
        for i, (op, ops, line) in enumerate(_instructions(km.group(2))):
            if mfma and not op.startswith(("v_mfma", "v_smfmac")):
                touched = set()
                for o in ops:
                    first = o.split()
                    touched |= _acc_regs(first[0]) if first else set()
                for regs, age, src in mfma:
                    if regs & touched and age < MFMA_TO_OTHER_WAIT:
                        hits.append((kernel, i, line, "%d of %d wait states after `%s`" % (age, MFMA_TO_OTHER_WAIT, src)))
            if _is_vmem(op):
                read = set()
                for o in ops:
                    first = o.split()
                    read |= _sgprs(first[0]) if first else set()
                for regs, age, src in pending:
                    if regs & read and age < VALU_SGPR_TO_VMEM_WAIT:
                        hits.append((kernel, i, line, "%d of %d wait states after `%s`" % (age, VALU_SGPR_TO_VMEM_WAIT, src)))
                if _is_lds_direct(op, ops) and m0_age is not None and m0_age < M0_TO_LDS_DIRECT_WAIT:
                    hits.append((kernel, i, line, "%d of %d wait states after `%s`" % (m0_age, M0_TO_LDS_DIRECT_WAIT, m0_src)))
            step = int(ops[0], 0) + 1 if op == "s_nop" and ops else 1
            pending = [[r, a + step, s] for r, a, s in pending if a + step < VALU_SGPR_TO_VMEM_WAIT]
            mfma = [[r, a + step, s] for r, a, s in mfma if a + step < MFMA_TO_OTHER_WAIT]
            if op.startswith(("v_mfma", "v_smfmac")) and ops and _acc_regs(ops[0]):
                mfma = [m for m in mfma if m[0] != _acc_regs(ops[0])] + [[_acc_regs(ops[0]), 0, line]]
            if m0_age is not None:
                m0_age += step
            written = _valu_scalar_dst(op, ops)
            if written:
                pending.append([written, 0, line])
            if op.startswith("s_") and ops and ops[0] == "m0":
                m0_age, m0_src = 0, line
    return hits


# ---------------------------------------------------------------------------------------------------------------
# LDS reads written as asm.  The compiler places s_waitcnt for the loads it selects; the destination registers of
# a ds_read inside an asm statement are, to it, written when the statement ends, so nothing stops it from scheduling
# a use in front of the wait the source placed by hand, and a hand-counted `s_waitcnt lgkmcnt(N)` that is one too
# large lets an instruction read a register whose load has not returned.  Both give stale data, not a fault, and only
# sometimes.  This pass follows the LDS counter through the control-flow graph: LDS operations return in order, so
# after lgkmcnt(N) at most the N youngest are outstanding; any instruction that reads or writes a vector register a
# still outstanding read is going to write is reported.  Scalar loads share the counter and return out of order:
# while one is outstanding only lgkmcnt(0) is taken to retire anything.
# ---------------------------------------------------------------------------------------------------------------
_SMEM = "smem"
_MAX_STATES = 256


def _vgprs(tok):
    tok = tok.strip()
    m = re.match(r"^v\[(\d+):(\d+)\]$", tok)
    if m:
        return frozenset(range(int(m.group(1)), int(m.group(2)) + 1))
    m = re.match(r"^v(\d+)$", tok)
    return frozenset({int(m.group(1))}) if m else frozenset()


def _blocks(body):
    """[(label or None, [(op, ops, line), ...])] in layout order."""
    out, cur, name = [], [], None
    for raw in body.splitlines():
        line = raw.split(";")[0].split("//")[0].strip()
        if not line:
            continue
        if line.endswith(":"):
            out.append((name, cur))
            name, cur = line[:-1], []
            continue
        if line.startswith("."):
            continue
        parts = line.split(None, 1)
        ops = [a.strip() for a in parts[1].split(",")] if len(parts) > 1 else []
        cur.append((parts[0], ops, line))
        if parts[0].startswith(("s_branch", "s_cbranch", "s_endpgm", "s_setpc")):
            out.append((name, cur))
            name, cur = None, []
    out.append((name, cur))
    return [(n, b) for n, b in out if n is not None or b]


def _lds_step(state, op, ops, line, report):
    """Transfer function of one instruction on a tuple of outstanding LDS-counter operations (oldest first)."""
    if op == "s_waitcnt":
        text = " ".join(ops)
        m = re.search(r"lgkmcnt\((\d+)\)", text)
        if m is None:
            # a bare immediate: bits 11:8 hold the LDS counter on gfx9
            m2 = re.match(r"^(0x[0-9a-fA-F]+|\d+)$", text.strip())
            if m2 is None:
                return state
            n = (int(m2.group(1), 0) >> 8) & 0xF
        else:
            n = int(m.group(1))
        if n == 0:
            return ()
        if _SMEM in state:
            return state
        return state[len(state) - n:] if len(state) > n else state
    is_read = op.startswith(("ds_read", "ds_bpermute", "ds_permute", "ds_swizzle", "ds_consume", "ds_append"))
    # (a second read into the same registers is no hazard: LDS operations return in order)
    srcs = ops[1:] if is_read else ops
    used = frozenset().union(*[_vgprs(o.split()[0]) for o in srcs if o]) if srcs else frozenset()
    for dst in state:
        if dst is not _SMEM and dst & used:
            report(line, "touches v%s while the LDS read into it may be outstanding" % sorted(dst & used))
            break
    if is_read:
        return state + (_vgprs(ops[0]) if ops else frozenset(),)
    if op.startswith("ds_"):
        return state + (frozenset(),)
    if op.startswith(("s_load", "s_buffer_load", "s_scratch_load", "s_atc_probe", "s_memtime", "s_memrealtime")):
        return state + (_SMEM,)
    return state


def scan_lds_reads(text):
    """Uses of a register before the LDS read that writes it is known to have returned: (kernel, line, reason)."""
    hits = []
    for km in _KERNEL.finditer(text):
        kernel, blocks = km.group(1), _blocks(km.group(2))
        succ = _successors(blocks)
        seen = [set() for _ in blocks]
        seen[0].add(())
        work = [(0, ())]
        found = set()
        while work:
            b, state = work.pop()
            for op, ops, line in blocks[b][1]:
                state = _lds_step(state, op, ops, line, lambda l, why: found.add((l, why)))
                if len(state) > 15:  # the counter has four bits: the 16th operation is not issued before the oldest returns
                    state = state[-15:]
            for nb in succ[b]:
                if state not in seen[nb]:
                    if len(seen[nb]) >= _MAX_STATES:
                        found.add((blocks[nb][0] or "?", "too many distinct LDS-counter states reach this block"))
                        continue
                    seen[nb].add(state)
                    work.append((nb, state))
        hits += [(kernel, l, why) for l, why in sorted(found)]
    return hits


# ---- vector-memory loads against the VM counter ------------------------------------------------------------------
# The same question for vector-memory loads whose wait the compiler did not place: a global_load written as asm hands
# the compiler a destination register that it believes valid at once, and the s_waitcnt vmcnt(N) that really makes it
# so is counted by hand.  gfx9 has one counter for loads, stores and LDS-direct loads; operations of one kind return in
# order, so after vmcnt(N) everything but the N youngest has returned.  State: destination sets of the outstanding
# operations, oldest first (an empty set for stores, LDS-direct loads and atomics without return).  Any instruction
# that reads or writes a register whose load may still be outstanding is reported, except a later load into the same
# register (loads return in order).  Compiler-placed waits satisfy this by construction, which makes every kernel of
# the library a known-answer case for the scan.
_VMEM_PREFIX = ("global_", "buffer_", "flat_", "scratch_")


def _vm_wait_count(ops):
    text = " ".join(ops)
    m = re.search(r"vmcnt\((\d+)\)", text)
    if m is not None:
        return int(m.group(1))
    if "cnt(" in text:
        return None  # names other counters only
    m2 = re.match(r"^(0x[0-9a-fA-F]+|\d+)$", text.strip())
    if m2 is None:
        return None
    imm = int(m2.group(1), 0)
    return (imm & 0xF) | (((imm >> 14) & 0x3) << 4)  # bits 3:0 and 15:14 hold the VM counter on gfx9


def _vm_step(state, op, ops, line, report):
    """state: {vgpr: fewest operations known to be younger than the outstanding load into it}.  A load is complete
    once vmcnt(N) has been waited for with N <= that number; where paths join, the smaller number is kept."""
    if op == "s_waitcnt":
        n = _vm_wait_count(ops)
        if n is None or not state:
            return state
        return {r: c for r, c in state.items() if c < n}
    is_vmem = op.startswith(_VMEM_PREFIX)
    if not state and not is_vmem:
        return state
    is_load = is_vmem and "_load" in op and "_lds" not in op and "lds" not in [o.split()[-1] for o in ops if o]
    returns = is_load or (is_vmem and "atomic" in op and any(o.split()[-1] in ("glc", "sc0") for o in ops if o))
    dst = _vgprs(ops[0].split()[0]) if returns and ops else frozenset()
    if state:
        used = frozenset().union(*[_vgprs(o.split()[0]) for o in ops if o]) if ops else frozenset()
        srcs = frozenset().union(*[_vgprs(o.split()[0]) for o in ops[1:] if o]) if returns and len(ops) > 1 else used
        # (a later load into a register with a load outstanding is no hazard by itself: loads return in order)
        hit = [r for r in (srcs if is_load else used) if r in state]
        if hit:
            report(line, "touches v%s while the vector-memory load into it may be outstanding" % sorted(hit))
    if is_vmem:
        state = {r: c + 1 for r, c in state.items() if c + 1 < 63}  # six-bit counter: 63 younger ones mean it is back
        for r in dst:
            state[r] = 0
    return state


def scan_vmem_loads(text, only=None):
    """Uses of a register before the vector-memory load that writes it is known to have returned:
    (kernel, line, reason).  `only`: scan kernels whose name contains this string."""
    hits = []
    for km in _KERNEL.finditer(text):
        kernel, blocks = km.group(1), _blocks(km.group(2))
        if only is not None and only not in kernel:
            continue
        succ = _successors(blocks)
        entry = [None] * len(blocks)   # state at block entry (None: not reached yet)
        entry[0] = {}
        work = [0]
        found = set()
        while work:
            b = work.pop()
            state = dict(entry[b])
            for op, ops, line in blocks[b][1]:
                state = _vm_step(state, op, ops, line, lambda l, why: found.add((l, why)))
            for nb in succ[b]:
                old = entry[nb]
                if old is None:
                    entry[nb] = dict(state)
                    work.append(nb)
                    continue
                changed = False
                for r, c in state.items():
                    if r not in old or c < old[r]:
                        old[r] = c
                        changed = True
                if changed:
                    work.append(nb)
        hits += [(kernel, l, why) for l, why in sorted(found)]
    return hits


# Packed fp32 arithmetic is switched off for this library (a compiler flag removes the feature, and no source writes
# the instructions by hand); this confirms it on what was actually generated.
_PACKED_F32 = ("v_pk_add_f32", "v_pk_mul_f32", "v_pk_fma_f32")


def scan_packed_f32(text):
    hits = []
    for km in _KERNEL.finditer(text):
        for i, (op, _, line) in enumerate(_instructions(km.group(2))):
            if op.startswith(_PACKED_F32):
                hits.append((km.group(1), i, line, "packed fp32 arithmetic is not to be generated for this library"))
    return hits


def _successors(blocks):
    index = {n: i for i, (n, _) in enumerate(blocks) if n is not None}
    succ = []
    for i, (_, ins) in enumerate(blocks):
        last = ins[-1] if ins else None
        nxt = [i + 1] if i + 1 < len(blocks) else []
        target = [index[last[1][0]]] if last and last[1] and last[1][0] in index else []
        if last is None:
            succ.append(nxt)
        elif last[0] == "s_branch":
            succ.append(target)
        elif last[0].startswith("s_cbranch"):
            succ.append(nxt + target)
        elif last[0].startswith(("s_endpgm", "s_setpc")):
            succ.append([])
        else:
            succ.append(nxt)
    return succ


def _blocks_in_loops(succ):
    """Indices of the basic blocks that lie on a cycle of the control-flow graph (Tarjan, iterative)."""
    n = len(succ)
    order, low, on_stack, comp = [None] * n, [0] * n, [False] * n, [None] * n
    stack, counter, ncomp = [], 0, 0
    for root in range(n):
        if order[root] is not None:
            continue
        work = [(root, 0)]
        while work:
            v, k0 = work[-1]
            if k0 == 0:
                order[v] = low[v] = counter
                counter += 1
                stack.append(v)
                on_stack[v] = True
            descended = False
            for k in range(k0, len(succ[v])):
                w = succ[v][k]
                if order[w] is None:
                    work[-1] = (v, k + 1)
                    work.append((w, 0))
                    descended = True
                    break
                if on_stack[w]:
                    low[v] = min(low[v], order[w])
            if descended:
                continue
            if low[v] == order[v]:
                while True:
                    w = stack.pop()
                    on_stack[w] = False
                    comp[w] = ncomp
                    if w == v:
                        break
                ncomp += 1
            work.pop()
            if work:
                low[work[-1][0]] = min(low[work[-1][0]], low[v])
    size = {}
    for v in range(n):
        size[comp[v]] = size.get(comp[v], 0) + 1
    return [v for v in range(n) if size[comp[v]] > 1 or v in succ[v]]


# Kernels whose loops are known to touch scratch memory, with the reason each is tolerated.
SCRATCH_IN_LOOP_ALLOWED = {
    # stream-K on the element-by-element stager: the last resort for operands contiguous along neither axis
    "gemm_streamk_kernel": "the element-wise stager of the last-resort stream-K kernel spills",
    # rms_norm backward for rows of 8193-16384 elements, in the code the GPU parity suite last passed on: a pack
    # zeroed element by element stays in scratch.  variants.h: FG_V_RMS_BWD_ZERO_PACK removes it (not yet GPU-tested).
    "rms_bwd_rows_kernelIDF16_Li8ELi2ELi1024ELb0": "tested code keeps a two-pack row partly in scratch",
    "rms_bwd_rows_kernelIDF16bLi8ELi2ELi1024ELb0": "tested code keeps a two-pack row partly in scratch",
    "rms_bwd_rows_kernelIfLi4ELi2ELi1024ELb0": "tested code keeps a two-pack row partly in scratch",
}


def scan_scratch_in_loops(text, allowed=SCRATCH_IN_LOOP_ALLOWED):
    """Register spills (or private arrays) that are accessed inside a loop: (kernel, count, first instruction)."""
    hits = []
    for km in _KERNEL.finditer(text):
        if any(a in km.group(1) for a in allowed):
            continue
        blocks = _blocks(km.group(2))
        ops = [line for v in _blocks_in_loops(_successors(blocks)) for op, _, line in blocks[v][1] if op.startswith("scratch_")]
        if ops:
            hits.append((km.group(1), len(ops), ops[0]))
    return hits


def check_file(path):
    with open(path) as f:
        text = f.read()
    return (scan(text) + [(k, 0, line, why) for k, line, why in scan_lds_reads(text)] +
            [(k, 0, line, why) for k, line, why in scan_vmem_loads(text)] + scan_packed_f32(text) +
            [(k, 0, first, "%d scratch accesses inside a loop: registers spill there" % n)
             for k, n, first in scan_scratch_in_loops(text)])


def kernel_digests(text):
    """{kernel: (sha1 of its instruction stream, instruction and label lines)}.  Comments are dropped and the
    per-function number in basic-block labels (.LBB<n>_<m>) is removed, so that a kernel's digest does not depend on
    which other kernels its source instantiates; registers, immediates and instruction order all count."""
    import hashlib

    out = {}
    for km in _KERNEL.finditer(text):
        lines = []
        for line in km.group(2).split("\n"):
            line = re.sub(r"\.LBB\d+_", ".LBB_", line.split(";")[0].rstrip())
            if line.strip():
                lines.append(line)
        out[km.group(1)] = (hashlib.sha1("\n".join(lines).encode()).hexdigest(), len(lines))
    return out


def memory_trace(text, name_part):
    """One line per kernel whose name contains name_part: its vector-memory traffic in program order.
    L load, D LDS-direct load, S store, A atomic, | barrier, (n) a wait that leaves n operations in flight,
    k a scalar load issued after the first 40 instructions (a kernel argument fetched late), . a branch.
    A well-formed streaming kernel reads `LL..L(n)..(0)|..|S..S`: every request before the first wait."""
    lines = []
    for km in _KERNEL.finditer(text):
        if name_part not in km.group(1):
            continue
        out = []
        for i, (op, _, line) in enumerate(_instructions(km.group(2))):
            if op.startswith("global_load_lds") or (op.startswith("buffer_load") and line.endswith("lds")):
                out.append("D")
            elif op.startswith(("global_load", "buffer_load", "flat_load", "scratch_load")):
                out.append("L")
            elif op.startswith(("global_store", "buffer_store", "flat_store", "scratch_store")):
                out.append("S")
            elif op.startswith(("global_atomic", "buffer_atomic", "flat_atomic")):
                out.append("A")
            elif op == "s_barrier":
                out.append("|")
            elif op == "s_waitcnt" and "vmcnt" in line:
                out.append("(%s)" % re.search(r"vmcnt\((\d+)\)", line).group(1))
            elif op.startswith(("s_load", "s_buffer_load")) and i > 40:
                out.append("k")
            elif op.startswith(("s_cbranch", "s_branch")):
                out.append(".")
        lines.append("%s\n    %s" % (km.group(1), "".join(out)))
    return lines


if __name__ == "__main__":
    if len(sys.argv) >= 4 and sys.argv[1] == "--trace":
        # python isa_check.py --trace <part of a kernel name> <device .s files>
        for p in sys.argv[3:]:
            with open(p) as f:
                print("\n".join(memory_trace(f.read(), sys.argv[2])))
        sys.exit(0)
    bad = 0
    for p in sys.argv[1:]:
        found = check_file(p)
        bad += len(found)
        print("%s: %d hazard pair(s)" % (p, len(found)))
        for kernel, i, line, why in found[:20]:
            print("  %s  #%d  %s  <- %s" % (kernel[:80], i, line, why))
    sys.exit(1 if bad else 0)
