"""Wait-state check of the device assembly of the sources that issue memory instructions from inline asm.

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

The scan is textual: it walks each kernel's instructions in program order, counts every instruction as one wait
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


def check_file(path):
    with open(path) as f:
        return scan(f.read())


if __name__ == "__main__":
    bad = 0
    for p in sys.argv[1:]:
        found = check_file(p)
        bad += len(found)
        print("%s: %d hazard pair(s)" % (p, len(found)))
        for kernel, i, line, why in found[:20]:
            print("  %s  #%d  %s  <- %s" % (kernel[:80], i, line, why))
    sys.exit(1 if bad else 0)
