"""An interpreter for the gfx950 (GCN/CDNA) assembly that hipcc emits for this library's kernels.

It runs the compiler's own output (the `.s` text the build keeps beside the objects) on numpy: a wavefront is 64 lanes
wide, a workgroup's wavefronts each run until they stand at a barrier (or end), workgroups run one after the other.
Global memory is a set of registered buffers and EVERY access is checked against them; LDS, private memory and all
registers start out holding NaNs.  Memory operations stay "in flight" until an s_waitcnt covers them: using a register
a load in flight will write, or LDS bytes a write or an LDS-DMA in flight will fill, is an error, and so is LDS traffic
between two wavefronts with no barrier in between (class Exec).  It models function and ordering, not time: latencies,
wait states between dependent instructions and bank conflicts are outside it (csrc/isa_check.py scans for wait states).

Trust comes from the kernels the GPU parity suite has passed: the interpreter reproduces the oracle on those
(tests/test_interpreted_kernels.py, default build), and is then used on kernel variants that have not been on a GPU.
Instructions are added as kernels need them; an unknown one is an error that names it, never a guess.
"""
import re
import struct

import numpy as np
import yaml

U32 = np.uint32
POISON = 0x7FC07FC0
LANES = np.arange(64, dtype=np.uint64)
FULL = (1 << 64) - 1


class EmuError(Exception):
    pass


# ---------------------------------------------------------------------------------------------------------------
# memory
# ---------------------------------------------------------------------------------------------------------------
class Memory:
    """Registered buffers at made-up device addresses; every access must fall inside one of them."""

    def __init__(self):
        self.bufs = []   # (base, np.uint8 array, name)
        self.next = 0x4000000000000000   # far from anything the process itself maps

    def alloc(self, nbytes, name="buf", data=None):
        base = self.next
        arr = np.zeros(int(nbytes), dtype=np.uint8)
        if data is not None:
            raw = np.frombuffer(np.ascontiguousarray(data).tobytes(), dtype=np.uint8)
            arr[:raw.size] = raw
        self.bufs.append((base, arr, name))
        self.next += (int(nbytes) + 0xFFFF + 0x100000) & ~0xFFFF   # a gap after every buffer
        return base

    def map_external(self, base, nbytes, name="external"):
        """Make [base, base + nbytes) of THIS process's memory a buffer (zero-copy): a tensor's storage, for instance.
        Buffers mapped earlier that overlap it are dropped (their memory was freed and handed out again)."""
        import ctypes
        base, nbytes = int(base), int(nbytes)
        if nbytes <= 0:
            return
        self.bufs = [b for b in self.bufs if not (len(b) > 3 and b[0] < base + nbytes and base < b[0] + b[1].size)]
        arr = np.ctypeslib.as_array((ctypes.c_uint8 * nbytes).from_address(base))
        self.bufs.append((base, arr, name, "external"))

    def drop_externals(self):
        self.bufs = [b for b in self.bufs if len(b) == 3]

    def write(self, base, raw):
        arr = self.view(base)
        arr[:len(raw)] = np.frombuffer(bytes(raw), dtype=np.uint8)

    def view(self, base):
        for b, arr, *_ in self.bufs:
            if b == base:
                return arr
        raise KeyError(base)

    def _find(self, addrs, width, what):
        addrs = np.asarray(addrs, dtype=np.uint64)
        lo, hi = int(addrs.min()), int(addrs.max())
        for b, arr, *_ in self.bufs:
            if b <= lo and hi + width <= b + arr.size:
                return b, arr
        # not one buffer for all lanes: find per-lane (slow path), and report the first stray address
        for a in addrs.tolist():
            if not any(b[0] <= a and a + width <= b[0] + b[1].size for b in self.bufs):
                near = min(self.bufs, key=lambda x: abs(x[0] - a)) if self.bufs else None
                raise EmuError("%s: %d-byte access at %#x is outside every buffer (nearest: %s at %#x, %d bytes)" % (
                    what, width, a, near[2] if near else "-", near[0] if near else 0, near[1].size if near else 0))
        return None, None

    def load(self, addrs, width, what="load"):
        """addrs: uint64 [n] -> uint8 [n, width]"""
        if len(addrs) == 0:
            return np.zeros((0, width), dtype=np.uint8)
        b, arr = self._find(addrs, width, what)
        if arr is not None:
            idx = (np.asarray(addrs, dtype=np.uint64) - np.uint64(b)).astype(np.int64)[:, None] + np.arange(width)[None, :]
            return arr[idx]
        out = np.zeros((len(addrs), width), dtype=np.uint8)
        for i, a in enumerate(np.asarray(addrs).tolist()):
            for bb, arr2, *_ in self.bufs:
                if bb <= a and a + width <= bb + arr2.size:
                    out[i] = arr2[a - bb:a - bb + width]
                    break
        return out

    def store(self, addrs, data, what="store"):
        """addrs: uint64 [n]; data: uint8 [n, width]"""
        if len(addrs) == 0:
            return
        width = data.shape[1]
        b, arr = self._find(addrs, width, what)
        if arr is not None:
            idx = (np.asarray(addrs, dtype=np.uint64) - np.uint64(b)).astype(np.int64)[:, None] + np.arange(width)[None, :]
            arr[idx] = data
            return
        for i, a in enumerate(np.asarray(addrs).tolist()):
            for bb, arr2, *_ in self.bufs:
                if bb <= a and a + width <= bb + arr2.size:
                    arr2[a - bb:a - bb + width] = data[i]
                    break


# ---------------------------------------------------------------------------------------------------------------
# program text
# ---------------------------------------------------------------------------------------------------------------
_KERNEL = re.compile(r"^([A-Za-z_]\w*):[^\n]*\n(.*?)^\.Lfunc_end\d+:", re.S | re.M)


_TOK_REG = re.compile(r"^(?:-|neg\(|abs\(|sext\(|\|)*([vsa])(?:(\d+)|\[(\d+):(\d+)\])[)|]*$")
_WAIT = re.compile(r"(vmcnt|lgkmcnt|expcnt)\((\d+)\)")


class Instr:
    __slots__ = ("op", "base", "enc", "ops", "mods", "line", "vset", "sset", "wait", "ld_queue", "ld_only_dest")

    def __init__(self, op, ops, mods, line):
        self.op, self.ops, self.mods, self.line = op, ops, mods, line
        m = re.match(r"^(.*?)(_e32|_e64|_dpp|_sdwa|_e64_dpp)?$", op)
        self.base, self.enc = m.group(1), (m.group(2) or "")
        # registers the instruction names (sources and destinations alike), for the in-flight checks
        vs, ss = set(), set()
        for t in ops:
            mm = _TOK_REG.match(t)
            if mm:
                lo = int(mm.group(2) if mm.group(2) is not None else mm.group(3))
                hi = lo if mm.group(2) is not None else int(mm.group(4))
                if mm.group(1) == "s":
                    ss.update(range(lo, hi + 1))
                else:
                    vs.update(range(lo + (256 if mm.group(1) == "a" else 0), hi + 1 + (256 if mm.group(1) == "a" else 0)))
            elif t == "vcc":
                ss.update((106, 107))
            elif t in _SPECIAL_EARLY:
                ss.add(_SPECIAL_EARLY[t])
        self.vset, self.sset = frozenset(vs), frozenset(ss)
        # A load may name as its destination a register that an older load OF THE SAME COUNTER has yet to write (results
        # of one counter arrive in order: the compiler does this for loads under complementary EXEC masks).  Registers
        # that are only the destination, not also part of the address or data operands, get that exemption.
        self.ld_queue, self.ld_only_dest = None, frozenset()
        if (op.startswith(("global_load_", "scratch_load_")) and not op.startswith("global_load_lds")) or \
                op.startswith(("ds_read", "ds_bpermute", "ds_permute", "ds_swizzle")):
            self.ld_queue = 0 if op[0] != "d" else 1
            def regs_of(t):
                mm = _TOK_REG.match(t)
                if not mm or mm.group(1) == "s":
                    return set()
                lo = int(mm.group(2) if mm.group(2) is not None else mm.group(3))
                hi = lo if mm.group(2) is not None else int(mm.group(4))
                off = 256 if mm.group(1) == "a" else 0
                return set(range(lo + off, hi + 1 + off))
            others = set()
            for t in ops[1:]:
                others |= regs_of(t)
            self.ld_only_dest = frozenset(regs_of(ops[0]) - others)
        self.wait = None
        if op == "s_waitcnt":
            self.wait = {k: int(v) for k, v in _WAIT.findall(ops[0] if ops else "")}
            if ops and not self.wait and ops[0].strip():
                raise EmuError("cannot read the counts of %r" % line)


_SPECIAL_EARLY = {"vcc_lo": 106, "vcc_hi": 107, "m0": 124}


def _split_operands(text):
    """Split on commas that are not inside brackets."""
    out, depth, cur = [], 0, ""
    for ch in text:
        if ch in "[(":
            depth += 1
        elif ch in "])":
            depth -= 1
        if ch == "," and depth == 0:
            out.append(cur.strip())
            cur = ""
        else:
            cur += ch
    if cur.strip():
        out.append(cur.strip())
    return out


_MOD = re.compile(r"^(offset|offset0|offset1|quad_perm|row_shl|row_shr|row_ror|row_bcast|row_mask|bank_mask|bound_ctrl|"
                  r"dst_sel|dst_unused|src0_sel|src1_sel|op_sel|op_sel_hi|neg_lo|neg_hi|mul|div|cbsz|abid|blgp|"
                  r"wave_shl|wave_shr|wave_rol|wave_ror|row_newbcast|dim|unorm|format|bitop3):(.*)$")
_FLAGS = {"off", "glc", "slc", "nt", "sc0", "sc1", "lds", "clamp", "gds", "row_mirror", "row_half_mirror", "tfe", "scc",
          "vmcnt", "idxen", "offen"}


_FILE_CACHE = {}


def _file_index(text):
    """Per assembly text, parsed once: kernel bodies, kernel descriptors and the metadata records by kernel name."""
    key = (len(text), hash(text))
    if key not in _FILE_CACHE:
        bodies = {k.group(1): k.group(2) for k in _KERNEL.finditer(text)}
        kds = {m.group(1): m.group(2) for m in re.finditer(r"\.amdhsa_kernel (\S+)\n(.*?)\.end_amdhsa_kernel", text, re.S)}
        metas = {}
        mm = re.search(r"\.amdgpu_metadata\n---\n(.*?)\n\.\.\.\n", text, re.S)
        if mm:
            loader = getattr(yaml, "CSafeLoader", yaml.SafeLoader)
            for k in yaml.load(mm.group(1), Loader=loader)["amdhsa.kernels"]:
                metas[k[".name"]] = k
        _FILE_CACHE[key] = (bodies, kds, metas)
    return _FILE_CACHE[key]


def parse_program(text, name_part, exact=False):
    bodies, kds, metas = _file_index(text)
    km = [k for k in bodies if (name_part == k if exact else name_part in k)]
    if len(km) != 1:
        raise EmuError("%d kernels match %r" % (len(km), name_part))
    name, body = km[0], bodies[km[0]]
    instrs, labels = [], {}
    for raw in body.splitlines():
        line = raw.split(";")[0].strip()
        if not line or line.startswith("."):
            if line.endswith(":"):
                labels[line[:-1]] = len(instrs)
            continue
        if line.endswith(":"):
            labels[line[:-1]] = len(instrs)
            continue
        parts = line.split(None, 1)
        op = parts[0]
        rest = parts[1] if len(parts) > 1 else ""
        ops, mods = [], {}
        if op == "s_waitcnt" or op.startswith("s_nop") or op.startswith("s_sleep") or op.startswith("s_setprio"):
            instrs.append(Instr(op, [rest], {}, line))
            continue
        for tok in _split_operands(rest):
            # trailing modifiers share the last comma-separated field, separated by spaces
            fields = []
            depth, cur = 0, ""
            for ch in tok:
                if ch in "[(":
                    depth += 1
                elif ch in "])":
                    depth -= 1
                if ch == " " and depth == 0:
                    if cur:
                        fields.append(cur)
                    cur = ""
                else:
                    cur += ch
            if cur:
                fields.append(cur)
            first = True
            for f in fields:
                m = _MOD.match(f)
                if m:
                    mods[m.group(1)] = m.group(2)
                elif f in _FLAGS:
                    if f == "off" and first:
                        ops.append("off")
                    else:
                        mods[f] = True
                elif first:
                    ops.append(f)
                else:
                    raise EmuError("cannot parse %r in %r" % (f, line))
                first = False
        instrs.append(Instr(op, ops, mods, line))
    # kernel descriptor and metadata
    kd = {}
    for k, v in re.findall(r"\.amdhsa_(\w+) (\S+)", kds.get(name, "")):
        try:
            kd[k] = int(v, 0)
        except ValueError:
            kd[k] = v
    meta = metas.get(name, {})
    return Program(name, instrs, labels, kd, meta)


class Program:
    def __init__(self, name, instrs, labels, kd, meta):
        self.name, self.instrs, self.labels, self.kd, self.meta = name, instrs, labels, kd, meta


# ---------------------------------------------------------------------------------------------------------------
# numeric helpers
# ---------------------------------------------------------------------------------------------------------------
def f32(u):
    return np.asarray(u, dtype=U32).view(np.float32)


def u32(f):
    return np.asarray(f, dtype=np.float32).view(U32)


def i32(u):
    return np.asarray(u, dtype=U32).view(np.int32)


def mask_to_lanes(m):
    return ((np.uint64(m) >> LANES) & np.uint64(1)).astype(bool)


def lanes_to_mask(b):
    return int((b.astype(np.uint64) << LANES).sum(dtype=np.uint64))


def bf16_round(f):
    """fp32 array -> uint32 array holding the bf16 bits (round to nearest even, NaN kept quiet)."""
    u = u32(f).astype(np.uint64)
    nan = np.isnan(f)
    r = ((u + 0x7FFF + ((u >> 16) & 1)) >> 16).astype(U32)
    return np.where(nan, U32(0x7FC0) | ((u >> 16).astype(U32) & U32(0x8000)), r) & U32(0xFFFF)


def f16_bits(f):
    with np.errstate(over="ignore", invalid="ignore"):
        return np.asarray(f, dtype=np.float32).astype(np.float16).view(np.uint16).astype(U32)


def f16_to_f32(bits16):
    return np.asarray(bits16, dtype=np.uint16).view(np.float16).astype(np.float32)



# ---------------------------------------------------------------------------------------------------------------
# a wavefront
# ---------------------------------------------------------------------------------------------------------------
_SPECIAL = {"vcc_lo": 106, "vcc_hi": 107, "m0": 124, "exec_lo": 126, "exec_hi": 127, "flat_scratch_lo": 102,
            "flat_scratch_hi": 103, "xnack_mask_lo": 104, "xnack_mask_hi": 105}


class Wave:
    def __init__(self, nv=512):
        self.s = np.zeros(128, dtype=U32)
        self.v = np.zeros((nv, 64), dtype=U32)     # v0..v255, a0..a255 behind them
        self.scc = 0
        self.pc = 0
        self.done = False
        self.at_barrier = False
        self.scratch = {}
        self.wid = 0
        # memory operations issued and not yet covered by a wait, oldest first (see Exec.strict)
        self.vm_q, self.lds_q, self.smem_q = [], [], []
        self.pend_v, self.pend_s = {}, {}

    # 64-bit specials live in the scalar file
    @property
    def exec(self):
        return int(self.s[126]) | (int(self.s[127]) << 32)

    @exec.setter
    def exec(self, m):
        self.s[126], self.s[127] = m & 0xFFFFFFFF, (m >> 32) & 0xFFFFFFFF

    @property
    def vcc(self):
        return int(self.s[106]) | (int(self.s[107]) << 32)

    @vcc.setter
    def vcc(self, m):
        self.s[106], self.s[107] = m & 0xFFFFFFFF, (m >> 32) & 0xFFFFFFFF


_REG = re.compile(r"^([vsa])(\d+)$")
_RANGE = re.compile(r"^([vsa])\[(\d+):(\d+)\]$")


def _parse_lit(tok, fkind):
    """Literal or inline constant -> 32-bit pattern (int).  fkind: 'f32', 'f16' or 'int'."""
    t = tok
    if re.match(r"^-?0x[0-9a-fA-F]+$", t):
        v = int(t, 16)
        return v & 0xFFFFFFFFFFFFFFFF
    if re.match(r"^-?\d+$", t):
        return int(t) & 0xFFFFFFFFFFFFFFFF
    if re.match(r"^-?\d*\.\d+(e[-+]?\d+)?$|^-?\d+\.\d*(e[-+]?\d+)?$|^-?\d+e[-+]?\d+$", t):
        f = float(t)
        if fkind == "f16":
            return int(np.array([f], dtype=np.float16).view(np.uint16)[0])
        if fkind == "f64":
            return struct.unpack("<Q", struct.pack("<d", f))[0]
        return struct.unpack("<I", struct.pack("<f", f))[0]
    raise EmuError("cannot parse literal %r" % tok)


class Exec:
    """Executes one instruction of one wave."""

    def __init__(self, mem, lds, program, strict=True):
        self.mem, self.lds, self.prog = mem, lds, program
        # strict: memory operations stay "in flight" until an s_waitcnt covers them.  Touching a register a load in
        # flight will write, reading LDS bytes a write or LDS-DMA in flight will fill, and LDS traffic between two
        # wavefronts with no barrier in between are errors: the counts written by hand into asm statements, and the
        # barriers of the software pipelines, are checked as executed.
        self.strict = strict
        n = lds.size
        self.epoch = 1
        self.w_epoch = np.zeros(n, dtype=np.int32)
        self.w_wave = np.zeros(n, dtype=np.int16)
        self.r_epoch = np.zeros(n, dtype=np.int32)
        self.r_wave = np.zeros(n, dtype=np.int16)       # -1: read by several wavefronts in this epoch
        self.fill_owner = np.zeros(n, dtype=np.int16)   # wave id + 1 of a ds_write in flight, -(wave id + 1) of an LDS-DMA
        self.read_inflight = np.zeros(n, dtype=np.int16)

    # ---- LDS --------------------------------------------------------------------------------------------------
    def _lds_index(self, ins, addrs, width):
        a = np.asarray(addrs).astype(np.int64)
        if a.size and ((a < 0).any() or (a + width > self.lds.size).any()):
            raise EmuError("LDS access outside the %d bytes allocated (address %d): %r" %
                           (self.lds.size, int(a.max()), ins.line))
        return a[:, None] + np.arange(width)[None, :]

    def lds_get(self, w, ins, addrs, width, track=True):
        """Bytes [n, width] at the given addresses.  Returns (raw, flat byte indices)."""
        ix = self._lds_index(ins, addrs, width)
        if self.strict and ix.size:
            flat = ix.ravel()
            own = self.fill_owner[flat]
            bad = (own != 0) & (own != w.wid + 1)
            if bad.any():
                o = int(own[bad][0])
                raise EmuError("wave %d reads LDS byte %d while %s of wave %d is in flight (no wait covers it): %r" % (
                    w.wid, int(flat[bad][0]), "an LDS-DMA" if o < 0 else "a ds_write", abs(o) - 1, ins.line))
            race = (self.w_epoch[flat] == self.epoch) & (self.w_wave[flat] != w.wid)
            if race.any():
                raise EmuError("wave %d reads LDS byte %d written by wave %d with no barrier in between: %r" % (
                    w.wid, int(flat[race][0]), int(self.w_wave[flat][race][0]), ins.line))
            if track:
                same = self.r_epoch[flat] == self.epoch
                self.r_wave[flat] = np.where(same & (self.r_wave[flat] != w.wid), -1, w.wid)
                self.r_epoch[flat] = self.epoch
        return self.lds[ix], ix

    def lds_put(self, w, ins, addrs, raw, dma=False):
        ix = self._lds_index(ins, addrs, raw.shape[1])
        if self.strict and ix.size:
            flat = ix.ravel()
            waw = (self.w_epoch[flat] == self.epoch) & (self.w_wave[flat] != w.wid)
            if waw.any():
                raise EmuError("wave %d writes LDS byte %d written by wave %d with no barrier in between: %r" % (
                    w.wid, int(flat[waw][0]), int(self.w_wave[flat][waw][0]), ins.line))
            war = (self.r_epoch[flat] == self.epoch) & (self.r_wave[flat] != w.wid)
            if war.any():
                raise EmuError("wave %d writes LDS byte %d read by another wave with no barrier in between: %r" % (
                    w.wid, int(flat[war][0]), ins.line))
            own = self.fill_owner[flat]
            if ((own != 0) & (own != w.wid + 1)).any() or (dma and (own != 0).any()):
                raise EmuError("wave %d writes LDS bytes another write in flight targets: %r" % (w.wid, ins.line))
            if dma and (self.read_inflight[flat] > 0).any():
                raise EmuError("wave %d starts an LDS-DMA onto bytes an LDS read in flight has yet to fetch: %r" % (w.wid, ins.line))
            self.w_epoch[flat] = self.epoch
            self.w_wave[flat] = w.wid
            self.fill_owner[flat] = -(w.wid + 1) if dma else (w.wid + 1)
        self.lds[ix] = raw
        return ix

    def barrier_released(self):
        self.epoch += 1

    # ---- operations in flight -----------------------------------------------------------------------------------
    def issue(self, w, queue, vregs=(), sregs=(), fill=None, fetch=None):
        """Record a memory operation: registers it will write, LDS bytes it fills (fill) or fetches (fetch)."""
        if not self.strict:
            return
        q = 0 if queue == "vm_q" else 1
        for r in vregs:
            w.pend_v.setdefault(r, [0, 0])[q] += 1
        for r in sregs:
            w.pend_s[r] = w.pend_s.get(r, 0) + 1
        if fetch is not None:
            np.add.at(self.read_inflight, fetch.ravel(), 1)
        getattr(w, queue).append((tuple(vregs), tuple(sregs), fill, fetch, q))

    def _retire(self, w, entry):
        vregs, sregs, fill, fetch, q = entry
        for r in vregs:
            c = w.pend_v[r]
            c[q] -= 1
            if c[0] == 0 and c[1] == 0:
                del w.pend_v[r]
        for r in sregs:
            if w.pend_s[r] == 1:
                del w.pend_s[r]
            else:
                w.pend_s[r] -= 1
        if fill is not None:
            self.fill_owner[fill.ravel()] = 0
        if fetch is not None:
            np.subtract.at(self.read_inflight, fetch.ravel(), 1)

    def wait(self, w, counts):
        """s_waitcnt: vmcnt(n) leaves at most the n youngest vector-memory operations in flight (they complete in
        order); lgkmcnt(n) does so for the LDS operations (in order among themselves), and only lgkmcnt(0) says
        anything about scalar loads, which return in any order."""
        if "vmcnt" in counts:
            while len(w.vm_q) > counts["vmcnt"]:
                self._retire(w, w.vm_q.pop(0))
        if "lgkmcnt" in counts:
            while len(w.lds_q) > counts["lgkmcnt"]:
                self._retire(w, w.lds_q.pop(0))
            if counts["lgkmcnt"] == 0:
                while w.smem_q:
                    self._retire(w, w.smem_q.pop(0))

    def check_registers(self, w, ins):
        if w.pend_v and not ins.vset.isdisjoint(w.pend_v):
            hit = ins.vset & set(w.pend_v)
            if ins.ld_queue is not None:
                hit = {r for r in hit if not (r in ins.ld_only_dest and w.pend_v[r][1 - ins.ld_queue] == 0)}
            if not hit:
                return self._check_sregs(w, ins)
            r = sorted(hit)[0]
            raise EmuError("wave %d: %s%d is the destination of a load still in flight (vmcnt %d, lgkmcnt %d outstanding): %r" % (
                w.wid, "a" if r >= 256 else "v", r % 256, len(w.vm_q), len(w.lds_q), ins.line))
        self._check_sregs(w, ins)

    def _check_sregs(self, w, ins):
        if w.pend_s and not ins.sset.isdisjoint(w.pend_s):
            r = sorted(ins.sset & set(w.pend_s))[0]
            raise EmuError("wave %d: s%d is the destination of a scalar load still in flight: %r" % (w.wid, r, ins.line))

    # ---- scalar operands ---------------------------------------------------------------------------------------
    def sreg_index(self, tok):
        m = _REG.match(tok)
        if m and m.group(1) == "s":
            return int(m.group(2)), 1
        m = _RANGE.match(tok)
        if m and m.group(1) == "s":
            return int(m.group(2)), int(m.group(3)) - int(m.group(2)) + 1
        if tok == "vcc":
            return 106, 2
        if tok == "exec":
            return 126, 2
        if tok in _SPECIAL:
            return _SPECIAL[tok], 1
        return None

    def sread(self, w, tok, bits=32, fkind="int"):
        if tok in ("scc", "src_scc"):
            return w.scc
        r = self.sreg_index(tok)
        if r is not None:
            i, n = r
            v = int(w.s[i])
            if bits == 64:
                v |= int(w.s[i + 1]) << 32
            return v
        if tok == "src_shared_base":
            return 0
        v = _parse_lit(tok, fkind)
        return v & ((1 << bits) - 1)

    def swrite(self, w, tok, val, bits=32):
        r = self.sreg_index(tok)
        if r is None:
            raise EmuError("not a scalar destination: %r" % tok)
        i, _ = r
        w.s[i] = val & 0xFFFFFFFF
        if bits == 64:
            w.s[i + 1] = (val >> 32) & 0xFFFFFFFF

    # ---- vector operands ---------------------------------------------------------------------------------------
    def vindex(self, tok):
        m = _REG.match(tok)
        if m and m.group(1) in "va":
            return int(m.group(2)) + (256 if m.group(1) == "a" else 0), 1
        m = _RANGE.match(tok)
        if m and m.group(1) in "va":
            return int(m.group(2)) + (256 if m.group(1) == "a" else 0), int(m.group(3)) - int(m.group(2)) + 1
        return None

    def vread(self, w, tok, bits=32, fkind="f32"):
        """Operand -> uint32[64] (bits=32) or uint64[64] (bits=64), with -x / |x| applied as float sign operations."""
        neg = ab = False
        t = tok
        if t.startswith("-") and not re.match(r"^-[\d.]", t):
            neg, t = True, t[1:]
        if t.startswith("|") and t.endswith("|"):
            ab, t = True, t[1:-1]
        if t.startswith("neg(") and t.endswith(")"):
            neg, t = True, t[4:-1]
        if t.startswith("abs(") and t.endswith(")"):
            ab, t = True, t[4:-1]
        r = self.vindex(t)
        if r is not None:
            i, n = r
            if bits == 64:
                val = w.v[i].astype(np.uint64) | (w.v[i + 1].astype(np.uint64) << np.uint64(32))
            else:
                val = w.v[i].copy()
        else:
            sv = self.sread(w, t, bits, fkind)
            val = np.full(64, sv, dtype=np.uint64 if bits == 64 else U32)
        if ab or neg:
            sign = np.uint64(1 << 63) if bits == 64 else (U32(0x8000) if fkind == "f16" else U32(0x80000000))
            if ab:
                val = val & ~sign
            if neg:
                val = val ^ sign
        return val

    def vwrite(self, w, tok, val, mask=None, bits=32):
        i, n = self.vindex(tok)
        lanes = mask_to_lanes(w.exec if mask is None else mask)
        if bits == 64:
            val = np.asarray(val, dtype=np.uint64)
            w.v[i][lanes] = (val & np.uint64(0xFFFFFFFF)).astype(U32)[lanes]
            w.v[i + 1][lanes] = (val >> np.uint64(32)).astype(U32)[lanes]
        else:
            w.v[i][lanes] = np.asarray(val, dtype=U32)[lanes]


# ---------------------------------------------------------------------------------------------------------------
# instruction semantics
# ---------------------------------------------------------------------------------------------------------------
def _dpp_source(ins, w, val, exec_lanes):
    """Per-lane source of a DPP operand: (permuted values, lanes whose source exists)."""
    m = ins.mods
    idx = np.arange(64)
    row, pos = idx // 16, idx % 16
    valid = np.ones(64, bool)
    if "quad_perm" in m:
        q = [int(x) for x in m["quad_perm"].strip("[]").split(",")]
        src = (idx & ~3) + np.array(q)[idx & 3]
    elif "row_shr" in m:
        n = int(m["row_shr"], 0)
        src, valid = idx - n, pos - n >= 0
    elif "row_shl" in m:
        n = int(m["row_shl"], 0)
        src, valid = idx + n, pos + n < 16
    elif "row_ror" in m:
        n = int(m["row_ror"], 0)
        src = row * 16 + (pos - n) % 16
    elif "row_bcast" in m:
        n = int(m["row_bcast"], 0)
        if n == 15:
            src, valid = row * 16 - 1, row >= 1
        elif n == 31:
            src, valid = np.full(64, 31), idx >= 32
        else:
            raise EmuError("row_bcast:%d" % n)
    elif "wave_shr" in m:
        src, valid = idx - 1, idx >= 1
    elif "wave_shl" in m:
        src, valid = idx + 1, idx < 63
    elif "wave_ror" in m:
        src = (idx - 1) % 64
    elif "wave_rol" in m:
        src = (idx + 1) % 64
    elif m.get("row_mirror"):
        src = row * 16 + 15 - pos
    elif m.get("row_half_mirror"):
        src = (idx & ~7) + 7 - (idx & 7)
    else:
        raise EmuError("unknown DPP control in %r" % ins.line)
    src = np.clip(src, 0, 63)
    # a source lane that is switched off in EXEC reads as invalid as well
    valid = valid & exec_lanes[src]
    return val[src], valid


def _dpp_write_mask(ins, w, valid):
    m = ins.mods
    idx = np.arange(64)
    rm = int(m.get("row_mask", "0xf"), 0)
    bm = int(m.get("bank_mask", "0xf"), 0)
    en = (((rm >> (idx // 16)) & 1) == 1) & (((bm >> ((idx % 16) // 4)) & 1) == 1)
    bound = "bound_ctrl" in m      # written bound_ctrl:0 by older assemblers and bound_ctrl:1 by newer ones: the bit is set
    lanes = mask_to_lanes(w.exec) & en
    if not bound:
        lanes = lanes & valid
    return lanes


_SEL = {"BYTE_0": (0, 8), "BYTE_1": (8, 8), "BYTE_2": (16, 8), "BYTE_3": (24, 8), "WORD_0": (0, 16), "WORD_1": (16, 16),
        "DWORD": (0, 32)}


def _sdwa_src(val, sel, sext=False):
    sh, n = _SEL[sel]
    if n == 32:
        return val
    out = (val >> U32(sh)) & U32((1 << n) - 1)
    if sext:
        out = np.where(out >> U32(n - 1) == 1, out | U32((0xFFFFFFFF << n) & 0xFFFFFFFF), out)
    return out


def _cmp(op, a, b):
    return {"lt": a < b, "le": a <= b, "gt": a > b, "ge": a >= b, "eq": a == b, "ne": a != b, "lg": a != b,
            "nlt": ~(a < b), "nle": ~(a <= b), "ngt": ~(a > b), "nge": ~(a >= b), "neq": ~(a == b), "nlg": ~(a != b),
            "o": ~(np.isnan(a) | np.isnan(b)) if a.dtype.kind == "f" else np.ones(64, bool),
            "u": (np.isnan(a) | np.isnan(b)) if a.dtype.kind == "f" else np.zeros(64, bool),
            "t": np.ones(64, bool), "f": np.zeros(64, bool)}[op]


def _fma32(a, b, c):
    with np.errstate(all="ignore"):
        return (a.astype(np.float64) * b.astype(np.float64) + c.astype(np.float64)).astype(np.float32)


_F32_BIN = {
    "v_add_f32": lambda a, b: a + b, "v_sub_f32": lambda a, b: a - b, "v_subrev_f32": lambda a, b: b - a,
    "v_mul_f32": lambda a, b: a * b, "v_max_f32": lambda a, b: np.fmax(a, b), "v_min_f32": lambda a, b: np.fmin(a, b),
    "v_mul_legacy_f32": lambda a, b: np.where((a == 0) | (b == 0), np.float32(0), a * b),
}
_F32_UN = {
    "v_exp_f32": lambda a: np.exp2(a), "v_log_f32": lambda a: np.log2(a), "v_rcp_f32": lambda a: np.float32(1) / a,
    "v_rcp_iflag_f32": lambda a: np.float32(1) / a, "v_rsq_f32": lambda a: np.float32(1) / np.sqrt(a),
    "v_sqrt_f32": lambda a: np.sqrt(a), "v_rndne_f32": lambda a: np.rint(a), "v_trunc_f32": lambda a: np.trunc(a),
    "v_floor_f32": lambda a: np.floor(a), "v_ceil_f32": lambda a: np.ceil(a), "v_fract_f32": lambda a: a - np.floor(a),
}
_U32_BIN = {
    "v_add_u32": lambda a, b: a + b, "v_sub_u32": lambda a, b: a - b, "v_subrev_u32": lambda a, b: b - a,
    "v_and_b32": lambda a, b: a & b, "v_or_b32": lambda a, b: a | b, "v_xor_b32": lambda a, b: a ^ b,
    "v_lshlrev_b32": lambda a, b: b << (a & U32(31)), "v_lshrrev_b32": lambda a, b: b >> (a & U32(31)),
    "v_ashrrev_i32": lambda a, b: (i32(b) >> (a & U32(31)).astype(np.int32)).view(U32),
    "v_mul_lo_u32": lambda a, b: (a.astype(np.uint64) * b.astype(np.uint64)).astype(U32),
    "v_mul_hi_u32": lambda a, b: ((a.astype(np.uint64) * b.astype(np.uint64)) >> np.uint64(32)).astype(U32),
    "v_mul_hi_i32": lambda a, b: ((i32(a).astype(np.int64) * i32(b).astype(np.int64)) >> np.int64(32)).astype(np.int32).view(U32),
    "v_mul_u32_u24": lambda a, b: ((a & U32(0xFFFFFF)).astype(np.uint64) * (b & U32(0xFFFFFF)).astype(np.uint64)).astype(U32),
    "v_mul_i32_i24": lambda a, b: ((((a << U32(8)).view(np.int32) >> 8).astype(np.int64)) * (((b << U32(8)).view(np.int32) >> 8).astype(np.int64))).astype(np.int32).view(U32),
    "v_max_i32": lambda a, b: np.maximum(i32(a), i32(b)).view(U32), "v_min_i32": lambda a, b: np.minimum(i32(a), i32(b)).view(U32),
    "v_max_u32": lambda a, b: np.maximum(a, b), "v_min_u32": lambda a, b: np.minimum(a, b),
}
_U32_TRI = {
    "v_add3_u32": lambda a, b, c: a + b + c, "v_lshl_add_u32": lambda a, b, c: (a << (b & U32(31))) + c,
    "v_add_lshl_u32": lambda a, b, c: (a + b) << (c & U32(31)), "v_lshl_or_b32": lambda a, b, c: (a << (b & U32(31))) | c,
    "v_and_or_b32": lambda a, b, c: (a & b) | c, "v_or3_b32": lambda a, b, c: a | b | c,
    "v_xad_u32": lambda a, b, c: (a ^ b) + c, "v_bfi_b32": lambda a, b, c: (a & b) | (~a & c),
    "v_mad_u32_u24": lambda a, b, c: ((a & U32(0xFFFFFF)).astype(np.uint64) * (b & U32(0xFFFFFF)).astype(np.uint64)).astype(U32) + c,
    "v_bfe_u32": lambda a, b, c: (a >> (b & U32(31))) & ((U32(1) << (c & U32(31))) - U32(1)),
    "v_alignbit_b32": lambda a, b, c: (((a.astype(np.uint64) << np.uint64(32)) | b.astype(np.uint64)) >> (c & U32(31)).astype(np.uint64)).astype(U32),
    "v_alignbyte_b32": lambda a, b, c: (((a.astype(np.uint64) << np.uint64(32)) | b.astype(np.uint64)) >> ((c & U32(3)) * U32(8)).astype(np.uint64)).astype(U32),
}


def _perm_b32(a, b, sel):
    """v_perm_b32: bytes of {a (high dword), b (low dword)} selected by each byte of sel."""
    src = np.stack([(b >> U32(8 * k)) & U32(0xFF) for k in range(4)] + [(a >> U32(8 * k)) & U32(0xFF) for k in range(4)])
    out = np.zeros(64, dtype=U32)
    for k in range(4):
        s = (sel >> U32(8 * k)) & U32(0xFF)
        byte = np.zeros(64, dtype=U32)
        for lane in range(64):
            sv = int(s[lane])
            if sv <= 7:
                byte[lane] = src[sv, lane]
            elif sv == 0x0C:
                byte[lane] = 0
            elif sv >= 0x0D:
                byte[lane] = 0xFF
            else:  # 8..11: sign of a byte pair
                hi = [1, 3, 5, 7][sv - 8]
                byte[lane] = 0xFF if (src[hi, lane] & 0x80) else 0
        out |= byte << U32(8 * k)
    return out


def _offset(ins):
    return int(ins.mods.get("offset", "0"), 0)


def _global_addr(ex, w, ins, addr_tok, base_tok):
    if base_tok == "off":
        a = ex.vread(w, addr_tok, 64)
    else:
        a = ex.vread(w, addr_tok, 32).astype(np.uint64) + np.uint64(ex.sread(w, base_tok, 64))
    return a + np.uint64(_offset(ins) & 0xFFFFFFFFFFFFFFFF)


_LOAD_W = {"ubyte": 1, "sbyte": 1, "ushort": 2, "sshort": 2, "dword": 4, "dwordx2": 8, "dwordx3": 12, "dwordx4": 16,
           "short_d16": 2, "short_d16_hi": 2, "ubyte_d16": 1, "ubyte_d16_hi": 1, "sbyte_d16": 1, "sbyte_d16_hi": 1}
_STORE_W = {"byte": 1, "short": 2, "dword": 4, "dwordx2": 8, "dwordx3": 12, "dwordx4": 16, "short_d16_hi": 2, "byte_d16_hi": 1}


def _land(ex, w, ins, kind, act, raw):
    """Write loaded bytes raw [n, width] of the active lanes `act` into the destination registers."""
    width = _LOAD_W[kind]
    i, n = ex.vindex(ins.ops[0])
    if width >= 4:
        words = np.ascontiguousarray(raw).view(U32).reshape(len(act), width // 4)
        for k in range(width // 4):
            w.v[i + k][act] = words[:, k]
        return
    if width == 2:
        val = raw[:, 0].astype(U32) | (raw[:, 1].astype(U32) << U32(8))
        if kind == "sshort":
            val = np.where(val & U32(0x8000), val | U32(0xFFFF0000), val)
    else:
        val = raw[:, 0].astype(U32)
        if kind.startswith("sbyte"):
            val = np.where(val & U32(0x80), val | U32(0xFFFFFF00), val)
    if kind.endswith("d16_hi"):
        w.v[i][act] = (w.v[i][act] & U32(0xFFFF)) | ((val & U32(0xFFFF)) << U32(16))
    elif kind.endswith("d16"):
        w.v[i][act] = (w.v[i][act] & U32(0xFFFF0000)) | (val & U32(0xFFFF))
    else:
        w.v[i][act] = val


def _lift(ex, w, kind, act, data_tok):
    """Bytes [n, width] the active lanes store from the data registers."""
    width = _STORE_W[kind]
    i, n = ex.vindex(data_tok)
    if width >= 4:
        words = np.stack([w.v[i + k][act] for k in range(width // 4)], axis=1)
        return np.ascontiguousarray(words).view(np.uint8).reshape(len(act), width)
    val = w.v[i][act]
    if kind.endswith("d16_hi"):
        val = val >> U32(16)
    return np.stack([((val >> U32(8 * k)) & U32(0xFF)).astype(np.uint8) for k in range(width)], axis=1)


def _do_load(ex, w, ins, kind, addrs, lanes, space):
    width = _LOAD_W[kind]
    act = np.nonzero(lanes)[0]
    if len(act) == 0:
        return
    if space == "global":
        raw = ex.mem.load(addrs[act], width, ins.line)
    else:
        raw, ix = ex.lds_get(w, ins, addrs[act], width)
        i, n = ex.vindex(ins.ops[0])
        ex.issue(w, "lds_q", vregs=range(i, i + max(n, (width + 3) // 4)), fetch=ix)
    _land(ex, w, ins, kind, act, raw)


def _do_store(ex, w, ins, kind, addrs, lanes, data_tok, space):
    width = _STORE_W[kind]
    act = np.nonzero(lanes)[0]
    if len(act) == 0:
        return
    raw = _lift(ex, w, kind, act, data_tok)
    if space == "global":
        ex.mem.store(addrs[act], raw, ins.line)
    else:
        ex.issue(w, "lds_q", fill=ex.lds_put(w, ins, addrs[act], raw))


def _scc_logic(w, val):
    w.scc = 1 if val != 0 else 0


def step(ex, w):
    """Execute the instruction at w.pc.  Returns nothing; sets w.done / w.at_barrier."""
    ins = ex.prog.instrs[w.pc]
    w.pc += 1
    op, base, ops, mods = ins.op, ins.base, ins.ops, ins.mods
    S = ex.sread
    if ex.strict:
        if ins.wait is not None:
            ex.wait(w, ins.wait)
            return
        ex.check_registers(w, ins)
    # ------------------------------------------------------------------ no-ops and control
    if op in ("s_waitcnt", "s_nop", "s_sleep", "s_setprio") or op.startswith(("s_waitcnt", "s_setprio", "s_nop")):
        return
    if op == "s_endpgm":
        w.done = True
        return
    if op == "s_barrier":
        w.at_barrier = True
        return
    if op == "s_branch":
        w.pc = ex.prog.labels[ops[0]]
        return
    if op.startswith("s_cbranch_"):
        cond = {"s_cbranch_scc0": w.scc == 0, "s_cbranch_scc1": w.scc == 1, "s_cbranch_vccz": w.vcc == 0,
                "s_cbranch_vccnz": w.vcc != 0, "s_cbranch_execz": w.exec == 0, "s_cbranch_execnz": w.exec != 0}[op]
        if cond:
            w.pc = ex.prog.labels[ops[0]]
        return
    # ------------------------------------------------------------------ scalar memory
    if op.startswith("s_load_dword"):
        n = {"s_load_dword": 1, "s_load_dwordx2": 2, "s_load_dwordx4": 4, "s_load_dwordx8": 8, "s_load_dwordx16": 16}[op]
        addr = S(w, ops[1], 64)
        off = ops[2] if len(ops) > 2 else "0"
        addr += S(w, off, 32) if ex.sreg_index(off) is not None else int(off, 0)
        raw = ex.mem.load(np.array([addr], dtype=np.uint64), 4 * n, ins.line)[0]
        words = np.ascontiguousarray(raw).view(U32)
        i, _ = ex.sreg_index(ops[0])
        w.s[i:i + n] = words
        ex.issue(w, "smem_q", sregs=range(i, i + n))
        return
    # ------------------------------------------------------------------ scalar ALU
    if op.startswith("s_"):
        return _salu(ex, w, ins)
    # ------------------------------------------------------------------ vector memory
    if op.startswith("global_load_lds_"):
        kind = op[len("global_load_lds_"):]
        width = _LOAD_W[kind]
        addrs = _global_addr(ex, w, ins, ops[0], ops[1])
        lanes = mask_to_lanes(w.exec)
        act = np.nonzero(lanes)[0]
        raw = ex.mem.load(addrs[act], width, ins.line)
        # LDS address: M0 base + instruction offset + lane * width (each lane's data lands consecutively)
        base_lds = (int(w.s[124]) & 0x3FFFF) + _offset(ins)   # the instruction offset moves both addresses
        a = base_lds + act.astype(np.int64) * width
        ex.issue(w, "vm_q", fill=ex.lds_put(w, ins, a, raw, dma=True))
        return
    if op.startswith("global_load_"):
        kind = op[len("global_load_"):]
        addrs = _global_addr(ex, w, ins, ops[1], ops[2])
        _do_load(ex, w, ins, kind, addrs, mask_to_lanes(w.exec), "global")
        i, n = ex.vindex(ops[0])
        ex.issue(w, "vm_q", vregs=range(i, i + max(n, (_LOAD_W[kind] + 3) // 4)))
        return
    if op.startswith("global_store_"):
        kind = op[len("global_store_"):]
        addrs = _global_addr(ex, w, ins, ops[0], ops[2])
        _do_store(ex, w, ins, kind, addrs, mask_to_lanes(w.exec), ops[1], "global")
        ex.issue(w, "vm_q")
        return
    if op.startswith("global_atomic_"):
        return _global_atomic(ex, w, ins)
    if op.startswith("scratch_"):
        return _scratch(ex, w, ins)
    if op.startswith("ds_"):
        return _ds(ex, w, ins)
    if op.startswith("v_"):
        return _valu(ex, w, ins)
    raise EmuError("unknown instruction: %r" % ins.line)


def _sext(v, bits):
    v &= (1 << bits) - 1
    return v - (1 << bits) if v >> (bits - 1) else v


def _salu(ex, w, ins):
    op, ops = ins.op, ins.ops
    S, W = ex.sread, ex.swrite
    M32, M64 = 0xFFFFFFFF, 0xFFFFFFFFFFFFFFFF
    if op in ("s_mov_b32", "s_movk_i32"):
        v = S(w, ops[1], 32)
        if op == "s_movk_i32":
            v = _sext(v, 16) & M32
        return W(w, ops[0], v)
    if op == "s_mov_b64":
        return W(w, ops[0], S(w, ops[1], 64), 64)
    if op in ("s_cmov_b32",):
        if w.scc:
            W(w, ops[0], S(w, ops[1], 32))
        return
    if op in ("s_add_u32", "s_add_i32", "s_sub_u32", "s_sub_i32", "s_addc_u32", "s_subb_u32"):
        a, b = S(w, ops[1], 32), S(w, ops[2], 32)
        if op == "s_add_u32":
            r = a + b
            w.scc = 1 if r > M32 else 0
        elif op == "s_addc_u32":
            r = a + b + w.scc
            w.scc = 1 if r > M32 else 0
        elif op == "s_sub_u32":
            r = a - b
            w.scc = 1 if b > a else 0
        elif op == "s_subb_u32":
            r = a - b - w.scc
            w.scc = 1 if b + w.scc > a else 0
        elif op == "s_add_i32":
            r = _sext(a, 32) + _sext(b, 32)
            w.scc = 1 if not (-(1 << 31) <= r < (1 << 31)) else 0
        else:
            r = _sext(a, 32) - _sext(b, 32)
            w.scc = 1 if not (-(1 << 31) <= r < (1 << 31)) else 0
        return W(w, ops[0], r & M32)
    if op in ("s_addk_i32", "s_mulk_i32"):
        a, k = _sext(S(w, ops[0], 32), 32), _sext(S(w, ops[1], 32), 16)
        r = a + k if op == "s_addk_i32" else a * k
        if op == "s_addk_i32":
            w.scc = 1 if not (-(1 << 31) <= r < (1 << 31)) else 0
        return W(w, ops[0], r & M32)
    if op == "s_mul_i32":
        return W(w, ops[0], (S(w, ops[1], 32) * S(w, ops[2], 32)) & M32)
    if op == "s_mul_hi_u32":
        return W(w, ops[0], (S(w, ops[1], 32) * S(w, ops[2], 32)) >> 32)
    if op == "s_mul_hi_i32":
        return W(w, ops[0], ((_sext(S(w, ops[1], 32), 32) * _sext(S(w, ops[2], 32), 32)) >> 32) & M32)
    if op in ("s_lshl_b32", "s_lshr_b32", "s_ashr_i32"):
        a, n = S(w, ops[1], 32), S(w, ops[2], 32) & 31
        r = (a << n) & M32 if op == "s_lshl_b32" else (a >> n if op == "s_lshr_b32" else (_sext(a, 32) >> n) & M32)
        _scc_logic(w, r)
        return W(w, ops[0], r)
    if op in ("s_lshl_b64", "s_lshr_b64", "s_ashr_i64"):
        a, n = S(w, ops[1], 64), S(w, ops[2], 32) & 63
        r = (a << n) & M64 if op == "s_lshl_b64" else (a >> n if op == "s_lshr_b64" else (_sext(a, 64) >> n) & M64)
        _scc_logic(w, r)
        return W(w, ops[0], r, 64)
    m = re.match(r"^s_lshl(\d)_add_u32$", op)
    if m:
        r = (S(w, ops[1], 32) << int(m.group(1))) + S(w, ops[2], 32)
        w.scc = 1 if r > M32 else 0
        return W(w, ops[0], r & M32)
    m = re.match(r"^s_(and|or|xor|andn2|orn2|nand|nor|xnor)_b(32|64)$", op)
    if m:
        bits = int(m.group(2))
        mask = M32 if bits == 32 else M64
        a, b = S(w, ops[1], bits), S(w, ops[2], bits)
        r = {"and": a & b, "or": a | b, "xor": a ^ b, "andn2": a & ~b, "orn2": a | ~b, "nand": ~(a & b), "nor": ~(a | b),
             "xnor": ~(a ^ b)}[m.group(1)] & mask
        _scc_logic(w, r)
        return W(w, ops[0], r, bits)
    m = re.match(r"^s_not_b(32|64)$", op)
    if m:
        bits = int(m.group(1))
        r = ~S(w, ops[1], bits) & (M32 if bits == 32 else M64)
        _scc_logic(w, r)
        return W(w, ops[0], r, bits)
    m = re.match(r"^s_(and|or|xor|andn2|orn2|andn1|orn1)_saveexec_b64$", op)
    if m:
        src, old = S(w, ops[1], 64), w.exec
        new = {"and": src & old, "or": src | old, "xor": src ^ old, "andn2": src & ~old, "orn2": src | ~old,
               "andn1": ~src & old, "orn1": ~src | old}[m.group(1)] & M64
        W(w, ops[0], old, 64)
        w.exec = new
        _scc_logic(w, new)
        return
    if op == "s_abs_i32":
        r = abs(_sext(S(w, ops[1], 32), 32)) & M32
        _scc_logic(w, r)
        return W(w, ops[0], r)
    m = re.match(r"^s_(min|max)_(i|u)32$", op)
    if m:
        a, b = S(w, ops[1], 32), S(w, ops[2], 32)
        if m.group(2) == "i":
            a, b = _sext(a, 32), _sext(b, 32)
        r = min(a, b) if m.group(1) == "min" else max(a, b)
        w.scc = 1 if r == a else 0
        return W(w, ops[0], r & M32)
    if op in ("s_cselect_b32", "s_cselect_b64"):
        bits = 64 if op.endswith("64") else 32
        return W(w, ops[0], S(w, ops[1], bits) if w.scc else S(w, ops[2], bits), bits)
    m = re.match(r"^s_cmp(k?)_(eq|lg|gt|ge|lt|le)_(i32|u32|u64)$", op)
    if m:
        bits = 64 if m.group(3) == "u64" else 32
        a, b = S(w, ops[0], bits), S(w, ops[1], bits)
        if m.group(1) == "k":
            b = _sext(b, 16) & M32 if m.group(3) == "i32" else b & 0xFFFF
        if m.group(3) == "i32":
            a, b = _sext(a, 32), _sext(b, 32)
        w.scc = 1 if {"eq": a == b, "lg": a != b, "gt": a > b, "ge": a >= b, "lt": a < b, "le": a <= b}[m.group(2)] else 0
        return
    m = re.match(r"^s_bitcmp([01])_b(32|64)$", op)
    if m:
        bit = (S(w, ops[0], int(m.group(2))) >> (S(w, ops[1], 32) & (int(m.group(2)) - 1))) & 1
        w.scc = 1 if bit == int(m.group(1)) else 0
        return
    if op in ("s_bfe_u32", "s_bfe_i32", "s_bfe_u64", "s_bfe_i64"):
        bits = 64 if op.endswith("64") else 32
        a, c = S(w, ops[1], bits), S(w, ops[2], 32)
        off, wd = c & (bits - 1), (c >> 16) & 0x7F
        r = (a >> off) & ((1 << wd) - 1)
        if op[6] == "i" and wd and (r >> (wd - 1)) & 1:
            r |= ((1 << bits) - 1) & ~((1 << wd) - 1)
        _scc_logic(w, r)
        return W(w, ops[0], r, bits)
    if op in ("s_bcnt1_i32_b32", "s_bcnt1_i32_b64"):
        r = bin(S(w, ops[1], 64 if op.endswith("64") else 32)).count("1")
        _scc_logic(w, r)
        return W(w, ops[0], r)
    if op in ("s_ff1_i32_b32", "s_ff1_i32_b64"):
        a = S(w, ops[1], 64 if op.endswith("64") else 32)
        return W(w, ops[0], ((a & -a).bit_length() - 1) & M32 if a else M32)
    if op in ("s_flbit_i32_b32", "s_flbit_i32_b64"):
        bits = 64 if op.endswith("64") else 32
        a = S(w, ops[1], bits)
        return W(w, ops[0], (bits - a.bit_length()) if a else M32)
    if op == "s_flbit_i32":
        a = S(w, ops[1], 32)
        x = a ^ 0xFFFFFFFF if a >> 31 else a
        return W(w, ops[0], (32 - x.bit_length()) if x else M32)
    if op == "s_sext_i32_i16":
        return W(w, ops[0], _sext(S(w, ops[1], 32), 16) & M32)
    if op == "s_sext_i32_i8":
        return W(w, ops[0], _sext(S(w, ops[1], 32), 8) & M32)
    if op == "s_pack_ll_b32_b16":
        return W(w, ops[0], (S(w, ops[1], 32) & 0xFFFF) | ((S(w, ops[2], 32) & 0xFFFF) << 16))
    if op == "s_pack_lh_b32_b16":
        return W(w, ops[0], (S(w, ops[1], 32) & 0xFFFF) | (S(w, ops[2], 32) & 0xFFFF0000))
    if op == "s_pack_hh_b32_b16":
        return W(w, ops[0], (S(w, ops[1], 32) >> 16) | (S(w, ops[2], 32) & 0xFFFF0000))
    if op == "s_brev_b32":
        return W(w, ops[0], int("{:032b}".format(S(w, ops[1], 32))[::-1], 2))
    raise EmuError("unknown scalar instruction: %r" % ins.line)


# ---------------------------------------------------------------------------------------------------------------
# vector ALU
# ---------------------------------------------------------------------------------------------------------------
def _strip(tok):
    neg = ab = sext = False
    t = tok
    if t.startswith("-") and not re.match(r"^-[\d.]", t):
        neg, t = True, t[1:]
    if t.startswith("neg(") and t.endswith(")"):
        neg, t = True, t[4:-1]
    if t.startswith("|") and t.endswith("|"):
        ab, t = True, t[1:-1]
    if t.startswith("abs(") and t.endswith(")"):
        ab, t = True, t[4:-1]
    if t.startswith("sext(") and t.endswith(")"):
        sext, t = True, t[5:-1]
    return t, neg, ab, sext


def _typed(kind, raw):
    if kind == "f32":
        return f32(raw)
    if kind == "f16":
        return f16_to_f32(raw & U32(0xFFFF))
    if kind in ("u32", "b32"):
        return raw
    if kind == "i32":
        return i32(raw)
    if kind in ("u64", "b64"):
        return raw
    if kind == "i64":
        return raw.view(np.int64)
    if kind == "f64":
        return raw.view(np.float64)
    if kind == "u16":
        return raw & U32(0xFFFF)
    if kind == "i16":
        return (raw & U32(0xFFFF)).astype(np.uint16).view(np.int16).astype(np.int32)
    raise EmuError("operand kind %r" % kind)


def _untyped(kind, val):
    if kind == "f32":
        return u32(val)
    if kind == "f16":
        return f16_bits(val)
    if kind in ("u32", "b32"):
        return np.asarray(val).astype(U32)
    if kind == "i32":
        return np.asarray(val).astype(np.int32).view(U32)
    if kind in ("u64", "b64"):
        return np.asarray(val).astype(np.uint64)
    if kind == "i64":
        return np.asarray(val).astype(np.int64).view(np.uint64)
    if kind == "f64":
        return np.asarray(val, dtype=np.float64).view(np.uint64)
    if kind in ("u16", "i16"):
        return np.asarray(val).astype(np.int64).astype(np.uint64).astype(U32) & U32(0xFFFF)
    raise EmuError("result kind %r" % kind)


class _V:
    """Source/destination access of one vector instruction with its encoding's extras (DPP, SDWA, modifiers)."""

    def __init__(self, ex, w, ins):
        self.ex, self.w, self.ins = ex, w, ins
        self.exec_lanes = mask_to_lanes(w.exec)
        self.write_lanes = self.exec_lanes
        self.dpp = "dpp" in ins.enc
        self.sdwa = "sdwa" in ins.enc
        self.dpp_valid = None

    def raw(self, tok, pos, bits=32, fkind="f32"):
        t, neg, ab, sext = _strip(tok)
        r = self.ex.vindex(t)
        if r is not None:
            i, _ = r
            if bits == 64:
                val = self.w.v[i].astype(np.uint64) | (self.w.v[i + 1].astype(np.uint64) << np.uint64(32))
            else:
                val = self.w.v[i].copy()
        else:
            sv = self.ex.sread(self.w, t, bits, fkind)
            val = np.full(64, sv, dtype=np.uint64 if bits == 64 else U32)
        if self.dpp and pos == 0:
            val, valid = _dpp_source(self.ins, self.w, val, self.exec_lanes)
            self.dpp_valid = valid
            self.write_lanes = _dpp_write_mask(self.ins, self.w, valid)
            val = np.where(valid, val, U32(0))
        if self.sdwa and pos in (0, 1):
            sel = self.ins.mods.get("src%d_sel" % pos, "DWORD")
            val = _sdwa_src(val, sel, sext)
        return val, neg, ab

    def src(self, tok, pos, kind):
        bits = 64 if kind.endswith("64") else 32
        fk = "f16" if kind == "f16" else ("f64" if kind == "f64" else ("f32" if kind == "f32" else "int"))
        val, neg, ab = self.raw(tok, pos, bits, fk)
        t = _typed(kind, val)
        if kind[0] == "f":
            if ab:
                t = np.abs(t)
            if neg:
                t = -t
        elif neg or ab:
            raise EmuError("sign modifier on an integer operand: %r" % self.ins.line)
        return t

    def dst(self, tok, kind, val):
        mods = self.ins.mods
        if kind[0] == "f":
            with np.errstate(all="ignore"):
                if "mul" in mods:
                    val = val * val.dtype.type(int(mods["mul"], 0))
                if "div" in mods:
                    val = val / val.dtype.type(int(mods["div"], 0))
                if mods.get("clamp"):
                    val = np.where(np.isnan(val), 0, np.clip(val, 0, 1)).astype(val.dtype)
        elif mods.get("clamp"):
            raise EmuError("integer clamp is not modelled: %r" % self.ins.line)
        raw = _untyped(kind, val)
        bits = 64 if kind.endswith("64") else 32
        if self.sdwa:
            sel = mods.get("dst_sel", "DWORD")
            if sel != "DWORD":
                sh, n = _SEL[sel]
                i, _ = self.ex.vindex(tok)
                old = self.w.v[i]
                field = (raw & U32((1 << n) - 1)) << U32(sh)
                unused = mods.get("dst_unused", "UNUSED_PAD")
                keep = U32(~(((1 << n) - 1) << sh) & 0xFFFFFFFF)
                if unused == "UNUSED_PRESERVE":
                    raw = (old & keep) | field
                elif unused == "UNUSED_SEXT":
                    sign = (raw >> U32(n - 1)) & U32(1)
                    above = U32((0xFFFFFFFF << (sh + n)) & 0xFFFFFFFF)
                    raw = field | np.where(sign == 1, above, U32(0))
                else:
                    raw = field
        self.ex.vwrite(self.w, tok, raw, lanes_to_mask(self.write_lanes), bits)

    def mask_out(self, tok, bools):
        """Write a lane mask to an SGPR pair (or vcc): inactive lanes give 0."""
        self.ex.swrite(self.w, tok, lanes_to_mask(bools & self.exec_lanes), 64)

    def mask_in(self, tok):
        return mask_to_lanes(self.ex.sread(self.w, tok, 64))


def _class_f32(x, mask):
    u = u32(x)
    e = (u >> U32(23)) & U32(0xFF)
    man = u & U32(0x7FFFFF)
    neg = (u >> U32(31)) == 1
    nan = (e == 255) & (man != 0)
    snan = nan & ((man >> U32(22)) == 0)
    qnan = nan & ~snan
    inf = (e == 255) & (man == 0)
    zero = (e == 0) & (man == 0)
    den = (e == 0) & (man != 0)
    norm = (e != 0) & (e != 255)
    cls = [snan, qnan, neg & inf, neg & norm, neg & den, neg & zero, ~neg & zero, ~neg & den, ~neg & norm, ~neg & inf]
    out = np.zeros(64, bool)
    for bit, c in enumerate(cls):
        out |= (((mask >> U32(bit)) & U32(1)) == 1) & c
    return out


def _exp_of(x):
    return ((u32(x) >> U32(23)) & U32(0xFF)).astype(np.int32)


def _div_scale_f32(s0, s1, s2):
    """v_div_scale_f32: returns (result, vcc lanes).  s1 = denominator, s2 = numerator, s0 = the one being scaled."""
    with np.errstate(all="ignore"):
        out = s0.copy()
        vcc = np.zeros(64, bool)
        e1, e2 = _exp_of(s1), _exp_of(s2)
        up = np.ldexp(s0, 64).astype(np.float32)
        down = np.ldexp(s0, -64).astype(np.float32)
        same_den = u32(s0) == u32(s1)
        same_num = u32(s0) == u32(s2)
        nanres = (s2 == 0) | (s1 == 0)
        big = (e2 - e1) >= 96
        den1 = (e1 == 0)
        rcp_den = e1 >= 253
        quo_den = (e2 - e1) <= -126
        tiny_num = e2 <= 23
        done = np.zeros(64, bool)

        def take(cond, val=None, setvcc=False, only=None):
            nonlocal out, vcc, done
            c = cond & ~done
            if setvcc:
                vcc = vcc | c
            if val is not None:
                sel = c if only is None else (c & only)
                out = np.where(sel, val, out)
            done = done | c

        take(nanres, np.full(64, np.nan, np.float32))
        take(big, up, True, same_den)
        take(den1, up)
        take(rcp_den & quo_den, up, True, same_den)
        take(rcp_den, down)
        take(quo_den, up, True, same_num)
        take(tiny_num, up)
        return out, vcc


def _div_fixup_f32(q, den, num):
    with np.errstate(all="ignore"):
        sign = (u32(den) ^ u32(num)) & U32(0x80000000)
        inf = (U32(0x7F800000) | sign).view(np.float32)
        zero = sign.view(np.float32)
        res = ((u32(q) & U32(0x7FFFFFFF)) | sign).view(np.float32)
        e1, e2 = _exp_of(den), _exp_of(num)
        res = np.where((e2 - e1) < -150, zero, res)
        res = np.where(np.isinf(den) | (num == 0), zero, res)
        res = np.where((den == 0) | np.isinf(num), inf, res)
        res = np.where(np.isinf(den) & np.isinf(num), np.float32(np.nan), res)
        res = np.where((den == 0) & (num == 0), np.float32(np.nan), res)
        res = np.where(np.isnan(den), den, res)
        res = np.where(np.isnan(num), num, res)
        return res.astype(np.float32)


def _rtz_f16(x):
    """fp32 -> fp16 bits, rounding toward zero."""
    with np.errstate(all="ignore"):
        h = np.asarray(x, np.float32).astype(np.float16)
        over = np.abs(h.astype(np.float32)) > np.abs(x)
        bits = h.view(np.uint16).astype(U32)
        bits = np.where(over & ~np.isnan(x), bits - U32(1), bits)     # one step toward zero (covers inf -> max finite)
        return bits & U32(0xFFFF)


def _cvt_int(x, lo, hi):
    with np.errstate(all="ignore"):
        t = np.trunc(np.where(np.isnan(x), 0, x).astype(np.float64))
        return np.clip(t, lo, hi)


def _valu(ex, w, ins):
    base, ops, mods = ins.base, ins.ops, ins.mods
    V = _V(ex, w, ins)
    lanes = V.exec_lanes
    # ---- moves and lane traffic
    if base == "v_mov_b32":
        return V.dst(ops[0], "b32", V.src(ops[1], 0, "b32"))
    if base == "v_mov_b64":
        return V.dst(ops[0], "b64", V.src(ops[1], 0, "b64"))
    if base in ("v_accvgpr_write_b32", "v_accvgpr_read_b32", "v_accvgpr_mov_b32"):
        return V.dst(ops[0], "b32", V.src(ops[1], 0, "b32"))
    if base == "v_readfirstlane_b32":
        first = int(np.argmax(lanes)) if lanes.any() else 0
        return ex.swrite(w, ops[0], int(V.src(ops[1], 0, "b32")[first]))
    if base == "v_readlane_b32":
        lane = ex.sread(w, ops[2], 32) & 63
        return ex.swrite(w, ops[0], int(V.src(ops[1], 0, "b32")[lane]))
    if base == "v_writelane_b32":
        lane = ex.sread(w, ops[2], 32) & 63
        i, _ = ex.vindex(ops[0])
        w.v[i][lane] = ex.sread(w, ops[1], 32)
        return
    if base == "v_swap_b32":
        a, b = V.src(ops[0], 9, "b32"), V.src(ops[1], 9, "b32")
        V.dst(ops[0], "b32", b)
        return V.dst(ops[1], "b32", a)
    if base in ("v_mbcnt_lo_u32_b32", "v_mbcnt_hi_u32_b32"):
        m = V.src(ops[1], 0, "u32")
        idx = np.arange(64)
        if base == "v_mbcnt_lo_u32_b32":
            below = np.where(idx >= 32, 0xFFFFFFFF, (1 << idx) - 1).astype(np.uint64).astype(U32)
        else:
            below = np.where(idx < 32, 0, (1 << np.maximum(idx - 32, 0)) - 1).astype(np.uint64).astype(U32)
        cnt = np.array([bin(int(x)).count("1") for x in (m & below)], dtype=U32)
        return V.dst(ops[0], "u32", cnt + V.src(ops[2], 1, "u32"))
    if base == "v_cndmask_b32":
        picks = []
        for pos in (0, 1):                       # sign modifiers act on the bit pattern as fp32
            val, neg, ab = V.raw(ops[1 + pos], pos)
            if ab:
                val = val & U32(0x7FFFFFFF)
            if neg:
                val = val ^ U32(0x80000000)
            picks.append(val)
        return V.dst(ops[0], "b32", np.where(V.mask_in(ops[3]), picks[1], picks[0]))
    # ---- compares
    m = re.match(r"^v_cmp(x?)_(class|[a-z]+)_(f16|f32|f64|i16|u16|i32|u32|i64|u64)$", base)
    if m:
        kind = m.group(3)
        a = V.src(ops[1], 0, kind)
        if m.group(2) == "class":
            res = _class_f32(a, V.src(ops[2], 1, "u32"))
        else:
            b = V.src(ops[2], 1, kind)
            with np.errstate(invalid="ignore"):
                res = _cmp(m.group(2), a, b)
        V.mask_out(ops[0], res)
        if m.group(1) == "x":
            w.exec = lanes_to_mask(res & lanes)
        return
    # ---- carries
    m = re.match(r"^v_(add|sub|subrev|addc|subb|subbrev)_co_u32$", base)
    if m:
        kind = m.group(1)
        a = V.src(ops[2], 0, "u32").astype(np.uint64)
        b = V.src(ops[3], 1, "u32").astype(np.uint64)
        cin = V.mask_in(ops[4]).astype(np.uint64) if kind in ("addc", "subb", "subbrev") else np.zeros(64, np.uint64)
        if kind in ("subrev", "subbrev"):
            a, b = b, a
        if kind in ("add", "addc"):
            r = a + b + cin
            carry = r > np.uint64(0xFFFFFFFF)
        else:
            carry = (b + cin) > a
            r = (a - b - cin) & np.uint64(0xFFFFFFFF)
        V.dst(ops[0], "u32", r & np.uint64(0xFFFFFFFF))
        old = V.mask_in(ops[1])
        return ex.swrite(w, ops[1], lanes_to_mask(np.where(lanes, carry, old)), 64)
    if base in ("v_mad_u64_u32", "v_mad_i64_i32"):
        if base == "v_mad_u64_u32":
            a, b = V.src(ops[2], 0, "u32").astype(np.uint64), V.src(ops[3], 1, "u32").astype(np.uint64)
            c = V.src(ops[4], 2, "u64")
            prod = a * b
            r = prod + c
            carry = r < prod
        else:
            a, b = V.src(ops[2], 0, "i32").astype(np.int64), V.src(ops[3], 1, "i32").astype(np.int64)
            c = V.src(ops[4], 2, "i64")
            r = (a * b + c).view(np.uint64)
            carry = np.zeros(64, bool)       # the overflow flag of the signed form is never consumed by compiled code
        V.dst(ops[0], "u64", r)
        if ops[1] not in ("null",):
            ex.swrite(w, ops[1], lanes_to_mask(carry & lanes), 64)
        return
    if base == "v_lshl_add_u64":
        a, sh, c = V.src(ops[1], 0, "u64"), V.src(ops[2], 1, "u32"), V.src(ops[3], 2, "u64")
        return V.dst(ops[0], "u64", (a << (sh & U32(7)).astype(np.uint64)) + c)
    if base in ("v_lshlrev_b64", "v_lshrrev_b64", "v_ashrrev_i64"):
        sh = (V.src(ops[1], 0, "u32") & U32(63)).astype(np.uint64)
        a = V.src(ops[2], 1, "u64")
        r = a << sh if base == "v_lshlrev_b64" else (a >> sh if base == "v_lshrrev_b64" else (a.view(np.int64) >> sh.astype(np.int64)).view(np.uint64))
        return V.dst(ops[0], "u64", r)
    # ---- table-driven 32-bit integer
    if base in _U32_BIN:
        return V.dst(ops[0], "u32", _U32_BIN[base](V.src(ops[1], 0, "u32"), V.src(ops[2], 1, "u32")))
    if base in _U32_TRI:
        return V.dst(ops[0], "u32", _U32_TRI[base](V.src(ops[1], 0, "u32"), V.src(ops[2], 1, "u32"), V.src(ops[3], 2, "u32")))
    if base == "v_not_b32":
        return V.dst(ops[0], "u32", ~V.src(ops[1], 0, "u32"))
    if base == "v_bfe_i32":
        a, off, wd = V.src(ops[1], 0, "u32"), V.src(ops[2], 1, "u32") & U32(31), V.src(ops[3], 2, "u32") & U32(31)
        r = (a >> off) & ((U32(1) << wd) - U32(1))
        sign = np.where(wd > 0, (r >> np.maximum(wd, 1) - U32(1)) & U32(1), 0)
        return V.dst(ops[0], "u32", np.where(sign == 1, r | ~((U32(1) << wd) - U32(1)), r))
    if base == "v_perm_b32":
        return V.dst(ops[0], "u32", _perm_b32(V.src(ops[1], 0, "u32"), V.src(ops[2], 1, "u32"), V.src(ops[3], 2, "u32")))
    if base in ("v_med3_i32", "v_med3_u32", "v_max3_i32", "v_min3_i32", "v_max3_u32", "v_min3_u32"):
        k = "i32" if base.endswith("i32") else "u32"
        st = np.sort(np.stack([V.src(ops[1], 0, k), V.src(ops[2], 1, k), V.src(ops[3], 2, k)]), axis=0)
        return V.dst(ops[0], k, st[{"med3": 1, "max3": 2, "min3": 0}[base[2:6]]])
    if base in ("v_ffbh_u32", "v_ffbl_b32", "v_bcnt_u32_b32"):
        a = V.src(ops[1], 0, "u32")
        if base == "v_bcnt_u32_b32":
            return V.dst(ops[0], "u32", np.array([bin(int(x)).count("1") for x in a], U32) + V.src(ops[2], 1, "u32"))
        if base == "v_ffbh_u32":
            return V.dst(ops[0], "u32", np.array([32 - int(x).bit_length() if x else 0xFFFFFFFF for x in a], dtype=np.uint64))
        return V.dst(ops[0], "u32", np.array([(int(x) & -int(x)).bit_length() - 1 if x else 0xFFFFFFFF for x in a], dtype=np.uint64))
    # ---- fp32
    with np.errstate(all="ignore"):
        if base in _F32_BIN:
            return V.dst(ops[0], "f32", _F32_BIN[base](V.src(ops[1], 0, "f32"), V.src(ops[2], 1, "f32")).astype(np.float32))
        if base in _F32_UN:
            return V.dst(ops[0], "f32", _F32_UN[base](V.src(ops[1], 0, "f32")).astype(np.float32))
        if base == "v_fma_f32" or base == "v_mad_f32":
            return V.dst(ops[0], "f32", _fma32(V.src(ops[1], 0, "f32"), V.src(ops[2], 1, "f32"), V.src(ops[3], 2, "f32")))
        if base in ("v_fmac_f32", "v_mac_f32"):
            return V.dst(ops[0], "f32", _fma32(V.src(ops[1], 0, "f32"), V.src(ops[2], 1, "f32"), V.src(ops[0], 2, "f32")))
        if base == "v_fmamk_f32":
            return V.dst(ops[0], "f32", _fma32(V.src(ops[1], 0, "f32"), V.src(ops[2], 9, "f32"), V.src(ops[3], 1, "f32")))
        if base == "v_fmaak_f32":
            return V.dst(ops[0], "f32", _fma32(V.src(ops[1], 0, "f32"), V.src(ops[2], 1, "f32"), V.src(ops[3], 9, "f32")))
        if base in ("v_max3_f32", "v_min3_f32", "v_med3_f32"):
            a, b, c = V.src(ops[1], 0, "f32"), V.src(ops[2], 1, "f32"), V.src(ops[3], 2, "f32")
            if base == "v_max3_f32":
                r = np.fmax(np.fmax(a, b), c)
            elif base == "v_min3_f32":
                r = np.fmin(np.fmin(a, b), c)
            else:
                r = np.fmax(np.fmin(a, b), np.fmin(np.fmax(a, b), c))
            return V.dst(ops[0], "f32", r)
        if base == "v_ldexp_f32":
            e = np.clip(V.src(ops[2], 1, "i32"), -300, 300)
            return V.dst(ops[0], "f32", np.ldexp(V.src(ops[1], 0, "f32").astype(np.float64), e).astype(np.float32))
        if base == "v_frexp_mant_f32":
            return V.dst(ops[0], "f32", np.frexp(V.src(ops[1], 0, "f32"))[0].astype(np.float32))
        if base == "v_frexp_exp_i32_f32":
            x = V.src(ops[1], 0, "f32")
            return V.dst(ops[0], "i32", np.where(np.isfinite(x) & (x != 0), np.frexp(x)[1], 0))
        if base == "v_div_scale_f32":
            r, vcc = _div_scale_f32(V.src(ops[2], 0, "f32"), V.src(ops[3], 1, "f32"), V.src(ops[4], 2, "f32"))
            V.dst(ops[0], "f32", r)
            return V.mask_out(ops[1], vcc)
        if base == "v_div_fmas_f32":
            r = _fma32(V.src(ops[1], 0, "f32"), V.src(ops[2], 1, "f32"), V.src(ops[3], 2, "f32"))
            scaled = np.ldexp(r.astype(np.float64), 32).astype(np.float32)
            return V.dst(ops[0], "f32", np.where(mask_to_lanes(w.vcc), scaled, r))
        if base == "v_div_fixup_f32":
            return V.dst(ops[0], "f32", _div_fixup_f32(V.src(ops[1], 0, "f32"), V.src(ops[2], 1, "f32"), V.src(ops[3], 2, "f32")))
        # ---- conversions
        if base == "v_cvt_f32_f16":
            return V.dst(ops[0], "f32", V.src(ops[1], 0, "f16"))
        if base == "v_cvt_f16_f32":
            return V.dst(ops[0], "f16", V.src(ops[1], 0, "f32"))
        if base == "v_cvt_f32_u32":
            return V.dst(ops[0], "f32", V.src(ops[1], 0, "u32").astype(np.float32))
        if base == "v_cvt_f32_i32":
            return V.dst(ops[0], "f32", V.src(ops[1], 0, "i32").astype(np.float32))
        if base == "v_cvt_u32_f32":
            return V.dst(ops[0], "u32", _cvt_int(V.src(ops[1], 0, "f32"), 0, 0xFFFFFFFF).astype(np.uint64))
        if base == "v_cvt_i32_f32":
            return V.dst(ops[0], "i32", _cvt_int(V.src(ops[1], 0, "f32"), -(1 << 31), (1 << 31) - 1).astype(np.int64))
        if base in ("v_cvt_f32_ubyte0", "v_cvt_f32_ubyte1", "v_cvt_f32_ubyte2", "v_cvt_f32_ubyte3"):
            k = int(base[-1])
            return V.dst(ops[0], "f32", ((V.src(ops[1], 0, "u32") >> U32(8 * k)) & U32(0xFF)).astype(np.float32))
        if base == "v_cvt_pk_bf16_f32":
            lo, hi = bf16_round(V.src(ops[1], 0, "f32")), bf16_round(V.src(ops[2], 1, "f32"))
            return V.dst(ops[0], "u32", lo | (hi << U32(16)))
        if base == "v_cvt_pk_f16_f32":
            lo, hi = f16_bits(V.src(ops[1], 0, "f32")), f16_bits(V.src(ops[2], 1, "f32"))
            return V.dst(ops[0], "u32", lo | (hi << U32(16)))
        if base == "v_cvt_pkrtz_f16_f32":
            lo, hi = _rtz_f16(V.src(ops[1], 0, "f32")), _rtz_f16(V.src(ops[2], 1, "f32"))
            return V.dst(ops[0], "u32", lo | (hi << U32(16)))
        # ---- mixed precision fma
        if base in ("v_fma_mix_f32", "v_fma_mixlo_f16", "v_fma_mixhi_f16"):
            def bits_list(name):
                t = mods.get(name)
                return [int(x) for x in t.strip("[]").split(",")] if t else [0, 0, 0]
            sel, sel_hi = bits_list("op_sel"), bits_list("op_sel_hi")
            vals = []
            for k in range(3):
                val, neg, ab = V.raw(ops[1 + k], k, 32, "f16" if sel_hi[k] else "f32")
                if sel_hi[k]:
                    x = f16_to_f32((val >> U32(16 if sel[k] else 0)) & U32(0xFFFF))
                else:
                    x = f32(val)
                if ab:
                    x = np.abs(x)
                if neg:
                    x = -x
                vals.append(x)
            r = _fma32(*vals)
            if base == "v_fma_mix_f32":
                return V.dst(ops[0], "f32", r)
            if mods.get("clamp"):
                r = np.where(np.isnan(r), 0, np.clip(r, 0, 1)).astype(np.float32)
            h = f16_bits(r)
            i, _ = ex.vindex(ops[0])
            old = w.v[i]
            new = (old & U32(0xFFFF0000)) | h if base == "v_fma_mixlo_f16" else (old & U32(0xFFFF)) | (h << U32(16))
            return ex.vwrite(w, ops[0], new, lanes_to_mask(V.write_lanes))
    return _valu_more(ex, w, ins, V)


def _reg_block(w, start, count):
    """count consecutive registers from `start` as a [count, 64] view."""
    return w.v[start:start + count]


def _frag16(regs, kind):
    """[n, 64] uint32 registers holding 2n 16-bit values per lane -> float64 [64, 2n] in element order."""
    lo = regs & U32(0xFFFF)
    hi = regs >> U32(16)
    inter = np.empty((regs.shape[0] * 2, 64), dtype=U32)
    inter[0::2], inter[1::2] = lo, hi
    if kind == "bf16":
        vals = (inter << U32(16)).view(np.float32)
    else:
        vals = inter.astype(np.uint16).view(np.float16).astype(np.float32)
    return vals.astype(np.float64).T


def _mfma(ex, w, ins):
    """Matrix instructions.  Lane l = (block b, index i): A holds row i of the M x K operand, K elements b*kv .. b*kv+kv-1;
    B holds column i of the K x N operand, the same K elements; D/C hold column i and rows 8*(r/4) + 4*b + r%4 (32 x 32,
    b = l / 32) or 4*b + r (16 x 16, b = l / 16) in register r."""
    base, ops, mods = ins.base, ins.ops, ins.mods
    for k in ("cbsz", "abid", "blgp"):
        if int(mods.get(k, "0"), 0):
            raise EmuError("MFMA modifier %s is not modelled: %r" % (k, ins.line))
    m = re.match(r"^v_mfma_f32_(\d+)x(\d+)x(\d+)_?(bf16|f16|f32|xf32)$", base)
    if not m:
        raise EmuError("unknown matrix instruction: %r" % ins.line)
    M, N, K, kind = int(m.group(1)), int(m.group(2)), int(m.group(3)), m.group(4)
    if M != N or M not in (16, 32) or kind == "xf32":
        raise EmuError("matrix shape not modelled: %r" % ins.line)
    nb = 64 // M                      # lane blocks
    kv = K // nb                      # K elements per lane
    lanes = np.arange(64)
    idx, blk = lanes % M, lanes // M
    ai, an = ex.vindex(ops[1])
    bi, bn = ex.vindex(ops[2])
    if kind == "f32":
        if an != kv or bn != kv:
            raise EmuError("operand width: %r" % ins.line)
        a = _reg_block(w, ai, an).view(np.float32).astype(np.float64).T
        b = _reg_block(w, bi, bn).view(np.float32).astype(np.float64).T
    else:
        if an * 2 != kv or bn * 2 != kv:
            raise EmuError("operand width: %r" % ins.line)
        a, b = _frag16(_reg_block(w, ai, an), kind), _frag16(_reg_block(w, bi, bn), kind)
    A = np.zeros((M, K))
    B = np.zeros((K, N))
    kk = blk[:, None] * kv + np.arange(kv)[None, :]
    A[idx[:, None], kk] = a
    B[kk, idx[:, None]] = b
    nreg = M * N // 64
    di, dn = ex.vindex(ops[0])
    if dn != nreg:
        raise EmuError("result width: %r" % ins.line)
    r = np.arange(nreg)
    if M == 32:
        rows = 8 * (r[:, None] // 4) + 4 * blk[None, :] + r[:, None] % 4       # [nreg, 64]
    else:
        rows = 4 * blk[None, :] + r[:, None]
    cols = np.broadcast_to(idx[None, :], rows.shape)
    c = ex.vindex(ops[3])
    if c is not None:
        if c[1] != nreg:
            raise EmuError("accumulator width: %r" % ins.line)
        C = _reg_block(w, c[0], nreg).view(np.float32).astype(np.float64)
    else:
        C = np.full((nreg, 64), float(f32(np.array([ex.sread(w, ops[3], 32, "f32")], dtype=U32))[0]))
    with np.errstate(all="ignore"):
        D = (A @ B)[rows, cols] + C
        w.v[di:di + nreg] = D.astype(np.float32).view(U32)      # matrix instructions ignore EXEC


def _bitop3(a, b, c, table):
    out = np.zeros(64, dtype=U32)
    for i in range(8):
        if (table >> i) & 1:
            ta = a if i & 4 else ~a
            tb = b if i & 2 else ~b
            tc = c if i & 1 else ~c
            out |= ta & tb & tc
    return out


def _valu_more(ex, w, ins, V):
    base, ops, mods = ins.base, ins.ops, ins.mods
    if base.startswith("v_mfma_"):
        return _mfma(ex, w, ins)
    if base in ("v_permlane16_swap_b32", "v_permlane32_swap_b32"):
        di, _ = ex.vindex(ops[0])
        si, _ = ex.vindex(ops[1])
        d, s_ = w.v[di].copy(), w.v[si].copy()
        if base == "v_permlane16_swap_b32":
            pairs = ((slice(16, 32), slice(0, 16)), (slice(48, 64), slice(32, 48)))
        else:
            pairs = ((slice(32, 64), slice(0, 32)),)
        nd, ns = d.copy(), s_.copy()
        for dsl, ssl in pairs:
            nd[dsl], ns[ssl] = s_[ssl], d[dsl]
        w.v[di], w.v[si] = nd, ns           # lane swaps ignore EXEC on this target
        return
    if base == "v_bitop3_b32":
        return V.dst(ops[0], "u32", _bitop3(V.src(ops[1], 0, "u32"), V.src(ops[2], 1, "u32"), V.src(ops[3], 2, "u32"),
                                             int(mods["bitop3"], 0)))
    if base == "v_dot2c_f32_f16":
        a, b = V.src(ops[1], 0, "u32"), V.src(ops[2], 1, "u32")
        acc = V.src(ops[0], 2, "f32").astype(np.float64)
        lo = f16_to_f32(a & U32(0xFFFF)).astype(np.float64) * f16_to_f32(b & U32(0xFFFF)).astype(np.float64)
        hi = f16_to_f32(a >> U32(16)).astype(np.float64) * f16_to_f32(b >> U32(16)).astype(np.float64)
        return V.dst(ops[0], "f32", (acc + lo + hi).astype(np.float32))
    m = re.match(r"^v_(add|sub|subrev|mul_lo|lshlrev|lshrrev|max|min)_(u16|b16)$", base)
    if m:
        a, b = V.src(ops[1], 0, "u16"), V.src(ops[2], 1, "u16")
        r = {"add": lambda: a + b, "sub": lambda: a - b, "subrev": lambda: b - a, "mul_lo": lambda: a * b,
             "lshlrev": lambda: b << (a & U32(15)), "lshrrev": lambda: b >> (a & U32(15)), "max": lambda: np.maximum(a, b),
             "min": lambda: np.minimum(a, b)}[m.group(1)]()
        return V.dst(ops[0], "u16", r & U32(0xFFFF))
    if base == "v_pack_b32_f16":
        sel = [int(x) for x in mods["op_sel"].strip("[]").split(",")] if "op_sel" in mods else [0, 0, 0]
        a, b = V.raw(ops[1], 0, 32, "f16")[0], V.raw(ops[2], 1, 32, "f16")[0]
        lo = (a >> U32(16 if sel[0] else 0)) & U32(0xFFFF)
        hi = (b >> U32(16 if sel[1] else 0)) & U32(0xFFFF)
        return V.dst(ops[0], "u32", lo | (hi << U32(16)))
    if base == "v_mad_i32_i24":
        a = ((V.src(ops[1], 0, "u32") << U32(8)).view(np.int32) >> 8).astype(np.int64)
        b = ((V.src(ops[2], 1, "u32") << U32(8)).view(np.int32) >> 8).astype(np.int64)
        return V.dst(ops[0], "i32", (a * b + V.src(ops[3], 2, "i32").astype(np.int64)).astype(np.int64) & 0xFFFFFFFF)
    raise EmuError("unknown vector instruction: %r" % ins.line)


# ---------------------------------------------------------------------------------------------------------------
# LDS, scratch, atomics
# ---------------------------------------------------------------------------------------------------------------
def _lds_bytes(ex, ins, a, width):
    a = a.astype(np.int64)
    if (a < 0).any() or (a + width > ex.lds.size).any():
        raise EmuError("LDS access outside the %d bytes allocated (address %d): %r" %
                       (ex.lds.size, int(a.max()), ins.line))
    return a[:, None] + np.arange(width)[None, :]


def _atomic_apply(name, old, data, cmp=None):
    """One lane's read-modify-write on Python ints / floats.  Returns the new value (32-bit pattern)."""
    M = 0xFFFFFFFF
    if name in ("add", "add_u32"):
        return (old + data) & M
    if name in ("sub", "sub_u32"):
        return (old - data) & M
    if name in ("umax", "max_u32"):
        return max(old, data)
    if name in ("umin", "min_u32"):
        return min(old, data)
    if name in ("smax", "max_i32"):
        return max(_sext(old, 32), _sext(data, 32)) & M
    if name in ("smin", "min_i32"):
        return min(_sext(old, 32), _sext(data, 32)) & M
    if name in ("and", "and_b32"):
        return old & data
    if name in ("or", "or_b32"):
        return old | data
    if name in ("xor", "xor_b32"):
        return old ^ data
    if name in ("swap", "wrxchg_b32"):
        return data
    if name in ("inc", "inc_u32"):
        return 0 if old >= data else old + 1
    if name in ("dec", "dec_u32"):
        return data if (old == 0 or old > data) else old - 1
    if name in ("add_f32",):
        a = np.array([old], dtype=U32).view(np.float32)[0]
        b = np.array([data], dtype=U32).view(np.float32)[0]
        return int(np.array([a + b], dtype=np.float32).view(U32)[0])
    if name in ("fmax", "max_f32"):
        a = np.array([old, data], dtype=U32).view(np.float32)
        return int(np.array([np.fmax(a[0], a[1])], dtype=np.float32).view(U32)[0])
    raise EmuError("atomic %r is not modelled" % name)


def _ds(ex, w, ins):
    op, ops, mods = ins.op, ins.ops, ins.mods
    lanes = mask_to_lanes(w.exec)
    act = np.nonzero(lanes)[0]
    off = _offset(ins)
    m = re.match(r"^ds_read_(b32|b64|b96|b128)$", op)
    if m:
        addrs = ex.vread(w, ops[1], 32).astype(np.int64) + off
        return _do_load(ex, w, ins, {"b32": "dword", "b64": "dwordx2", "b96": "dwordx3", "b128": "dwordx4"}[m.group(1)],
                        addrs, lanes, "lds")
    m = re.match(r"^ds_read_(u8|i8|u16|i16|u16_d16|u16_d16_hi|u8_d16|u8_d16_hi|i8_d16|i8_d16_hi)$", op)
    if m:
        kind = {"u8": "ubyte", "i8": "sbyte", "u16": "ushort", "i16": "sshort", "u16_d16": "short_d16",
                "u16_d16_hi": "short_d16_hi", "u8_d16": "ubyte_d16", "u8_d16_hi": "ubyte_d16_hi", "i8_d16": "sbyte_d16",
                "i8_d16_hi": "sbyte_d16_hi"}[m.group(1)]
        addrs = ex.vread(w, ops[1], 32).astype(np.int64) + off
        return _do_load(ex, w, ins, kind, addrs, lanes, "lds")
    m = re.match(r"^ds_write_(b32|b64|b96|b128|b8|b16|b16_d16_hi|b8_d16_hi)$", op)
    if m:
        kind = {"b32": "dword", "b64": "dwordx2", "b96": "dwordx3", "b128": "dwordx4", "b8": "byte", "b16": "short",
                "b16_d16_hi": "short_d16_hi", "b8_d16_hi": "byte_d16_hi"}[m.group(1)]
        addrs = ex.vread(w, ops[0], 32).astype(np.int64) + off
        return _do_store(ex, w, ins, kind, addrs, lanes, ops[1], "lds")
    m = re.match(r"^ds_(read|write)2(st64)?_(b32|b64)$", op)
    if m:
        width = 4 if m.group(3) == "b32" else 8
        unit = width * (64 if m.group(2) else 1)
        o0 = int(mods.get("offset0", "0"), 0) * unit
        o1 = int(mods.get("offset1", "0"), 0) * unit
        nd = width // 4
        if m.group(1) == "read":
            base = ex.vread(w, ops[1], 32).astype(np.int64)
            i, _ = ex.vindex(ops[0])
            fetched = []
            for k, o in enumerate((o0, o1)):
                raw, ix = ex.lds_get(w, ins, base[act] + o, width)
                words = np.ascontiguousarray(raw).view(U32).reshape(len(act), nd)
                for d in range(nd):
                    w.v[i + k * nd + d][act] = words[:, d]
                fetched.append(ix)
            ex.issue(w, "lds_q", vregs=range(i, i + 2 * nd), fetch=np.concatenate([f.ravel() for f in fetched]))
        else:
            base = ex.vread(w, ops[0], 32).astype(np.int64)
            filled = []
            for k, o in enumerate((o0, o1)):
                i, _ = ex.vindex(ops[1 + k])
                words = np.stack([w.v[i + d][act] for d in range(nd)], axis=1)
                filled.append(ex.lds_put(w, ins, base[act] + o, np.ascontiguousarray(words).view(np.uint8).reshape(len(act), width)))
            ex.issue(w, "lds_q", fill=np.concatenate([f.ravel() for f in filled]))
        return
    if op in ("ds_bpermute_b32", "ds_permute_b32"):
        addr = ((ex.vread(w, ops[1], 32).astype(np.int64) + off) >> 2) & 63
        data = ex.vread(w, ops[2], 32)
        if op == "ds_bpermute_b32":
            res = np.where(lanes[addr], data[addr], U32(0))
        else:
            res = np.zeros(64, dtype=U32)
            for lane in act:                       # later lanes win, as the hardware's write order does
                res[addr[lane]] = data[lane]
        ex.vwrite(w, ops[0], res)
        return ex.issue(w, "lds_q", vregs=(ex.vindex(ops[0])[0],))
    if op == "ds_swizzle_b32":
        pat = off
        data = ex.vread(w, ops[1], 32)
        idx = np.arange(64)
        if pat & 0x8000:                            # quad permute
            src = (idx & ~3) | ((pat >> (2 * (idx & 3))) & 3)
        else:
            and_m, or_m, xor_m = pat & 31, (pat >> 5) & 31, (pat >> 10) & 31
            src = (idx & 32) | ((((idx & 31) & and_m) | or_m) ^ xor_m)
        ex.vwrite(w, ops[0], np.where(lanes[src], data[src], U32(0)))
        return ex.issue(w, "lds_q", vregs=(ex.vindex(ops[0])[0],))
    if op == "ds_read_b64_tr_b16":
        # Each group of 16 lanes holds a 16 x 16 block of 16-bit elements, lane r of the group addressing 4 consecutive
        # elements of row (r % 16)... lane i of the group reads its own 8 bytes; the result for lane i, element j is the
        # element that lane (4 * j' ...) supplied.  Transposition: within a group, treat the 16 lanes x 4 elements as a
        # 16 x 4 matrix per lane-quad-block and redistribute so that lane i receives element (i % 4 ... ).
        return _ds_read_tr16(ex, w, ins)
    m = re.match(r"^ds_(add|sub|max|min|and|or|xor|inc|dec|wrxchg)(_rtn)?_(u32|i32|b32|f32)$", op)
    if m:
        rtn = bool(m.group(2))
        a_tok, d_tok = (ops[1], ops[2]) if rtn else (ops[0], ops[1])
        addrs = ex.vread(w, a_tok, 32).astype(np.int64) + off
        data = ex.vread(w, d_tok, 32)
        name = "%s_%s" % (m.group(1), m.group(3))
        out = np.zeros(64, dtype=U32)
        for lane in act:                      # atomics are the sanctioned way to share bytes without a barrier: not tracked
            ix = _lds_bytes(ex, ins, addrs[lane:lane + 1], 4)
            old = int(np.ascontiguousarray(ex.lds[ix]).view(U32)[0, 0])
            new = _atomic_apply(name, old, int(data[lane]))
            ex.lds[ix] = np.array([new], dtype=U32).view(np.uint8).reshape(1, 4)
            out[lane] = old
        if rtn:
            ex.vwrite(w, ops[0], out)
        return ex.issue(w, "lds_q", vregs=(ex.vindex(ops[0])[0],) if rtn else ())
    raise EmuError("unknown LDS instruction: %r" % ins.line)


def _ds_read_tr16(ex, w, ins):
    """ds_read_b64_tr_b16: every lane reads 8 bytes (four 16-bit elements) at its address; within each group of 16 lanes
    the 16 x 4 elements are redistributed so that lane i receives, as element e, element i % 4 of lane 4 * e + i / 4."""
    lanes = mask_to_lanes(w.exec)
    if not lanes.all():
        raise EmuError("transposing LDS read under a partial EXEC is not modelled: %r" % ins.line)
    addrs = ex.vread(w, ins.ops[1], 32).astype(np.int64) + _offset(ins)
    raw, ix = ex.lds_get(w, ins, addrs, 8)
    el = np.ascontiguousarray(raw).view(np.uint16).reshape(64, 4).astype(U32)
    i = np.arange(64)
    grp, li = i // 16 * 16, i % 16
    out = np.zeros((64, 4), dtype=U32)
    for e in range(4):
        out[:, e] = el[grp + 4 * e + li // 4, li % 4]
    d, _ = ex.vindex(ins.ops[0])
    w.v[d] = out[:, 0] | (out[:, 1] << U32(16))
    w.v[d + 1] = out[:, 2] | (out[:, 3] << U32(16))
    ex.issue(w, "lds_q", vregs=(d, d + 1), fetch=ix)


def _global_atomic(ex, w, ins):
    op, ops = ins.op, ins.ops
    name = op[len("global_atomic_"):]
    lanes = mask_to_lanes(w.exec)
    act = np.nonzero(lanes)[0]
    rtn = len(ops) == 4
    if name == "cmpswap":
        rtn = len(ops) == 4
    a_tok, d_tok, b_tok = (ops[1], ops[2], ops[3]) if rtn else (ops[0], ops[1], ops[2])
    addrs = _global_addr(ex, w, ins, a_tok, b_tok)
    di, _ = ex.vindex(d_tok)
    out = np.zeros(64, dtype=U32)
    for lane in act:
        a = addrs[lane:lane + 1]
        old = int(np.ascontiguousarray(ex.mem.load(a, 4, ins.line)).view(U32)[0])
        if name == "cmpswap":
            new = int(w.v[di][lane]) if old == int(w.v[di + 1][lane]) else old
        else:
            new = _atomic_apply(name, old, int(w.v[di][lane]))
        ex.mem.store(a, np.array([new], dtype=U32).view(np.uint8).reshape(1, 4), ins.line)
        out[lane] = old
    if rtn:
        ex.vwrite(w, ops[0], out)
    ex.issue(w, "vm_q", vregs=(ex.vindex(ops[0])[0],) if rtn else ())


def _scratch(ex, w, ins):
    """Private memory: each lane owns `private_segment_fixed_size` bytes; an access beyond them is an error."""
    op, ops = ins.op, ins.ops
    lanes = mask_to_lanes(w.exec)
    act = np.nonzero(lanes)[0]
    size = w.scratch_mem.shape[1]
    load = op.startswith("scratch_load_")
    kind = op[len("scratch_load_"):] if load else op[len("scratch_store_"):]
    v_tok, s_tok = (ops[1], ops[2]) if load else (ops[0], ops[2])
    addr = np.full(64, _offset(ins), dtype=np.int64)
    if v_tok != "off":
        addr = addr + ex.vread(w, v_tok, 32).astype(np.int64)
    if s_tok != "off":
        addr = addr + ex.sread(w, s_tok, 32)
    width = _LOAD_W[kind] if load else _STORE_W[kind]
    if len(act) == 0:
        return
    if (addr[act] < 0).any() or (addr[act] + width > size).any():
        raise EmuError("scratch access outside the %d private bytes: %r" % (size, ins.line))
    ix = addr[act][:, None] + np.arange(width)[None, :]
    if load:
        _land(ex, w, ins, kind, act, w.scratch_mem[act[:, None], ix])
        i, n = ex.vindex(ops[0])
        ex.issue(w, "vm_q", vregs=range(i, i + max(n, (width + 3) // 4)))
    else:
        w.scratch_mem[act[:, None], ix] = _lift(ex, w, kind, act, ops[1])
        ex.issue(w, "vm_q")


# ---------------------------------------------------------------------------------------------------------------
# launch
# ---------------------------------------------------------------------------------------------------------------
def pack_kernarg(prog, values, grid, block, dynamic_lds=0):
    """Kernel-argument segment from the code object's metadata: explicit arguments from `values` (ints, floats or bytes,
    in declaration order), the hidden ones the way the HIP runtime fills them."""
    args = prog.meta[".args"]
    size = prog.meta[".kernarg_segment_size"]
    buf = bytearray(size)
    vi = 0
    for a in args:
        off, sz, kind = a[".offset"], a[".size"], a[".value_kind"]
        if kind in ("global_buffer", "by_value"):
            v = values[vi]
            vi += 1
            if isinstance(v, (bytes, bytearray)):
                if len(v) != sz:
                    raise EmuError("argument %d: %d bytes given, %d expected" % (vi - 1, len(v), sz))
                raw = bytes(v)
            elif isinstance(v, float):
                raw = struct.pack("<f" if sz == 4 else "<d", v)
            else:
                raw = int(v).to_bytes(sz, "little", signed=v < 0)
            buf[off:off + sz] = raw
        elif kind.startswith("hidden_block_count_"):
            buf[off:off + 4] = struct.pack("<I", grid["xyz".index(kind[-1])])
        elif kind.startswith("hidden_group_size_"):
            buf[off:off + 2] = struct.pack("<H", block["xyz".index(kind[-1])])
        elif kind.startswith("hidden_remainder_"):
            buf[off:off + 2] = struct.pack("<H", 0)
        elif kind == "hidden_grid_dims":
            buf[off:off + 2] = struct.pack("<H", 3 if grid[2] > 1 else (2 if grid[1] > 1 else 1))
        elif kind == "hidden_dynamic_lds_size":
            buf[off:off + 4] = struct.pack("<I", dynamic_lds)
        # the remaining hidden arguments (offsets, printf buffer, queue pointers …) stay zero
    if vi != len(values):
        raise EmuError("%d argument values given, the kernel declares %d" % (len(values), vi))
    return bytes(buf)


def launch(prog, mem, values, grid, block, dynamic_lds=0, max_steps=50_000_000, groups=None, trace=None, strict=True):
    """Run the kernel over `grid` workgroups of `block` work-items (3-tuples).  `groups` limits the run to the listed
    workgroup ids (tuples); every memory access of the run is bounds-checked by `mem`."""
    kd = prog.kd
    grid, block = tuple(grid), tuple(block)
    karg = pack_kernarg(prog, values, grid, block, dynamic_lds)
    kaddr = mem.alloc(len(karg) + 64, "kernarg")
    mem.write(kaddr, karg)
    lds_size = int(kd.get("group_segment_fixed_size", 0)) + dynamic_lds
    priv = int(kd.get("private_segment_fixed_size", 0))
    nthreads = block[0] * block[1] * block[2]
    # what the runtime would refuse at launch
    if lds_size > 160 * 1024:
        raise EmuError("%s: %d bytes of LDS requested, a workgroup can have 163840" % (prog.name, lds_size))
    limit = int(prog.meta.get(".max_flat_workgroup_size", 1024))
    if nthreads > limit or nthreads == 0:
        raise EmuError("%s: %d work-items per workgroup, the kernel is built for at most %d" % (prog.name, nthreads, limit))
    if min(grid) < 1 or grid[0] > 0x7FFFFFFF or grid[1] > 65535 or grid[2] > 65535:
        raise EmuError("%s: grid %r is outside what a launch accepts" % (prog.name, grid))
    nwaves = (nthreads + 63) // 64
    tid = np.arange(nwaves * 64)
    tx, ty, tz = tid % block[0], (tid // block[0]) % block[1], tid // (block[0] * block[1])
    packed = (tx | (ty << 10) | (tz << 20)).astype(U32)
    user = int(kd.get("user_sgpr_count", 2))
    if kd.get("user_sgpr_kernarg_preload_length", 0):
        raise EmuError("kernel-argument preloading is not modelled")
    steps = 0
    all_groups = [(x, y, z) for z in range(grid[2]) for y in range(grid[1]) for x in range(grid[0])]
    for g in (groups if groups is not None else all_groups):
        # LDS and registers start out holding NaNs (0x7FC07FC0: a NaN as fp32, as two bf16 and as two fp16; as an
        # address or index it is far outside everything): what a kernel consumes without having written it shows up
        lds = np.tile(np.array([0xC0, 0x7F], dtype=np.uint8), (lds_size + 1) // 2)[:lds_size].copy()
        ex = Exec(mem, lds, prog, strict=strict)
        waves = []
        for wi in range(nwaves):
            w = Wave()
            w.wid = wi
            w.v[:] = U32(POISON)
            w.s[:] = U32(POISON)
            w.s[106:108] = 0
            w.scratch_mem = np.full((64, max(priv, 0)), 0xFF, dtype=np.uint8)     # private memory starts as NaNs too
            # user SGPRs in the ABI's order; only the ones HIP kernels for this target ask for are modelled
            si = 0
            for name, n in (("private_segment_buffer", 4), ("dispatch_ptr", 2), ("queue_ptr", 2),
                            ("kernarg_segment_ptr", 2), ("dispatch_id", 2), ("flat_scratch_init", 2),
                            ("private_segment_size", 1)):
                if kd.get("user_sgpr_" + name, 0):
                    if name == "kernarg_segment_ptr":
                        w.s[si], w.s[si + 1] = kaddr & 0xFFFFFFFF, kaddr >> 32
                    si += n
            if si != user:
                raise EmuError("user SGPR layout: %d counted, descriptor says %d" % (si, user))
            for k, axis in enumerate("xyz"):
                if kd.get("system_sgpr_workgroup_id_" + axis, 1 if axis == "x" else 0):
                    w.s[si] = g[k]
                    si += 1
            w.v[0] = packed[wi * 64:(wi + 1) * 64]
            live = tid[wi * 64:(wi + 1) * 64] < nthreads
            w.exec = lanes_to_mask(live)
            waves.append(w)
        while True:
            progressed = False
            for w in waves:
                while not w.done and not w.at_barrier:
                    if trace is not None:
                        trace(g, w, prog.instrs[w.pc])
                    step(ex, w)
                    steps += 1
                    progressed = True
                    if steps > max_steps:
                        raise EmuError("more than %d instructions: runaway loop?" % max_steps)
            if all(w.done for w in waves):
                break
            if all(w.done or w.at_barrier for w in waves):
                for w in waves:
                    w.at_barrier = False
                ex.barrier_released()
                continue
            if not progressed:
                raise EmuError("workgroup %r makes no progress" % (g,))
    return steps
