"""Build libfg_mi355.so (gfx950 only) with hipcc: one object per source, compiled in parallel.

Usage: python flaggems_amd/csrc/build.py [--force] [--jobs N] [--variant NAME=VALUE ... --tag TAG]
The library lands next to the package (flaggems_amd/libfg_mi355.so) so it travels with the tree.

--variant sets switches of csrc/variants.h (kernel variants that have not passed the parity suite on a GPU; every
switch defaults to the tested code), e.g. `--variant ROWS_UPFRONT=1 --variant DMA_COPY_RUNS=3 --tag cand`.  A variant
build needs a --tag: it lands in flaggems_amd/libfg_mi355.TAG.so with its objects in csrc/build_TAG, beside the default
library, and is loaded by setting FG_LIB_PATH to it (flaggems_amd/_C.py).
"""
import argparse
import os
import re
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor

HERE = os.path.dirname(os.path.abspath(__file__))
if HERE not in sys.path:
    sys.path.insert(0, HERE)
PKG = os.path.dirname(HERE)
OUT = os.path.join(PKG, "libfg_mi355.so")
OBJ_DIR = os.path.join(HERE, "build")

SOURCES = [
    "abi.cpp",
    "norm.hip",
    "softmax.hip",
    "backward.hip",
    "transpose.hip",
    "rope.hip",
    "kvcache.hip",
    "silu_mul.hip",
    "gemm.hip",
    "gemm_skinny.hip",
    "gemm_streamk.hip",
    "gemm_dma.hip",
    "attn_varlen.hip",
    "probe.hip",
]

# The device assembly of every HIP source is kept (-save-temps) and scanned by isa_check.py: wait states the compiler
# cannot keep around instructions issued from inline asm (gemm_dma.hip, attn_varlen.hip), and no packed fp32 arithmetic
# anywhere.
ASM_CHECKED = {s for s in SOURCES if s.endswith(".hip")}

HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
FLAGS = [
    "--offload-arch=gfx950",
    "-O3",
    "-std=c++17",
    "-fPIC",
    "-Wall",
    "-Wno-unused-function",
    # packed-fp32 arithmetic is switched off for every device function of this library
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
]


def _newer(src_paths, target):
    if not os.path.exists(target):
        return True
    t = os.path.getmtime(target)
    return any(os.path.getmtime(p) > t for p in src_paths)


_DIAG = re.compile(r"^\S+:\d+:\d+: (warning|error|note): ")
# expected diagnostics: the host pass does not know the device feature switch; the asm copies set M0 themselves and
# say so in their clobber lists, which the compiler remarks on for every instantiation
_EXPECTED = ("packed-fp32-ops", "inline asm clobber list contains reserved registers: m0",
             "Reserved registers on the clobber list may not be preserved")


def _quiet(text):
    """The compiler's output without the expected diagnostics (each with its include trail, source excerpt and caret
    lines)."""
    out, trail, skipping = [], [], False
    for line in text.splitlines():
        if line.startswith("In file included"):
            trail.append(line)
            continue
        if _DIAG.match(line):
            skipping = any(e in line for e in _EXPECTED)
            if not skipping:
                out.extend(trail)
            trail = []
        if not skipping and "warnings generated" not in line and not any(e in line for e in _EXPECTED):
            out.append(line)
    return "\n".join(out)


def _compile(src, force, obj_dir=OBJ_DIR, defines=()):
    path = os.path.join(HERE, src)
    obj = os.path.join(obj_dir, src + ".o")
    headers = [os.path.join(HERE, f) for f in os.listdir(HERE) if f.endswith(".h")]
    headers.append(os.path.join(os.path.dirname(PKG), "include", "fg_mi355.h"))
    if not force and not _newer([path] + headers, obj):
        return obj, ""
    lang = ["-x", "hip"] if src.endswith(".hip") else []
    keep = ["-save-temps=obj"] if src in ASM_CHECKED else []
    cmd = [HIPCC] + FLAGS + list(defines) + keep + lang + ["-c", path, "-o", obj]
    p = subprocess.run(cmd, capture_output=True, text=True)
    log = _quiet(p.stdout + p.stderr)
    if p.returncode != 0:
        raise RuntimeError("hipcc failed for %s:\n%s" % (src, log))
    if keep:
        _check_wait_states(src, obj, obj_dir)
    return obj, log


def _check_wait_states(src, obj, obj_dir=OBJ_DIR):
    """Scan the device assembly the object was assembled from; drop the other intermediate files."""
    import isa_check

    stem = os.path.join(obj_dir, os.path.splitext(src)[0])
    asm = stem + "-hip-amdgcn-amd-amdhsa-gfx950.s"
    if not os.path.exists(asm):
        os.remove(obj)
        raise RuntimeError("no device assembly for %s at %s: the wait-state check cannot run" % (src, asm))
    hits = isa_check.check_file(asm)
    for f in os.listdir(obj_dir):
        full = os.path.join(obj_dir, f)
        if full != asm and full != obj and (f.startswith(os.path.basename(stem) + "-") or f.startswith(src + "-")):
            os.remove(full)
    if hits:
        os.remove(obj)  # a later build without --force must not link it
        lines = ["  %s: %s  <- %s" % (k[:70], line, why) for k, _, line, why in hits[:10]]
        raise RuntimeError("%s: the device assembly fails %d check(s) of isa_check.py:\n%s" % (src, len(hits), "\n".join(lines)))


# The value at which each switch of variants.h is on trial (its default is the GPU-tested code).  A library built with
# all of them ("cand") is what the interpreted tests run beside the default one.
TRIAL = {"ROWS_UPFRONT": 1, "SHORT_UPFRONT": 1, "SCATTER_EARLY": 1, "ROPE_ARGS": 1, "ATTN_Q_UNCOND": 1, "DECODE_Q_EARLY": 1,
         "RMS_BWD_ZERO_PACK": 1, "ADDMM_BCAST_BRANCH": 1, "DMA_SCALAR_BASES": 1, "DMA_COPY_RUNS": 3, "ATTN_ROWSUM_MFMA": 1,
         "RMS_TWO_ROWS": 1, "SKINNY_ASM_A": 1, "SILU_GRAD_KERNEL": 1}


def variant_defines(variants):
    """{"ROWS_UPFRONT": 1} -> ["-DFG_V_ROWS_UPFRONT=1"]; the names are checked against csrc/variants.h."""
    known = set(re.findall(r"^#define FG_V_(\w+) ", open(os.path.join(HERE, "variants.h")).read(), re.M))
    out = []
    for name, value in sorted((variants or {}).items()):
        if name not in known:
            raise ValueError("unknown variant %r (variants.h has %s)" % (name, ", ".join(sorted(known))))
        out.append("-DFG_V_%s=%d" % (name, int(value)))
    return out


def build(force=False, jobs=None, verbose=True, variants=None, tag=None):
    defines = variant_defines(variants)
    if defines and not tag:
        raise ValueError("a variant build needs a tag: the default library is always the tested code")
    obj_dir, out = OBJ_DIR, OUT
    if tag:
        if not re.fullmatch(r"[A-Za-z0-9_]+", tag):
            raise ValueError("bad tag %r" % tag)
        obj_dir = OBJ_DIR + "_" + tag
        out = os.path.join(PKG, "libfg_mi355.%s.so" % tag)
        stamp = os.path.join(obj_dir, "defines.txt")
        if os.path.exists(stamp) and open(stamp).read() != " ".join(defines):
            force = True  # the objects there were built with other switches
    os.makedirs(obj_dir, exist_ok=True)
    if tag:
        with open(os.path.join(obj_dir, "defines.txt"), "w") as f:
            f.write(" ".join(defines))
    srcs = [s for s in SOURCES if os.path.exists(os.path.join(HERE, s))]
    jobs = jobs or min(8, len(srcs))
    with ThreadPoolExecutor(max_workers=jobs) as ex:
        results = list(ex.map(lambda s: _compile(s, force, obj_dir, defines), srcs))
    objs = [o for o, _ in results]
    for _, log in results:
        if log.strip() and verbose:
            print(log, file=sys.stderr)
    if force or _newer(objs, out):
        cmd = [HIPCC, "--offload-arch=gfx950", "-shared", "-fPIC", "-o", out] + objs
        p = subprocess.run(cmd, capture_output=True, text=True)
        if p.returncode != 0:
            raise RuntimeError("link failed:\n" + p.stdout + p.stderr)
    return out


if __name__ == "__main__":
    ap = argparse.ArgumentParser()
    ap.add_argument("--force", action="store_true")
    ap.add_argument("--jobs", type=int, default=None)
    ap.add_argument("--variant", action="append", default=[], metavar="NAME=VALUE")
    ap.add_argument("--tag", default=None)
    a = ap.parse_args()
    print(build(force=a.force, jobs=a.jobs, variants=dict(v.split("=", 1) for v in a.variant), tag=a.tag))
