"""Shape of the memory traffic of the row kernels' "requests up front" variants at the benchmark configurations, read
from their device assembly: every load is requested before the first wait, and no kernel argument is fetched late.
A branch around a load, or a value first touched behind a reduction, silently turns one trip to memory per row into
several; the results stay right, so only a look at the generated code shows it.

The variants are switches of flaggems_amd/csrc/variants.h (off in the default build until they have passed the GPU
parity suite), so this test compiles the five sources concerned to device assembly itself, with the switches on.
Skipped when hipcc is not installed."""
import importlib.util
import os
import re
import shutil
import subprocess
from concurrent.futures import ThreadPoolExecutor

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
CSRC = os.path.join(ROOT, "flaggems_amd", "csrc")
_spec = importlib.util.spec_from_file_location("fg_isa_check", os.path.join(CSRC, "isa_check.py"))
isa_check = importlib.util.module_from_spec(_spec)
_spec.loader.exec_module(isa_check)
_spec = importlib.util.spec_from_file_location("fg_build", os.path.join(CSRC, "build.py"))
fg_build = importlib.util.module_from_spec(_spec)
_spec.loader.exec_module(fg_build)

VARIANTS = {"ROWS_UPFRONT": 1, "SHORT_UPFRONT": 1, "SCATTER_EARLY": 1, "ROPE_ARGS": 1, "RMS_BWD_ZERO_PACK": 1,
            "RMS_TWO_ROWS": 1, "SKINNY_ASM_A": 1}
SOURCES = ["norm", "softmax", "backward", "rope", "kvcache", "gemm_skinny"]


@pytest.fixture(scope="module")
def variant_asm(tmp_path_factory):
    """{source: device assembly text} of the five sources built with the variants on."""
    if not os.path.exists(fg_build.HIPCC):
        pytest.skip("no hipcc at %s" % fg_build.HIPCC)
    out = tmp_path_factory.mktemp("variant_asm")
    defines = fg_build.variant_defines(VARIANTS)

    def one(src):
        dst = os.path.join(str(out), src + ".s")
        cmd = [fg_build.HIPCC] + fg_build.FLAGS + defines + ["-x", "hip", "--cuda-device-only", "-S",
                                                            os.path.join(CSRC, src + ".hip"), "-o", dst]
        p = subprocess.run(cmd, capture_output=True, text=True)
        assert p.returncode == 0, p.stderr[-2000:]
        with open(dst) as f:
            return src, f.read()

    with ThreadPoolExecutor(max_workers=len(SOURCES)) as ex:
        texts = dict(ex.map(one, SOURCES))
    shutil.rmtree(str(out), ignore_errors=True)
    for src, text in texts.items():
        hits = isa_check.scan(text) + isa_check.scan_packed_f32(text) + isa_check.scan_vmem_loads(text) + [
            (k, 0, first, "%d scratch accesses inside a loop" % n)
            for k, n, first in isa_check.scan_scratch_in_loops(text, allowed={})]
        assert not hits, (src, hits[:3])
    return texts


# (source, kernel instantiation, what it serves)
CASES = [
    ("softmax", "softmax_rows_kernelIDF16bDF16bLi8ELi2ELi128ELb0", "softmax [131072, 2048] bf16"),
    ("softmax", "softmax_rows_kernelIDF16bDF16bLi8ELi8ELi1024ELb0", "softmax, eight packs a thread"),
    ("norm", "rms_rows_kernelIDF16bLi8ELi1ELi512ELb1", "fused_add_rms_norm [4096, 4096] bf16"),
    ("norm", "rms_rows_kernelIfLi4ELi2ELi512ELb1", "fused_add_rms_norm [4096, 4096] fp32"),
    ("norm", "rms_rows_kernelIDF16bLi8ELi1ELi512ELb0", "rms_norm [16384, 4096] bf16"),
    ("norm", "rms_rows2_kernelIDF16bLi8ELi512ELb1", "fused_add_rms_norm [4096, 4096] bf16, two rows per workgroup"),
    ("norm", "rms_rows2_kernelIfLi4ELi1024ELb1", "fused_add_rms_norm [4096, 4096] fp32, two rows per workgroup"),
    ("backward", "bwd_rows_kernelIDF16bDF16bLi8ELi1ELi256ELi0", "softmax backward [131072, 2048] bf16"),
    ("backward", "bwd_rows_kernelIDF16bDF16bLi8ELi4ELi1024ELi0", "softmax backward, four packs a thread"),
    ("backward", "bwd_rows_kernelIDF16bDF16bLi8ELi2ELi1024ELi1", "log_softmax backward, two packs a thread"),
    ("softmax", "softmax_short_kernelIDF16bDF16bLb0ELi16", "softmax, a wave per row of up to 1024 elements"),
    ("backward", "bwd_short_kernelIDF16bDF16bLi0ELi8", "softmax backward, a wave per row of up to 512 elements"),
    ("norm", "rms_short_kernelIDF16bLb0ELi8", "rms_norm, a wave per unaligned row of up to 512 elements"),
]


def _trace(asm, source, kernel):
    lines = isa_check.memory_trace(asm[source], kernel)
    assert len(lines) == 1, (kernel, len(lines))
    return lines[0].split("\n")[1].strip().replace(".", "")


@pytest.mark.parametrize("source,kernel,what", CASES)
def test_every_request_goes_out_before_the_first_wait(variant_asm, source, kernel, what):
    trace = _trace(variant_asm, source, kernel)
    assert "k" not in trace, "%s: a kernel argument is fetched late: %s" % (what, trace)
    head = re.match(r"^[L|]+", trace).group(0)
    assert "L" not in trace[len(head):], "%s: a load is issued behind a wait: %s" % (what, trace)
    assert trace.count("L") >= 1 and trace.rstrip("|").endswith("S"), trace


def test_skinny_gemm_with_asm_loads_never_drains_the_ring(variant_asm):
    """FG_V_SKINNY_ASM_A: the main loop of the K-contiguous skinny GEMM for more than eight rows holds counted waits
    only (the build of the default code waits for everything in flight once per trip), and the VM-counter scan, which
    the fixture has already run over the whole file, finds every register valid where it is used."""
    text = variant_asm["gemm_skinny"]
    for dtype in ("DF16b", "DF16_"):
        km = [k for k in isa_check._KERNEL.finditer(text) if "gemm_skinny_kc_kernelI%sLi16ELi8ELb1ELi1E" % dtype in k.group(1)]
        assert len(km) == 1
        blocks = isa_check._blocks(km[0].group(2))
        loop = isa_check._blocks_in_loops(isa_check._successors(blocks))
        main = max(loop, key=lambda b: sum(1 for op, _, _ in blocks[b][1] if op.startswith("v_mfma")))
        waits = [isa_check._vm_wait_count(ops) for op, ops, _ in blocks[main][1] if op == "s_waitcnt"]
        waits = [w for w in waits if w is not None]
        assert waits == [28] * 8, waits   # eight steps a trip, each leaving the 7 x 4 younger operations in flight
    assert isa_check.scan_lds_reads(text) == []


def test_the_trace_reads_a_known_kernel():
    text = ("k0:   ; @k0\n\ts_load_dwordx2 s[0:1], s[4:5], 0x0\n\tglobal_load_dwordx4 v[0:3], v8, s[0:1]\n"
            "\ts_waitcnt vmcnt(0)\n\ts_cbranch_scc1 .LBB0_1\n.LBB0_1:\n\tglobal_load_dwordx4 v[4:7], v8, s[0:1]\n"
            "\ts_barrier\n\ts_waitcnt vmcnt(0) lgkmcnt(0)\n\tglobal_store_dwordx4 v8, v[0:3], s[2:3]\n\ts_endpgm\n.Lfunc_end0:\n")
    assert isa_check.memory_trace(text, "k0") == ["k0\n    L(0).L|(0)S"]


def _groups(trace):
    """Runs of loads between waits: 'LL(1)(0)LLL(0)S' -> [2, 3]."""
    return [len(g) for g in re.findall(r"L+", trace)]


def test_rope_reads_position_then_everything_else_in_one_batch(variant_asm):
    trace = _trace(variant_asm, "rope", "rope_kernelIDF16bDF16bLi8ELb0")
    first = trace.index("L")
    assert "k" not in trace[first:], trace            # every argument is fetched before the first load
    groups = _groups(trace)
    # the position (one load in each arm of the int64 / int32 branch), then cos, sin and the two halves of the row
    assert groups[-1] == 4 and sum(groups[:-1]) == 2, trace


def test_cache_scatter_requests_the_row_with_the_slot(variant_asm):
    trace = _trace(variant_asm, "kvcache", "cache_scatter_kernelIDv4_jl")
    assert "k" not in trace[trace.index("L"):], trace
    assert _groups(trace)[0] == 5, trace              # four pieces of the row and the slot, one wait for all
