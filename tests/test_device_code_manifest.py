"""The default build's device code is the code that last passed the GPU parity suite.

tests/golden/device_code_manifest.txt holds, per kernel, a digest of the instruction stream of the build whose library
passed all of `pytest tests -m gpu` on an MI355X (tests/golden/make_device_manifest.py).  The library's build keeps the
device assembly of every HIP source (flaggems_amd/csrc/build/*.s); this test digests it the same way and compares.
Kernel variants that have not been through the suite live behind the switches of flaggems_amd/csrc/variants.h, all off by
default, so with a clean tree every kernel matches; a mismatch means a source change altered a tested kernel's
instructions and the GPU suite has to pass again before the manifest may follow.
Skipped when the build's assembly is not there (the tests may run against a prebuilt library)."""
import importlib.util
import os

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
BUILD = os.path.join(ROOT, "flaggems_amd", "csrc", "build")
MANIFEST = os.path.join(ROOT, "tests", "golden", "device_code_manifest.txt")

_spec = importlib.util.spec_from_file_location("fg_make_manifest", os.path.join(ROOT, "tests", "golden", "make_device_manifest.py"))
make_manifest = importlib.util.module_from_spec(_spec)
_spec.loader.exec_module(make_manifest)

# Kernels of the manifest's build that the sources no longer instantiate, with the reason.
NO_LONGER_BUILT = {
    # the 256x256 tile on the element-by-element stager: no launch path selected it, and it spilled 1174 registers
    ("gemm", "_ZN3fgk14gemm_dp_kernelIDF16_Li256ELi256ELi2ELi2EEEvNS_8GemmArgsE"),
    ("gemm", "_ZN3fgk14gemm_dp_kernelIDF16bLi256ELi256ELi2ELi2EEEvNS_8GemmArgsE"),
}


def _manifest():
    out = {}
    with open(MANIFEST) as f:
        for line in f:
            source, kernel, sha, n = line.split()
            out[(source, kernel)] = (sha, int(n))
    return out


def _built():
    if not os.path.isdir(BUILD) or not any(f.endswith(".s") for f in os.listdir(BUILD)):
        pytest.skip("no device assembly under %s (run flaggems_amd/csrc/build.py)" % BUILD)
    return make_manifest.digests_of_dir(BUILD)


def test_every_built_kernel_is_the_tested_kernel():
    want, got = _manifest(), _built()
    changed = sorted(k for k in got if k in want and got[k][0] != want[k][0])
    new = sorted(k for k in got if k not in want)
    assert not changed, "%d kernels differ from the code the GPU suite passed on, e.g. %s (%d -> %d lines)" % (
        len(changed), changed[0], want[changed[0]][1], got[changed[0]][1])
    assert not new, "%d kernels are not in the manifest (never run on a GPU), e.g. %s" % (len(new), new[0])


def test_no_tested_kernel_went_missing():
    want, got = _manifest(), _built()
    sources = {s for s, _ in got}
    missing = sorted(k for k in want if k not in got and k[0] in sources and k not in NO_LONGER_BUILT)
    assert not missing, "%d kernels of the manifest are no longer built, e.g. %s" % (len(missing), missing[0])
    assert sources >= {s for s, _ in want}, "sources without assembly: %s" % sorted({s for s, _ in want} - sources)


def test_digest_ignores_block_label_numbers_and_comments_only():
    isa = make_manifest.load_isa_check()
    a = "k0:\n\ts_mov_b32 s0, 1 ; note\n.LBB3_1:\n\ts_cbranch_scc1 .LBB3_1\n\ts_endpgm\n.Lfunc_end0:\n"
    b = "k0:\n\ts_mov_b32 s0, 1\n.LBB7_1:\n\ts_cbranch_scc1 .LBB7_1 ; other\n\ts_endpgm\n.Lfunc_end9:\n"
    c = "k0:\n\ts_mov_b32 s1, 1\n.LBB3_1:\n\ts_cbranch_scc1 .LBB3_1\n\ts_endpgm\n.Lfunc_end0:\n"
    assert isa.kernel_digests(a) == isa.kernel_digests(b)
    assert isa.kernel_digests(a) != isa.kernel_digests(c)
    assert isa.kernel_digests(a)["k0"][1] == 4
