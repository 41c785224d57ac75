"""GPU parity tests, unchanged, on the interpreter.

The tests listed in tests/emu/interpreted_suite.txt are test functions of the GPU suite (marked `gpu`, written for
cuda:0).  Here they run in child pytest processes with FG_INTERPRETED=1: tests/conftest.py then binds the HIP
stand-in before torch is imported, the `gpu` fixture hands out the CPU device, the operator wrappers and the ATen
overrides of flag_gems.enable() run as they are on CPU tensors, the library's host code runs as built, and every kernel
launch is executed from the compiled assembly by tests/emu/gcn_emu.py with bounds, waits and barriers checked
(see test_interpreted_kernels.py for what the interpreter is and how it is calibrated).  What this adds to the C-ABI
cases there: the Python side of every call (argument preparation, views and strides, workspace handling, the
dispatcher registrations) in front of the same kernels, and the GPU suite's own expectations.

The list holds the cases that finish within a few seconds each on the interpreter (small shapes); it includes GPU cases
that were added while no GPU could be used and have not run on one yet.  Tests that need a real device by
construction (HIP graphs, streams, the custom-op registrations on the CUDA key, assertions on `device.type`) are not on it.
"""
import os
import re
import subprocess
import sys

import pytest

REPO = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
LIST = os.path.join(REPO, "tests", "emu", "interpreted_suite.txt")
LANES = 7


def _node_ids():
    with open(LIST) as f:
        return [line.strip() for line in f if line.strip() and not line.startswith("#")]


@pytest.fixture(scope="module")
def outcome(tmp_path_factory):
    tmp = tmp_path_factory.mktemp("interp_suite")
    ids = _node_ids()
    env = dict(os.environ, FG_INTERPRETED="1", FG_SHIM_DIR=str(tmp))
    env.pop("FG_LIB_PATH", None)
    sys.path.insert(0, os.path.join(REPO, "tests", "emu"))
    try:
        from device import build_shim
    finally:
        sys.path.pop(0)
    build_shim(str(tmp))                                   # once, before the lanes start
    procs = []
    for lane in range(LANES):
        mine = ids[lane::LANES]
        if not mine:
            continue
        log = open(str(tmp / ("lane%d.log" % lane)), "w+")
        procs.append((mine, log, subprocess.Popen(
            [sys.executable, "-m", "pytest", "-q", "-m", "gpu", "-p", "no:cacheprovider", "--timeout", "300", "-rfE"] + mine,
            cwd=REPO, env=env, stdout=log, stderr=subprocess.STDOUT)))
    passed = launches = 0
    problems = []
    for mine, log, p in procs:
        rc = p.wait(timeout=2400)
        log.seek(0)
        text = log.read()
        log.close()
        m = re.search(r"(\d+) passed", text)
        passed += int(m.group(1)) if m else 0
        m = re.search(r"interpreted kernel launches: (\d+)", text)
        launches += int(m.group(1)) if m else 0
        if rc != 0 or not re.search(r"\b%d passed" % len(mine), text):
            problems.append(text[-3000:])
    return {"listed": len(ids), "passed": passed, "launches": launches, "problems": problems}


def test_listed_gpu_tests_pass_on_the_interpreter(outcome):
    assert not outcome["problems"], "\n\n".join(outcome["problems"])
    assert outcome["passed"] == outcome["listed"] and outcome["listed"] >= 100


def test_the_kernels_really_ran(outcome):
    # every listed test launches at least one kernel: nothing was answered by a torch fallback
    assert outcome["launches"] >= outcome["listed"]
