"""Runs cases of cases.py on the interpreted device, in a process of its own (no torch, no real HIP runtime in the
global symbol scope), and writes their arrays to an .npz.

    python tests/emu/worker.py --lib flaggems_amd/libfg_mi355.so --asm flaggems_amd/csrc/build --spec cases.json --out out.npz
"""
import argparse
import json
import os
import sys
import tempfile
import time
import traceback

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, HERE)


def _plant(kernel_part, what):
    import gcn_emu as E
    parse = E.parse_program

    def mutated(text, name, exact=False):
        prog = parse(text, name, exact)
        if kernel_part in name:
            n = 0
            for ins in prog.instrs:
                if ins.wait is not None:
                    key = {"vm+1": "vmcnt", "lgkm+1": "lgkmcnt"}.get(what)
                    if key and ins.wait.get(key, 0) > 0:
                        ins.wait[key] += 1
                        n += 1
                elif what == "nobarrier" and ins.op == "s_barrier":
                    ins.op = "s_nop"
                    n += 1
            assert n, "nothing to mutate in %s" % name
        return prog
    E.parse_program = mutated


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--lib", required=True)
    ap.add_argument("--asm", required=True)
    ap.add_argument("--spec", required=True)
    ap.add_argument("--out", required=True)
    ap.add_argument("--shim-dir", default=tempfile.gettempdir())
    ap.add_argument("--num-cu", type=int, default=256, help="compute units the stand-in reports (the host code sizes "
                    "grids, tiles and stream-K partitions from it; the library reads it once per process)")
    ap.add_argument("--no-device-info", action="store_true", help="skip the fg_device_info call a binder makes at start "
                    "(it also looks up the static scratch array): for cases about the library's first call")
    ap.add_argument("--mutate", default="", help="KERNEL_PART:WHAT, a deliberate defect planted in the parsed program of "
                    "every kernel whose name contains KERNEL_PART, to show that the interpreter's checks see it.  WHAT: "
                    "vm+1 / lgkm+1 (every counted wait, i.e. every non-zero count, lets one more operation stay in flight), "
                    "nobarrier (every s_barrier becomes a no-op)")
    a = ap.parse_args()
    assert "torch" not in sys.modules
    import cases
    from device import Device, build_shim
    if a.mutate:
        _plant(*a.mutate.split(":"))
    dev = Device(a.lib, a.asm, build_shim(a.shim_dir))
    dev.shim.shim_set_num_cu(a.num_cu)
    # device set-up the way a binder does it (also primes the static scratch array)
    import ctypes
    if not a.no_device_info:
        ncu, lds, arch = ctypes.c_int(), ctypes.c_int(), ctypes.c_int()
        rc = dev.call("fg_device_info", ctypes.c_int(0), ctypes.byref(ncu), ctypes.byref(lds), ctypes.byref(arch))
        assert rc == 0 and arch.value == 0x950 and ncu.value == a.num_cu, (rc, arch.value, ncu.value, dev.last_error())
    out = {}
    for spec in json.load(open(a.spec)):
        cid = spec["id"]
        rng = np.random.default_rng(spec.get("seed", 0))
        dev.launches.clear()
        t0 = time.time()
        env = spec.get("env") or {}
        try:
            for k, v in env.items():            # the library's FG_* switches, read again for this case
                os.environ[k] = v
            if env:
                dev.lib.fg_reload_options()
            res = getattr(cases, spec["fn"])(dev, rng, **spec["kw"])
            for k, v in res.items():
                out["%s|%s" % (cid, k)] = np.asarray(v)
            if res.get("rc", 0) != 0:
                out["%s|__message" % cid] = np.array(dev.last_error())
        except Exception as exc:
            out["%s|__error" % cid] = np.array("%s\n%s" % (exc, traceback.format_exc()))
        finally:
            for k in env:
                del os.environ[k]
            if env:
                dev.lib.fg_reload_options()
        out["%s|__kernels" % cid] = np.array(json.dumps([[n, list(g), list(b), s, st] for n, g, b, s, st in dev.launches]))
        out["%s|__seconds" % cid] = np.array(time.time() - t0)
        print("%-50s %6.1fs %s" % (cid, time.time() - t0, "ERROR" if ("%s|__error" % cid) in out else ""), flush=True)
    np.savez(a.out, **out)


if __name__ == "__main__":
    main()
