"""Writes tests/golden/device_code_manifest.txt: one line per device kernel of the library, `source kernel sha1 lines`,
the digest of the kernel's instruction stream (flaggems_amd/csrc/isa_check.py::kernel_digests).

The manifest records the device code that last passed the whole GPU parity suite.  tests/test_device_code_manifest.py
compares the default build against it, so a change to a source file that alters the instructions of a tested kernel
shows up on the CPU, before any GPU run.  Regenerate it only from a build whose library has just passed
`pytest tests -m gpu` on an MI355X:

    python flaggems_amd/csrc/build.py --force && python tests/golden/make_device_manifest.py

An assembly directory other than the build's own can be named as the first argument (files <source>.s or
<source>-hip-amdgcn-amd-amdhsa-gfx950.s)."""
import importlib.util
import os
import sys

ROOT = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
OUT = os.path.join(ROOT, "tests", "golden", "device_code_manifest.txt")
SUFFIX = "-hip-amdgcn-amd-amdhsa-gfx950.s"


def load_isa_check():
    spec = importlib.util.spec_from_file_location("fg_isa_check", os.path.join(ROOT, "flaggems_amd", "csrc", "isa_check.py"))
    mod = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(mod)
    return mod


def digests_of_dir(path):
    """{(source, kernel): (sha1, lines)} over every assembly file in `path`."""
    isa = load_isa_check()
    out = {}
    for f in sorted(os.listdir(path)):
        if not f.endswith(".s"):
            continue
        source = f[:-len(SUFFIX)] if f.endswith(SUFFIX) else f[:-2]
        with open(os.path.join(path, f)) as fh:
            for kernel, (sha, n) in isa.kernel_digests(fh.read()).items():
                out[(source, kernel)] = (sha, n)
    return out


def main():
    path = sys.argv[1] if len(sys.argv) > 1 else os.path.join(ROOT, "flaggems_amd", "csrc", "build")
    d = digests_of_dir(path)
    with open(OUT, "w") as f:
        for (source, kernel), (sha, n) in sorted(d.items()):
            f.write("%s %s %s %d\n" % (source, kernel, sha, n))
    print("%d kernels -> %s" % (len(d), OUT))


if __name__ == "__main__":
    main()
