"""libfg_mi355.so on a machine without a GPU: the library's host code runs as built, against a stand-in for the HIP
runtime (hip_shim.cpp), and every kernel launch it makes is executed from the kernel's compiled assembly by the
interpreter (gcn_emu.py) on numpy buffers.  Test infrastructure: nothing outside tests/ may import this.

Use from a process that has not loaded the real HIP runtime into the global symbol scope (importing torch does):
the stand-in must be the first definition of hipLaunchKernel & co. the dynamic linker finds when it binds the library.
"""
import ctypes
import glob
import os
import re
import subprocess
import sys

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
REPO = os.path.dirname(os.path.dirname(HERE))
sys.path.insert(0, HERE)
import gcn_emu as E  # noqa: E402

F16, BF16, F32 = 0, 1, 2


def build_shim(out_dir):
    out = os.path.join(out_dir, "libhipshim.so")
    src = os.path.join(HERE, "hip_shim.cpp")
    if not os.path.exists(out) or os.path.getmtime(out) < os.path.getmtime(src):
        subprocess.run(["g++", "-O1", "-w", "-shared", "-fPIC", "-D__HIP_PLATFORM_AMD__", "-I/opt/rocm/include", src,
                        "-o", out], check=True)
    return out


_LAUNCH_CB = ctypes.CFUNCTYPE(ctypes.c_int, ctypes.c_char_p, ctypes.POINTER(ctypes.c_uint), ctypes.POINTER(ctypes.c_uint),
                              ctypes.POINTER(ctypes.c_void_p), ctypes.c_size_t, ctypes.c_void_p)
_SYMBOL_CB = ctypes.CFUNCTYPE(ctypes.c_void_p, ctypes.c_char_p, ctypes.c_size_t)


class Device:
    """One interpreted GPU.  lib_path / asm_dir name a build of the library and the assembly saved beside its objects."""

    def __init__(self, lib_path, asm_dir, shim_path):
        self.mem = E.Memory()
        self.asm_dir = asm_dir
        self.index = {}       # mangled kernel name -> assembly file
        for f in glob.glob(os.path.join(asm_dir, "*-hip-amdgcn-amd-amdhsa-gfx950.s")):
            with open(f) as fh:
                for name in re.findall(r"^\s*\.amdhsa_kernel (\S+)$", fh.read(), re.M):
                    self.index[name] = f
        self.texts, self.programs = {}, {}
        self.launches = []    # (kernel name, grid, block, dynamic LDS, instructions executed)
        self.error = None
        self.group_filter = None    # callable(name, grid) -> list of workgroup ids to run, or None for all
        self.shim = ctypes.CDLL(shim_path, mode=ctypes.RTLD_GLOBAL)
        self._cb = (_LAUNCH_CB(self._on_launch), _SYMBOL_CB(self._on_symbol))
        self.shim.shim_set_callbacks(self._cb[0], self._cb[1])
        self.lib = ctypes.CDLL(lib_path)
        self.lib.fg_last_error.restype = ctypes.c_char_p
        if self.shim.shim_num_functions() == 0:
            raise RuntimeError("the library registered no kernels with the stand-in: the real HIP runtime was bound")

    # ---- memory ------------------------------------------------------------------------------------------------
    def upload(self, array, name="buf"):
        array = np.ascontiguousarray(array)
        return self.mem.alloc(array.nbytes, name, data=array.view(np.uint8))

    def alloc(self, nbytes, name="buf", fill=0):
        p = self.mem.alloc(nbytes, name)
        if fill:
            self.mem.view(p)[:] = fill
        return p

    def download(self, ptr, dtype, shape):
        return self.mem.view(ptr)[:int(np.prod(shape)) * np.dtype(dtype).itemsize].view(dtype).reshape(shape).copy()

    # ---- callbacks ---------------------------------------------------------------------------------------------
    def program(self, name):
        if name not in self.programs:
            f = self.index.get(name)
            if f is None:
                raise E.EmuError("kernel %s is in no assembly file of %s" % (name, self.asm_dir))
            if f not in self.texts:
                with open(f) as fh:
                    self.texts[f] = fh.read()
            self.programs[name] = E.parse_program(self.texts[f], name, exact=True)
        return self.programs[name]

    def _on_launch(self, name, grid, block, args, shmem, stream):
        try:
            name = name.decode()
            prog = self.program(name)
            values = []
            k = 0
            for a in prog.meta[".args"]:
                if a[".value_kind"] in ("global_buffer", "by_value"):
                    values.append(ctypes.string_at(args[k], a[".size"]))
                    k += 1
            g, b = (grid[0], grid[1], grid[2]), (block[0], block[1], block[2])
            groups = self.group_filter(name, g) if self.group_filter else None
            steps = E.launch(prog, self.mem, values, g, b, dynamic_lds=int(shmem), groups=groups)
            self.launches.append((name, g, b, int(shmem), steps))
            return 0
        except Exception as exc:  # the callback must not raise through the C frames
            import traceback
            self.error = "%s\n%s" % (exc, traceback.format_exc())
            return 1

    def _on_symbol(self, name, nbytes):
        return self.mem.alloc(nbytes, "symbol " + name.decode())

    # ---- calls -------------------------------------------------------------------------------------------------
    def call(self, fn, *args):
        """Call an entry point; raises with the interpreter's message if a launch failed inside it."""
        self.error = None
        rc = getattr(self.lib, fn)(*args)
        if self.error:
            raise E.EmuError("%s: %s" % (fn, self.error))
        return rc

    def last_error(self):
        return (self.lib.fg_last_error() or b"").decode()
