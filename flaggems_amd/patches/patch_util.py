"""Two ways to swap an implementation in: a class attribute, or a kernel of one of vLLM's torch
libraries (reference: src/flag_gems/patches/patch_util.py:1-32)."""
import torch

_LIB_NAMES = ("_C", "_moe_C", "_vllm_fa3_C")
_libs = {}


def patch_module_method(cls, method_name, new_method, verbose=True):
    """Replace cls.method_name; returns what was there so a caller can put it back."""
    old_method = getattr(cls, method_name, None)
    setattr(cls, method_name, new_method)
    if verbose:
        print(f"Patched {cls.__name__}.{method_name} with FLAGGEMS {new_method.__name__}")
    return old_method


def patch_vllm_lib(lib_name, fn_name, fn, key, verbose=True):
    """Register fn as the `key` kernel of torch.ops.<lib_name>.<fn_name>.  The IMPL handle of a library
    is created on first use and kept for the life of the process (dropping it would undo the patch)."""
    if lib_name not in _LIB_NAMES:
        raise ValueError(f"Library {lib_name} is not recognized.")
    if lib_name not in _libs:
        _libs[lib_name] = torch.library.Library(lib_name, "IMPL")
    _libs[lib_name].impl(fn_name, fn, key)
    if verbose:
        print(f"Patched torch.ops.{lib_name}.{fn_name} with FLAGGEMS {fn.__name__}")
