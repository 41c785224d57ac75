"""MI355X-native drop-in for the LLM-inference operator path of FlagGems.

Same public surface as the reference package for that path (src/flag_gems/__init__.py:1-377):
enable() / use_gems() / all_ops(), `device`, `vendor_name`, `testing`, `runtime`, `config`, the
operator functions at top level and under `ops` / `fused`.  Every operator is a hand-written
gfx950 kernel behind the C ABI of libfg_mi355.so; operators outside this path stay on PyTorch's
own ATen kernels.
"""
import logging

import torch

from . import config  # noqa: F401
from . import custom_ops  # noqa: F401  (defines torch.ops.flag_gems.*)
from . import runtime  # noqa: F401
from . import testing  # noqa: F401
from . import fused, ops  # noqa: F401
from . import modules  # noqa: F401
from . import patches  # noqa: F401
from .fused import *  # noqa: F401,F403
from .logging_utils import setup_flaggems_logging
from .ops import *  # noqa: F401,F403
from .patches import apply_gems_patches_to_vllm  # noqa: F401
from .runtime.register import Register

__version__ = "3.0"
device = runtime.device.name
vendor_name = runtime.device.vendor_name
aten_lib = torch.library.Library("aten", "IMPL")
registrar = Register
current_work_registrar = None


def _aten_table():
    """(aten overload, python kernel) rows of the reference's table that lie on this path
    (src/flag_gems/__init__.py:38-42,55-56,89,213-214,275)."""
    return (
        ("_flash_attention_forward", flash_attention_forward),  # noqa: F405
        ("_log_softmax", log_softmax),  # noqa: F405
        ("_log_softmax_backward_data", log_softmax_backward),  # noqa: F405
        ("_softmax", softmax),  # noqa: F405
        ("_softmax_backward_data", softmax_backward),  # noqa: F405
        ("addmm", addmm),  # noqa: F405
        ("addmm.out", addmm_out),  # noqa: F405
        ("bmm", bmm),  # noqa: F405
        ("mm", mm),  # noqa: F405
        ("mm.out", mm_out),  # noqa: F405
        ("rms_norm", rms_norm),  # noqa: F405
    )


def enable(lib=aten_lib, unused=None, registrar=registrar, record=False, once=False, path=None):
    """Override the ATen operators of this path on the CUDA (= ROCm) dispatch key.

    `unused` lists python function names to leave on ATen (e.g. ["mm"]); `record` logs every
    operator call to `path` (default ~/.flaggems/oplist.log), `once` de-duplicates by call site.
    """
    global current_work_registrar
    current_work_registrar = registrar(
        _aten_table(),
        user_unused_ops_list=list(set(unused or [])),
        cpp_patched_ops_list=list(set(config.aten_patch_list)),
        lib=lib,
    )
    setup_flaggems_logging(path=path, record=record, once=once)


class use_gems:
    """Context manager: overrides are active inside the block and removed on exit."""

    def __init__(self, unused=None, record=False, once=False, path=None):
        self.lib = torch.library.Library("aten", "IMPL")
        self.unused = [] if unused is None else unused
        self.registrar = Register
        self.record = record
        self.once = once
        self.path = path

    def __enter__(self):
        enable(lib=self.lib, unused=self.unused, registrar=self.registrar, record=self.record,
               once=self.once, path=self.path)

    def __exit__(self, exc_type, exc_val, exc_tb):
        global current_work_registrar
        self.lib._destroy()
        del self.lib
        del self.unused
        del self.registrar
        current_work_registrar = None
        if self.record:
            for handler in logging.root.handlers[:]:
                logging.root.removeHandler(handler)
            logging.basicConfig(level=logging.INFO)


def all_ops():
    return current_work_registrar.get_all_ops()


__all__ = ["enable", "use_gems", "all_ops", "apply_gems_patches_to_vllm"] + list(ops.__all__) + list(fused.__all__)
