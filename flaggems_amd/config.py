"""Build configuration flags, named as in the reference's src/flag_gems/config.py:5-37.

The reference distinguishes a pure-Python (Triton) path from an optional C extension.  Here the
native library is the only implementation, so `has_c_extension` reports whether it is built and
`use_c_extension` stays False: the Python wrappers call the C ABI themselves rather than routing
through torch.ops.flag_gems, and nothing is patched from C++ at import time.  The torch.ops.flag_gems
namespace itself is defined (custom_ops.py) for callers that use it directly.
"""
import os

from . import _C

has_c_extension = os.path.exists(_C.LIB_PATH)
use_c_extension = False
aten_patch_list = []
