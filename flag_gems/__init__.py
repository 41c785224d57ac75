"""Import-name alias: `import flag_gems` resolves to the MI355X-native package, so code written
against the reference (flag_gems.enable(), flag_gems.ops.mm, flag_gems.testing.assert_close, ...)
runs unchanged."""
import sys

import flaggems_amd as _impl
from flaggems_amd import *  # noqa: F401,F403
from flaggems_amd import (  # noqa: F401
    __version__, all_ops, apply_gems_patches_to_vllm, aten_lib, config, device, enable, fused, logging_utils, modules, ops,
    patches, runtime, testing,
    use_gems, vendor_name,
)

for _name in ("config", "fused", "logging_utils", "modules", "ops", "patches", "runtime", "testing"):
    sys.modules[__name__ + "." + _name] = getattr(_impl, _name)
sys.modules[__name__ + ".runtime.register"] = _impl.runtime.register
for _sub in ("mm", "addmm", "bmm", "softmax", "log_softmax", "rms_norm", "attention"):
    sys.modules[__name__ + ".ops." + _sub] = sys.modules["flaggems_amd.ops." + _sub]
for _sub in ("fused_add_rms_norm", "reshape_and_cache", "reshape_and_cache_flash", "rotary_embedding", "silu_and_mul"):
    sys.modules[__name__ + ".fused." + _sub] = sys.modules["flaggems_amd.fused." + _sub]
for _sub in ("activation", "normalization", "rotary_embedding"):
    sys.modules[__name__ + ".modules." + _sub] = sys.modules["flaggems_amd.modules." + _sub]
for _sub in ("patch_util", "patch_vllm_all"):
    sys.modules[__name__ + ".patches." + _sub] = sys.modules["flaggems_amd.patches." + _sub]
