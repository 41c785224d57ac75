"""The slice of the reference's runtime package that callers of the hot path touch
(src/flag_gems/runtime/__init__.py:6-42, backend/device.py:28-59, backend/_amd/__init__.py:3-7).

There is one backend: PyTorch-ROCm on MI355X.  It shows up in torch as device type "cuda" with
dispatch key "CUDA", exactly what the reference reports for vendor "amd".  No vendor probing, no
argv parsing, no tuning tables.
"""
import torch


class _Device:
    name = "cuda"
    vendor_name = "amd"
    dispatch_key = "CUDA"
    support_fp64 = True
    support_bf16 = True
    support_int64 = True

    @property
    def device_count(self):
        return torch.cuda.device_count()


device = _Device()
torch_device_fn = torch.cuda
# Python function names the AMD backend of the reference leaves to ATen
# (src/flag_gems/runtime/backend/_amd/__init__.py:7); none of them is on this path.
vendor_unused_ops = ("cumsum", "cos", "add")


def get_device_unused_op():
    return list(vendor_unused_ops)


from .register import Register  # noqa: E402,F401
