"""RMSNorm module with the optional fused residual add of serving stacks
(reference: src/flag_gems/modules/normalization.py:33-121)."""
import logging
import numbers

import torch
import torch.nn as nn

from ..fused import fused_add_rms_norm
from ..ops import rms_norm

logger = logging.getLogger("flag_gems.modules.normalization")

__all__ = ["gems_rms_forward", "GemsRMSNorm"]


def gems_rms_forward(x, residual, weight, eps):
    """Without a residual: the normalised tensor.  With one: (x, residual) after residual += x and
    x = rmsnorm(residual) * weight, both updated in place."""
    if residual is None:
        logger.debug("GEMS CUSTOM RMS_NORM")
        return rms_norm(x, list(weight.size()), weight, eps)
    logger.debug("GEMS CUSTOM FUSED_ADD_RMS_NORM")
    return fused_add_rms_norm(x, residual, list(weight.size()), weight, eps)


class GemsRMSNorm(nn.Module):
    """Interface of torch.nn.RMSNorm (normalized_shape, eps, elementwise_affine, device, dtype) plus the
    `residual` argument of forward.  Derived from nn.Module directly so that it also works where
    torch.nn.RMSNorm does not exist yet."""

    __constants__ = ["normalized_shape", "eps", "elementwise_affine"]

    def __init__(self, normalized_shape, eps=1e-6, elementwise_affine=True, device=None, dtype=None):
        super().__init__()
        if isinstance(normalized_shape, numbers.Integral):
            normalized_shape = (normalized_shape,)
        self.normalized_shape = tuple(normalized_shape)
        self.eps = eps
        self.elementwise_affine = elementwise_affine
        if elementwise_affine:
            self.weight = nn.Parameter(torch.empty(self.normalized_shape, device=device, dtype=dtype))
        else:
            self.register_parameter("weight", None)
        self.reset_parameters()

    def reset_parameters(self):
        if self.elementwise_affine:
            nn.init.ones_(self.weight)

    def forward(self, x, residual=None):
        return gems_rms_forward(x, residual, self.weight, self.eps)

    def extra_repr(self):
        return "{}, eps={}, elementwise_affine={}".format(self.normalized_shape, self.eps, self.elementwise_affine)
