"""silu(x) * y as a module (reference: src/flag_gems/modules/activation.py:17-37)."""
import logging

import torch.nn as nn

from ..fused import silu_and_mul

logger = logging.getLogger("flag_gems.modules.activation")

__all__ = ["gems_silu_and_mul", "GemsSiluAndMul"]


def gems_silu_and_mul(x, y):
    logger.debug("GEMS CUSTOM SILU_AND_MUL FORWARD")
    return silu_and_mul(x, y)


class GemsSiluAndMul(nn.Module):
    """forward(x, y) = silu(x) * y in one kernel."""

    def forward(self, x, y):
        return gems_silu_and_mul(x, y)
