"""nn.Module shims over the operators of this package, with the reference's names and constructor
arguments (src/flag_gems/modules/__init__.py:1-12), so that a model written against
`flag_gems.modules` runs on the gfx950 kernels unchanged."""
from .activation import GemsSiluAndMul
from .normalization import GemsRMSNorm
from .rotary_embedding import GemsDeepseekYarnRoPE, GemsRope

__all__ = ["GemsDeepseekYarnRoPE", "GemsRMSNorm", "GemsRope", "GemsSiluAndMul"]
