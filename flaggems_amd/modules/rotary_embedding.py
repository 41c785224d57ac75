"""Rotary position embedding modules: the cos/sin tables are built once on the host side of torch,
the rotation runs in the gfx950 kernel (reference: src/flag_gems/modules/rotary_embedding.py:36-291;
the YaRN frequency blend is the published DeepSeek-R1 recipe)."""
import logging
import math

import torch
import torch.nn as nn

from ..fused import apply_rotary_pos_emb

logger = logging.getLogger("flag_gems.modules.rotary_embedding")

__all__ = ["gems_rope_forward", "GemsDeepseekYarnRoPE", "GemsRope"]


def gems_rope_forward(query, key, cos, sin, position_ids=None, rotary_interleaved=False, inplace=False):
    logger.debug("GEMS CUSTOM ROPE FORWARD")
    return apply_rotary_pos_emb(query, key, cos, sin, position_ids, rotary_interleaved, inplace)


class GemsRope(nn.Module):
    """Plain RoPE.  Buffers `cos_cached` / `sin_cached` have shape (max_position_embeddings, rotary_dim // 2)
    and hold cos / sin of position * base^(-2i / rotary_dim).  forward(query (..., q_heads, d),
    key (..., k_heads, d), position_ids=None, inplace=False) returns the rotated (query, key)."""

    def __init__(self, rotary_dim, max_position_embeddings, base, rotary_interleaved, dtype, device):
        super().__init__()
        self.rotary_dim = rotary_dim
        self.max_position_embeddings = max_position_embeddings
        self.base = base
        self.rotary_interleaved = rotary_interleaved
        self.dtype = dtype
        self.device = device
        self._set_cos_sin_cache()

    def _exponents(self):
        return torch.arange(0, self.rotary_dim, 2, dtype=torch.float32, device=self.device) / self.rotary_dim

    def _compute_inv_freq(self):
        # written as a reciprocal, the way serving stacks build their tables: base ** (-e) differs from it in
        # the last bit, which a large position turns into a visible difference of the angle
        return 1.0 / (self.base ** self._exponents())

    def _table_scale(self):
        return 1.0

    def _set_cos_sin_cache(self):
        positions = torch.arange(self.max_position_embeddings, device=self.device, dtype=torch.float32)
        angles = torch.outer(positions, self._compute_inv_freq())
        scale = self._table_scale()
        self.register_buffer("cos_cached", (angles.cos() * scale).to(self.dtype), persistent=False)
        self.register_buffer("sin_cached", (angles.sin() * scale).to(self.dtype), persistent=False)

    def forward(self, query, key, position_ids=None, inplace=False):
        if not hasattr(self, "cos_cached") or not hasattr(self, "sin_cached"):
            self._set_cos_sin_cache()
        return gems_rope_forward(query, key, self.cos_cached, self.sin_cached, position_ids, self.rotary_interleaved, inplace)


def yarn_find_correction_dim(num_rotations, dim, base=10000, max_position_embeddings=2048):
    """Index of the frequency pair that completes `num_rotations` turns over the original context."""
    return dim * math.log(max_position_embeddings / (num_rotations * 2 * math.pi)) / (2 * math.log(base))


def yarn_find_correction_range(low_rot, high_rot, dim, base=10000, max_position_embeddings=2048):
    low = math.floor(yarn_find_correction_dim(low_rot, dim, base, max_position_embeddings))
    high = math.ceil(yarn_find_correction_dim(high_rot, dim, base, max_position_embeddings))
    return max(low, 0), min(high, dim - 1)


def yarn_get_mscale(scale=1, mscale=1):
    return 1.0 if scale <= 1 else 0.1 * mscale * math.log(scale) + 1.0


def yarn_linear_ramp_mask(lo, hi, dim):
    if lo == hi:
        hi += 0.001  # keeps the ramp finite
    return torch.clamp((torch.arange(dim, dtype=torch.float32) - lo) / (hi - lo), 0, 1)


class GemsDeepseekYarnRoPE(GemsRope):
    """YaRN RoPE as used by DeepSeek: frequencies below the correction range keep the original spacing,
    those above are divided by `scaling_factor`, with a linear blend in between; the tables are
    multiplied by mscale(scaling_factor, mscale) / mscale(scaling_factor, mscale_all_dim)."""

    def __init__(self, rotary_dim, max_position_embeddings=2048, base=10000, rotary_interleaved=False,
                 dtype=torch.float32, device=None, scaling_factor=1.0, original_max_position_embeddings=4096,
                 beta_fast=32.0, beta_slow=1.0, mscale=1.0, mscale_all_dim=0.0):
        self.scaling_factor = scaling_factor
        self.original_max_position_embeddings = original_max_position_embeddings
        self.beta_fast = beta_fast
        self.beta_slow = beta_slow
        self.mscale = mscale
        self.mscale_all_dim = mscale_all_dim
        super().__init__(rotary_dim=rotary_dim, max_position_embeddings=max_position_embeddings, base=base,
                         rotary_interleaved=rotary_interleaved, dtype=dtype, device=device)

    def _compute_inv_freq(self):
        spread = self.base ** self._exponents()
        extrapolated = 1.0 / spread
        interpolated = 1.0 / (self.scaling_factor * spread)
        low, high = yarn_find_correction_range(self.beta_fast, self.beta_slow, self.rotary_dim, self.base,
                                               self.original_max_position_embeddings)
        keep = 1.0 - yarn_linear_ramp_mask(low, high, self.rotary_dim // 2).to(device=self.device, dtype=torch.float32)
        return interpolated * (1 - keep) + extrapolated * keep

    def _table_scale(self):
        return float(yarn_get_mscale(self.scaling_factor, self.mscale) / yarn_get_mscale(self.scaling_factor, self.mscale_all_dim))
