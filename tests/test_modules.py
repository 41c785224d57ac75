"""Module shims (reference: modules_tests/test_gems_rotary_embedding.py, test_gems_normalization.py,
test_gems_activation.py).  The table builders run on the host and are checked here without a GPU; the
forward passes are in tests/test_gpu_modules.py."""
import math

import torch

import flag_gems
from flag_gems.modules import GemsDeepseekYarnRoPE, GemsRMSNorm, GemsRope, GemsSiluAndMul
from flag_gems.modules.rotary_embedding import (
    yarn_find_correction_dim, yarn_find_correction_range, yarn_get_mscale, yarn_linear_ramp_mask,
)
from oracle import torch_ref as O


def test_module_surface():
    assert flag_gems.modules.__all__ == sorted(flag_gems.modules.__all__)
    n = GemsRMSNorm(64, eps=1e-5)
    assert n.normalized_shape == (64,) and n.eps == 1e-5 and torch.equal(n.weight.data, torch.ones(64))
    assert "elementwise_affine=True" in repr(n)
    assert GemsRMSNorm([4, 8], elementwise_affine=False).weight is None
    assert isinstance(GemsSiluAndMul(), torch.nn.Module)


def test_rope_tables_match_the_oracle():
    for dim, max_pos, base in ((64, 128, 10000), (128, 77, 500000.0), (16, 5, 100)):
        rope = GemsRope(dim, max_pos, base, False, torch.float32, None)
        cos, sin = O.rope_cos_sin(max_pos, dim, base)
        assert rope.cos_cached.shape == (max_pos, dim // 2) and rope.sin_cached.shape == (max_pos, dim // 2)
        assert torch.allclose(rope.cos_cached, cos, atol=1e-6) and torch.allclose(rope.sin_cached, sin, atol=1e-6)
        # closed form of single entries
        i, p = dim // 4, max_pos - 1
        assert math.isclose(float(rope.cos_cached[p, i]), math.cos(p * base ** (-2 * i / dim)), abs_tol=1e-5)
    half = GemsRope(64, 16, 10000, True, torch.float16, None)
    assert half.cos_cached.dtype == torch.float16 and not dict(half.named_buffers()) == {}
    assert "cos_cached" not in half.state_dict()  # tables are rebuilt, not stored


def test_yarn_helpers():
    assert yarn_get_mscale(1.0, 5.0) == 1.0 and yarn_get_mscale(0.5, 1.0) == 1.0
    assert math.isclose(yarn_get_mscale(40, 1.0), 0.1 * math.log(40) + 1.0)
    # the correction index is where a frequency pair completes `n` turns over the original context:
    # base^(2 d / dim) * 2 pi * n == max_position_embeddings
    for n, dim, base, ctx in ((32, 64, 10000, 4096), (1, 128, 10000, 4096), (4, 96, 500000, 8192)):
        d = yarn_find_correction_dim(n, dim, base, ctx)
        assert math.isclose(base ** (2 * d / dim) * 2 * math.pi * n, ctx, rel_tol=1e-9)
    lo, hi = yarn_find_correction_range(32, 1, 64, 10000, 4096)
    assert 0 <= lo < hi <= 63
    assert yarn_find_correction_range(1e9, 1e-9, 64, 10000, 4096) == (0, 63)  # clamped to the table
    ramp = yarn_linear_ramp_mask(2, 6, 10)
    assert torch.equal(ramp, torch.tensor([0, 0, 0, 0.25, 0.5, 0.75, 1, 1, 1, 1.0]))
    assert torch.isfinite(yarn_linear_ramp_mask(3, 3, 8)).all()


def test_yarn_tables():
    plain = GemsRope(64, 256, 10000, False, torch.float32, None)
    same = GemsDeepseekYarnRoPE(64, 256, scaling_factor=1.0)
    # (the blend x * (1 - k) + x * k rounds differently from x; position 255 magnifies that to ~3e-5)
    assert torch.allclose(same.cos_cached, plain.cos_cached, atol=1e-4) and torch.allclose(same.sin_cached, plain.sin_cached, atol=1e-4)
    yarn = GemsDeepseekYarnRoPE(64, 256, scaling_factor=40, original_max_position_embeddings=4096, mscale=1.0,
                                mscale_all_dim=1.0)
    inv = yarn._compute_inv_freq()
    lo, hi = yarn_find_correction_range(32.0, 1.0, 64, 10000, 4096)
    base_freq = 1.0 / (10000.0 ** (torch.arange(0, 64, 2, dtype=torch.float32) / 64))
    assert torch.allclose(inv[: lo + 1], base_freq[: lo + 1])             # fast frequencies are kept
    assert torch.allclose(inv[hi:], base_freq[hi:] / 40)                  # slow ones are stretched by the factor
    mid = inv[lo + 1: hi]
    assert ((mid < base_freq[lo + 1: hi]) & (mid > base_freq[lo + 1: hi] / 40)).all()
    assert yarn._table_scale() == 1.0
    scaled = GemsDeepseekYarnRoPE(64, 256, scaling_factor=40, mscale=1.0, mscale_all_dim=0.0)
    ms = 0.1 * math.log(40) + 1.0
    assert math.isclose(scaled._table_scale(), ms, rel_tol=1e-6)
    assert torch.allclose(scaled.cos_cached, yarn.cos_cached * ms, atol=1e-6)
    assert math.isclose(float(scaled.cos_cached[0, 0]), ms, rel_tol=1e-6)  # cos(0) * mscale
