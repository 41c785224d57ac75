"""Forward passes of the module shims on the GPU against the CPU oracle (reference:
modules_tests/test_gems_normalization.py:19-112, test_gems_rotary_embedding.py:15-190, test_gems_activation.py)."""
import numpy as np
import pytest
import torch

from flag_gems.modules import GemsDeepseekYarnRoPE, GemsRMSNorm, GemsRope, GemsSiluAndMul
from oracle import torch_ref as O

from helpers import FLOAT_DTYPES, gems_assert_close

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("shape", [(4, 64), (8, 128), (1024, 1024), (3, 5, 4096)])
@pytest.mark.parametrize("dtype", FLOAT_DTYPES)
def test_gems_rmsnorm(gpu, shape, dtype):
    np.random.seed(42)
    n = shape[-1]
    x = torch.tensor(np.random.uniform(-0.1, 0.1, shape).astype(np.float32), dtype=dtype, device=gpu)
    w = torch.tensor(np.random.uniform(-0.1, 0.1, n).astype(np.float32), dtype=dtype, device=gpu)
    mod = GemsRMSNorm(n, eps=1e-6).to(dtype=dtype, device=gpu)
    mod.weight.data.copy_(w)
    with torch.no_grad():
        out = mod(x)
    gems_assert_close(out, O.rms_norm(x, w, 1e-6), dtype, reduce_dim=n)
    # with a residual: both tensors are updated in place and returned
    res = torch.randn_like(x) / (2 * n)
    ref_x, ref_res = O.fused_add_rms_norm(x, res, w, 1e-6)
    xi, ri = x.clone(), res.clone()
    with torch.no_grad():
        ox, orr = mod(xi, ri)
    assert ox.data_ptr() == xi.data_ptr() and orr.data_ptr() == ri.data_ptr()
    gems_assert_close(ox, ref_x, dtype, reduce_dim=n)
    gems_assert_close(orr, ref_res, dtype)


@pytest.mark.parametrize("q_heads,k_heads", [(8, 1), (8, 8)])
@pytest.mark.parametrize("head_dim", [64, 128, 256])
@pytest.mark.parametrize("interleaved", [True, False])
@pytest.mark.parametrize("yarn", [False, True])
def test_gems_rope_modules(gpu, q_heads, k_heads, head_dim, interleaved, yarn):
    torch.manual_seed(42)
    batch, seq, max_pos, dtype = 8, 77, 2048, torch.float32
    q = torch.randn(batch, seq, q_heads, head_dim, dtype=dtype, device=gpu)
    k = torch.randn(batch, seq, k_heads, head_dim, dtype=dtype, device=gpu)
    pos = torch.randint(0, max_pos, (batch, seq), device=gpu)
    if yarn:
        rope = GemsDeepseekYarnRoPE(head_dim, max_pos, base=10000, device=gpu, dtype=dtype, rotary_interleaved=interleaved,
                                    scaling_factor=40, original_max_position_embeddings=4096, beta_fast=32, beta_slow=1,
                                    mscale=1.0, mscale_all_dim=0.0)
    else:
        rope = GemsRope(head_dim, max_pos, 10000, interleaved, dtype, gpu)
    assert rope.cos_cached.shape == (max_pos, head_dim // 2) and rope.cos_cached.device.type == "cuda"
    ref_q, ref_k = O.apply_rotary_pos_emb(q, k, rope.cos_cached, rope.sin_cached, pos, interleaved)
    oq, ok = rope(q, k, position_ids=pos)
    gems_assert_close(oq, ref_q, dtype); gems_assert_close(ok, ref_k, dtype)
    qi, ki = q.clone(), k.clone()
    rq, rk = rope(qi, ki, position_ids=pos, inplace=True)
    assert rq.data_ptr() == qi.data_ptr() and torch.equal(qi, oq) and torch.equal(ki, ok)


@pytest.mark.parametrize("dtype", FLOAT_DTYPES)
def test_gems_silu_and_mul(gpu, dtype):
    torch.manual_seed(0)
    x = torch.randn(37, 11008, dtype=dtype, device=gpu); y = torch.randn_like(x)
    gems_assert_close(GemsSiluAndMul()(x, y), O.silu_and_mul(x, y), dtype)
