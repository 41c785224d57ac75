"""GPU parity of the HBM-bound operators (rms_norm, fused_add_rms_norm, softmax, rope, silu_and_mul,
reshape_and_cache_flash) against the CPU oracle and the committed golden fixtures.  Shapes follow
tests/test_norm_ops.py:516-632, tests/test_reduction_ops.py:507-523, tests/test_special_ops.py:164-219,
tests/test_binary_pointwise_ops.py:1377-1403 and tests/test_attention_ops.py:1389-1470 of the reference."""
import os
import random

import numpy as np
import pytest
import torch

import flag_gems
from oracle import torch_ref as O

from helpers import FLOAT_DTYPES, REDUCTION_SHAPES, SOFTMAX_SHAPES, gems_assert_close, gems_assert_equal

pytestmark = pytest.mark.gpu
GOLD = np.load(os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "golden_v1.npz"))


def g(name, dtype, dev):
    return torch.from_numpy(GOLD[name]).to(dtype).to(dev)


@pytest.mark.parametrize("dtype", FLOAT_DTYPES)
@pytest.mark.parametrize("shape", REDUCTION_SHAPES + [(64, 4096), (3, 5, 1024), (17, 8200), (5, 65536), (5, 4099), (3, 70001),
                                                      (2, 131072), (7, 1001), (9, 33), (6, 100), (4, 300), (3, 500)])
def test_rms_norm(gpu, shape, dtype):
    np.random.seed(0)
    x = torch.from_numpy(np.random.uniform(-0.1, 0.1, shape).astype(np.float32)).to(dtype).to(gpu)
    w = torch.from_numpy(np.random.uniform(-0.1, 0.1, shape[-1:]).astype(np.float32)).to(dtype).to(gpu)
    ref = O.rms_norm(x, w, 1e-5)
    res = flag_gems.rms_norm(x, list(shape[-1:]), w, 1e-5)
    gems_assert_close(res, ref, dtype)
    with flag_gems.use_gems():
        res2 = torch.nn.functional.rms_norm(x, list(shape[-1:]), w, 1e-5)
    assert torch.equal(res, res2)


def test_rms_norm_schema_defaults_and_autograd(gpu):
    x = torch.randn(6, 96, device=gpu)
    with flag_gems.use_gems():
        y = torch.nn.functional.rms_norm(x, [96])  # weight=None, eps=None
    xf = x.double().cpu()
    ref = xf * torch.rsqrt(xf.pow(2).mean(-1, keepdim=True) + torch.finfo(torch.float32).eps)
    gems_assert_close(y, ref, torch.float32)
    # two trailing dims
    w = torch.randn(4, 24, device=gpu)
    gems_assert_close(flag_gems.rms_norm(x.view(6, 4, 24), [4, 24], w, 1e-5), O.rms_norm(x, w.view(96), 1e-5).view(6, 4, 24),
                      torch.float32)
    # a graph through the override differentiates through the backward kernel
    xg = x.clone().requires_grad_(True)
    with flag_gems.use_gems():
        torch.nn.functional.rms_norm(xg, [96], torch.ones(96, device=gpu), 1e-5).sum().backward()
    ref_dx, _ = O.rms_norm_grads(x, torch.ones(96), 1e-5, torch.ones(6, 96))
    gems_assert_close(xg.grad, ref_dx, torch.float32)


@pytest.mark.parametrize("dtype", FLOAT_DTYPES)
@pytest.mark.parametrize("shape", REDUCTION_SHAPES + [(4096, 4096), (33, 1000), (5, 4099), (3, 70001), (2, 131072), (7, 1001), (9, 33), (4, 300)])
def test_fused_add_rms_norm(gpu, shape, dtype):
    torch.manual_seed(0)
    x = torch.randn(shape, dtype=dtype, device=gpu); r = torch.randn(shape, dtype=dtype, device=gpu)
    w = torch.randn(shape[-1:], dtype=dtype, device=gpu)
    ref_y, ref_r = O.fused_add_rms_norm(x, r, w, 1e-5)
    xi, ri = x.clone(), r.clone()
    y, rr = flag_gems.fused_add_rms_norm(xi, ri, list(shape[-1:]), w, 1e-5)
    gems_assert_close(y, ref_y, dtype)
    gems_assert_close(rr, ref_r, dtype)
    assert y.data_ptr() == xi.data_ptr() and rr.data_ptr() == ri.data_ptr()  # in place


@pytest.mark.parametrize("dtype", FLOAT_DTYPES)
@pytest.mark.parametrize("shape", SOFTMAX_SHAPES + [(16, 2048), (7, 40999), (5, 33), (3, 70000), (9, 1001), (6, 100), (4, 300),
                                                    (3, 600), (5, 1500), (2, 131072)])
@pytest.mark.parametrize("neg_inf", [False, True])
def test_softmax(gpu, shape, dtype, neg_inf):
    torch.manual_seed(0)
    for dim in range(len(shape)):
        x = torch.randn(shape, dtype=dtype, device=gpu)
        if neg_inf:
            x = torch.where(x < 0.0, float("-inf"), x)
        ref = O.softmax(x, dim)
        with flag_gems.use_gems():
            res = torch.nn.functional.softmax(x, dim=dim)
        gems_assert_close(res, ref, dtype, equal_nan=True)
    # half_to_float and a negative dim
    if dtype != torch.float32:
        res = flag_gems.softmax(x, -1, True)
        gems_assert_close(res, O.softmax(x, -1), torch.float32, equal_nan=True)


# Rows of every kernel of the inner axis (registers; one wave per short unaligned row; two sweeps for unaligned and
# for long rows) with a NaN, with nothing but -inf, with -inf in front of the first finite value, and untouched.
@pytest.mark.parametrize("dtype", FLOAT_DTYPES)
@pytest.mark.parametrize("N", [33, 256, 1001, 1500, 4097, 70001, 131072])
def test_softmax_special_rows(gpu, N, dtype):
    torch.manual_seed(N)
    x = torch.randn(5, N, dtype=dtype, device=gpu)
    x[0, N // 3] = float("nan")
    x[1] = float("-inf")
    x[2, : N - 2] = float("-inf")
    x[3, N - 1] = float("nan")
    for fn, ref_fn in ((flag_gems.softmax, O.softmax), (flag_gems.log_softmax, O.log_softmax)):
        res = fn(x, -1)
        ref = ref_fn(x, -1)
        assert torch.isnan(res[0]).all() and torch.isnan(res[1]).all() and torch.isnan(res[3]).all()
        gems_assert_close(res[2], ref[2], dtype, equal_nan=True)
        gems_assert_close(res[4], ref[4], dtype)


# log_softmax: the same kernels with (x - max) - log(sum) as the last step (reference test:
# tests/test_reduction_ops.py:466-480); vocabulary-sized rows included, -inf entries stay -inf.
@pytest.mark.parametrize("dtype", FLOAT_DTYPES)
@pytest.mark.parametrize("shape", SOFTMAX_SHAPES + [(16, 2048), (7, 40999), (5, 33), (3, 70000), (8, 32000), (2, 151936)])
def test_log_softmax(gpu, shape, dtype):
    torch.manual_seed(0)
    for dim in range(len(shape)):
        x = torch.randn(shape, dtype=dtype, device=gpu)
        ref = O.log_softmax(x, dim)
        with flag_gems.use_gems():
            res = torch.nn.functional.log_softmax(x, dim=dim)
        gems_assert_close(res, ref, dtype)
    xm = torch.where(x < -1.0, float("-inf"), x)
    res = flag_gems.log_softmax(xm, -1)
    fin = torch.isfinite(xm)
    live = fin.any(-1, keepdim=True)  # a row of nothing but -inf is NaN (-inf - -inf), as in torch
    assert (res[(~fin) & live] == float("-inf")).all()
    gems_assert_close(res[fin], O.log_softmax(xm, -1)[fin.cpu()], dtype)
    assert torch.isnan(res[(~live).expand_as(res)]).all()
    if dtype != torch.float32:  # half_to_float
        res = flag_gems.log_softmax(x, -1, True)
        assert res.dtype == torch.float32
        gems_assert_close(res, O.log_softmax(x, -1), torch.float32)
    # exp(log_softmax) is softmax
    torch.testing.assert_close(flag_gems.log_softmax(x, -1).double().exp().cpu(), O.softmax(x, -1), atol=1e-3, rtol=2e-2)


def test_softmax_full_size_properties(gpu):
    """[131072, 2048] bf16 with 1 % -inf (the benchmark input): rows sum to 1, masked entries are exact
    zeros, sampled rows match the oracle, and adding a constant to a row changes nothing."""
    torch.manual_seed(0)
    x = torch.randn(131072, 2048, device=gpu) * 2
    x[torch.rand_like(x) < 0.01] = float("-inf")
    x = x.bfloat16()
    y = flag_gems.softmax(x, -1)
    assert (y[x == float("-inf")] == 0).all()
    s = y.float().sum(-1)
    assert float((s - 1).abs().max()) < 2e-2  # 2048 bf16 roundings of values that sum to one
    rows = torch.tensor([0, 1, 777, 65535, 65536, 131071], device=gpu)
    gems_assert_close(y[rows], O.softmax(x[rows], -1), torch.bfloat16)
    xf = x[rows].float()
    gems_assert_close(flag_gems.softmax(xf + 4.0, -1), O.softmax(xf, -1), torch.float32)


@pytest.mark.parametrize("dtype", FLOAT_DTYPES)
@pytest.mark.parametrize("q_heads,k_heads", [(8, 1), (6, 2), (1, 1), (8, 8)])
@pytest.mark.parametrize("head_dim", [64, 96, 128, 256])
@pytest.mark.parametrize("interleaved", [False, True])
@pytest.mark.parametrize("has_pos", [False, True])
def test_apply_rotary_pos_emb(gpu, dtype, q_heads, k_heads, head_dim, interleaved, has_pos):
    torch.manual_seed(0)
    batch, seq, max_pos = 4, 33, 512
    q = torch.randn(batch, seq, q_heads, head_dim, dtype=dtype, device=gpu)
    k = torch.randn(batch, seq, k_heads, head_dim, dtype=dtype, device=gpu)
    pos = torch.randint(0, max_pos, (batch, seq), device=gpu) if has_pos else None
    cos, sin = O.rope_cos_sin(max_pos, head_dim, device=gpu)
    ref_q, ref_k = O.apply_rotary_pos_emb(q, k, cos, sin, pos, interleaved)
    oq, ok = flag_gems.apply_rotary_pos_emb(q, k, cos, sin, pos, interleaved)
    gems_assert_close(oq, ref_q, dtype); gems_assert_close(ok, ref_k, dtype)
    qi, ki = q.clone(), k.clone()
    rq, rk = flag_gems.apply_rotary_pos_emb(qi, ki, cos, sin, pos, interleaved, inplace=True)
    assert rq.data_ptr() == qi.data_ptr() and torch.equal(qi, oq) and torch.equal(ki, ok)


def test_rope_fused_qkv_views_and_table_layouts(gpu):
    """q/k as slices of one qkv buffer (token stride 3*H*D), int32 positions, bf16 cos/sin taken as
    halves of one [max_pos, D] table (row stride D), and an unaligned view that takes the scalar path."""
    torch.manual_seed(1)
    T, H, D = 50, 4, 128
    qkv = torch.randn(T, 3 * H * D, dtype=torch.bfloat16, device=gpu)
    q, k = qkv[:, : H * D].view(T, H, D), qkv[:, H * D: 2 * H * D].view(T, H, D)
    c32, s32 = O.rope_cos_sin(256, D, device=gpu)
    table = torch.cat([c32, s32], -1).bfloat16()
    cos, sin = table.chunk(2, -1)
    pos = torch.randint(0, 256, (T,), device=gpu, dtype=torch.int32)
    ref_q, ref_k = O.apply_rotary_pos_emb(q, k, cos, sin, pos, False)
    keep = qkv[:, 2 * H * D:].clone()
    flag_gems.apply_rotary_pos_emb(q, k, cos, sin, pos, False, inplace=True)
    gems_assert_close(q, ref_q, torch.bfloat16); gems_assert_close(k, ref_k, torch.bfloat16)
    assert torch.equal(qkv[:, 2 * H * D:], keep)  # v untouched
    buf = torch.randn(T * H * D + 1, dtype=torch.bfloat16, device=gpu)
    qu = buf[1:].view(T, H, D)  # 2-byte aligned only
    ref_q, _ = O.apply_rotary_pos_emb(qu, qu, cos, sin, pos, True)
    oq, _ = flag_gems.apply_rotary_pos_emb(qu, qu, cos, sin, pos, True)
    gems_assert_close(oq, ref_q, torch.bfloat16)


@pytest.mark.parametrize("dtype", FLOAT_DTYPES)
@pytest.mark.parametrize("shape", [(), (2, 19, 7), (1024, 1024), (16, 22016), (3, 4, 5, 6, 8), (33, 4099), (5, 1), (7, 8206)])
def test_silu_and_mul(gpu, shape, dtype):
    torch.manual_seed(0)
    if shape == (16, 22016):  # the two halves of a gate-up projection: strided rows, no copy
        gu = torch.randn(shape, dtype=dtype, device=gpu)
        a, b = gu[:, :11008], gu[:, 11008:]
    elif shape == (7, 8206):  # halves with an odd split: element-aligned starts, ragged last pack
        gu = torch.randn(shape, dtype=dtype, device=gpu)
        a, b = gu[:, :4103], gu[:, 4103:]
    else:
        a = torch.randn(shape, dtype=dtype, device=gpu); b = torch.randn(shape, dtype=dtype, device=gpu)
    ref = O.silu_and_mul(a, b)
    gems_assert_close(flag_gems.silu_and_mul(a, b), ref, dtype)
    out = torch.empty(a.shape, dtype=dtype, device=gpu)
    assert flag_gems.silu_and_mul_out(a, b, out) is out
    gems_assert_close(out, ref, dtype)


@pytest.mark.parametrize("dtype", FLOAT_DTYPES)
@pytest.mark.parametrize("head_size", [64, 80, 120, 256])
@pytest.mark.parametrize("block_size", [8, 16, 32])
@pytest.mark.parametrize("num_blocks", [1024, 10000])
def test_reshape_and_cache_flash(gpu, dtype, head_size, block_size, num_blocks):
    random.seed(0); torch.manual_seed(0)
    num_tokens, num_heads = 42, 8
    slots = torch.tensor(random.sample(range(num_blocks * block_size), num_tokens), dtype=torch.long, device=gpu)
    qkv = torch.randn(num_tokens, 3, num_heads, head_size, dtype=dtype, device=gpu)
    _, key, value = qkv.unbind(dim=1)  # strided views
    kc = torch.randn(num_blocks, block_size, num_heads, head_size, dtype=dtype, device=gpu); vc = torch.randn_like(kc)
    ref_k, ref_v = O.reshape_and_cache_flash(key, value, kc, vc, slots)
    flag_gems.reshape_and_cache_flash(key, value, kc, vc, slots, "auto", None, None)
    gems_assert_equal(kc, ref_k); gems_assert_equal(vc, ref_v)  # bit-exact, written slots and the untouched rest


def test_reshape_and_cache_flash_edges(gpu):
    torch.manual_seed(1)
    H, D, bs, nb = 2, 24, 4, 9
    key = torch.randn(7, H, D, dtype=torch.float16, device=gpu); value = torch.randn_like(key)
    kv = torch.zeros(2, nb, bs, H, D, dtype=torch.float16, device=gpu)
    kc, vc = kv.unbind(0)
    # negative slots are padding; int32 slots; fewer slots than key rows
    slots = torch.tensor([5, -1, 0, 35, -7], dtype=torch.int32, device=gpu)
    ref_k, ref_v = O.reshape_and_cache_flash(key, value, kc, vc, slots)
    flag_gems.reshape_and_cache_flash(key, value, kc, vc, slots, "auto", None, None)
    gems_assert_equal(kc, ref_k); gems_assert_equal(vc, ref_v)
    assert int((kc != 0).any(-1).any(-1).sum()) == 3
    # a page stride larger than a page (padded cache), single-byte elements
    big = torch.zeros(nb, bs + 1, H, D, dtype=torch.uint8, device=gpu)
    kc8, vc8 = big[:, :bs], big.clone()[:, :bs]
    k8 = torch.randint(1, 255, (7, H, D), dtype=torch.uint8, device=gpu)
    s64 = torch.tensor([1, 2, 3, 4, 5, 6, 30], device=gpu)
    ref_k, ref_v = O.reshape_and_cache_flash(k8, k8, kc8, vc8, s64)
    flag_gems.reshape_and_cache_flash(k8, k8, kc8, vc8, s64, "auto", None, None)
    gems_assert_equal(kc8, ref_k); gems_assert_equal(vc8, ref_v)
    assert int(big[:, bs].sum()) == 0  # the padding slot of every page stays zero
    # empty
    flag_gems.reshape_and_cache_flash(key[:0], value[:0], kc, vc, slots[:0], "auto", None, None)


def test_rowwise_golden(gpu):
    bf16, f16 = torch.bfloat16, torch.float16
    for tag, dt in (("bf16", bf16), ("f16", f16)):
        x, r, w = g(f"rms_{tag}_x", dt, gpu), g(f"rms_{tag}_r", dt, gpu), g(f"rms_{tag}_w", dt, gpu)
        gems_assert_close(flag_gems.rms_norm(x, [x.shape[-1]], w, 1e-5), torch.from_numpy(GOLD[f"rms_{tag}_y"]), dt)
        y, rr = flag_gems.fused_add_rms_norm(x.clone(), r.clone(), [x.shape[-1]], w, 1e-5)
        gems_assert_close(y, torch.from_numpy(GOLD[f"fused_{tag}_y"]), dt)
        gems_assert_close(rr, torch.from_numpy(GOLD[f"fused_{tag}_res"]), dt)
    gems_assert_close(flag_gems.softmax(g("softmax_bf16_x", bf16, gpu), -1), torch.from_numpy(GOLD["softmax_bf16_y"]), bf16,
                      equal_nan=True)
    for inter in (False, True):
        oq, ok = flag_gems.apply_rotary_pos_emb(g("rope_q", bf16, gpu), g("rope_k", bf16, gpu), g("rope_cos", torch.float32, gpu),
                                                g("rope_sin", torch.float32, gpu), g("rope_pos", torch.int64, gpu), inter)
        gems_assert_close(oq, torch.from_numpy(GOLD[f"rope_oq_{int(inter)}"]), bf16)
        gems_assert_close(ok, torch.from_numpy(GOLD[f"rope_ok_{int(inter)}"]), bf16)
    gems_assert_close(flag_gems.silu_and_mul(g("silu_a", f16, gpu), g("silu_b", f16, gpu)), torch.from_numpy(GOLD["silu_y"]), f16)
    kc, vc = g("cache_kc0", bf16, gpu), g("cache_vc0", bf16, gpu)
    flag_gems.reshape_and_cache_flash(g("cache_key", bf16, gpu), g("cache_val", bf16, gpu), kc, vc, g("cache_slots", torch.int64, gpu),
                                      "auto", None, None)
    gems_assert_equal(kc, torch.from_numpy(GOLD["cache_kc1"]).to(bf16)); gems_assert_equal(vc, torch.from_numpy(GOLD["cache_vc1"]).to(bf16))
    a, b, bias = g("mm_f16_a", f16, gpu), g("mm_f16_b", f16, gpu), g("mm_f16_bias", f16, gpu)
    gems_assert_close(flag_gems.mm(a, b), torch.from_numpy(GOLD["mm_f16_c"]), f16, reduce_dim=24)
    gems_assert_close(flag_gems.addmm(bias, a, b, alpha=-0.999, beta=100.001), torch.from_numpy(GOLD["addmm_f16_c"]), f16, reduce_dim=24)
