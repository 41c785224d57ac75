"""GPU parity of flash_attn_varlen_func over a paged KV cache against the CPU oracle
(ref_paged_attn of the reference's tests/test_attention_ops.py:819-995, atol 2e-2 / rtol 1e-2), plus
the decoder-layer pipeline of the benchmark configuration at a reduced token count."""
import os

import numpy as np
import pytest
import torch

import flag_gems
from oracle import torch_ref as O

pytestmark = pytest.mark.gpu
GOLD = np.load(os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "golden_v1.npz"))
ATOL, RTOL = 2e-2, 1e-2  # tests/test_attention_ops.py:990-992


def make_case(dev, seq_lens, Hq, Hk, D, block_size, num_blocks, dtype, seed=1234567890):
    torch.manual_seed(seed)
    qlens = [s[0] for s in seq_lens]; klens = [s[1] for s in seq_lens]
    q = torch.randn(sum(qlens), Hq, D, dtype=dtype, device=dev)
    kc = torch.randn(num_blocks, block_size, Hk, D, dtype=dtype, device=dev); vc = torch.randn_like(kc)
    cu = torch.tensor([0] + qlens, dtype=torch.int32, device=dev).cumsum(0, dtype=torch.int32)
    sk = torch.tensor(klens, dtype=torch.int32, device=dev)
    pages = (max(klens) + block_size - 1) // block_size
    bt = torch.randint(0, num_blocks, (len(seq_lens), pages), dtype=torch.int32, device=dev)  # pages may repeat
    return q, kc, vc, cu, sk, bt, qlens, klens


def check(dev, seq_lens, Hq, Hk, D, block_size, num_blocks, dtype, causal=True, alibi=False, softcap=None, window=None):
    q, kc, vc, cu, sk, bt, qlens, klens = make_case(dev, seq_lens, Hq, Hk, D, block_size, num_blocks, dtype)
    scale = D ** -0.5
    slopes, bias = None, None
    if alibi:
        slopes = torch.ones(len(seq_lens), Hq, device=dev, dtype=torch.float32) * 0.3
        bias = torch.zeros(len(seq_lens), Hq, max(qlens), max(klens))
        for i, (ql, kl) in enumerate(zip(qlens, klens)):
            bias[i, :, :ql, :kl] = O.alibi_bias(slopes[i:i + 1].cpu(), ql, kl, causal)[0]
    out, lse = flag_gems.ops.flash_attn_varlen_func(
        q, kc, vc, max(qlens), cu, max(klens), seqused_k=sk, softmax_scale=scale, causal=causal, window_size=window,
        softcap=softcap or 0.0, alibi_slopes=slopes, block_table=bt, return_softmax_lse=True,
    )
    ref, rlse = O.paged_attention(q, kc, vc, qlens, klens, bt, scale, causal=causal, attn_bias=bias, soft_cap=softcap,
                                  window=window, compute_dtype=torch.float32, return_lse=True)
    torch.testing.assert_close(out.float().cpu(), ref, atol=ATOL, rtol=RTOL)
    lse = lse.cpu()
    fin = torch.isfinite(rlse)
    torch.testing.assert_close(lse[fin], rlse[fin], atol=1e-2, rtol=1e-3)
    assert (lse[~fin] == float("inf")).all()  # rows with no visible key: out = 0, lse = +inf
    return out


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("Hq,Hk", [(4, 4), (8, 2), (16, 2)])
@pytest.mark.parametrize("D", [128, 192, 256])
@pytest.mark.parametrize("num_blocks", [32768, 2048])
@pytest.mark.parametrize("alibi,softcap", [(False, None), (True, None), (False, 10.0), (False, 50.0)])
def test_flash_attn_varlen_reference_grid(gpu, dtype, Hq, Hk, D, num_blocks, alibi, softcap):
    check(gpu, [(1, 1328), (5, 18), (129, 463)], Hq, Hk, D, 32, num_blocks, dtype, alibi=alibi, softcap=softcap)


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("Hq,Hk", [(6, 2), (3, 1), (32, 8)])
@pytest.mark.parametrize("D", [32, 48, 64, 72, 80, 96, 112, 120])
def test_flash_attn_varlen_more_heads_and_dims(gpu, dtype, Hq, Hk, D):
    check(gpu, [(1, 1328), (5, 18), (129, 463), (70, 70)], Hq, Hk, D, 16, 512, dtype)


@pytest.mark.parametrize("causal,window,alibi", [
    (False, None, False), (False, None, True), (True, (50, 0), False), (False, (20, 30), False), (True, (0, 0), False),
    (False, (700, -1), False),
])
def test_flash_attn_varlen_masks(gpu, causal, window, alibi):
    check(gpu, [(7, 300), (130, 130), (64, 200), (1, 1)], 8, 2, 128, 16, 512, torch.bfloat16, causal=causal, window=window,
          alibi=alibi)


def test_flash_attn_varlen_edges(gpu):
    # more queries than keys (leading rows see nothing), an empty KV, page size 1 and a large page
    check(gpu, [(300, 200), (130, 130), (64, 5)], 4, 2, 64, 16, 512, torch.bfloat16)
    check(gpu, [(5, 0), (3, 40)], 4, 4, 128, 16, 64, torch.float16)
    check(gpu, [(9, 77), (33, 33)], 8, 2, 128, 1, 256, torch.bfloat16)
    check(gpu, [(9, 777), (330, 330)], 8, 2, 128, 256, 16, torch.bfloat16)
    # decode batch: one query per sequence
    check(gpu, [(1, 17), (1, 1000), (1, 1), (1, 4096)], 32, 8, 128, 16, 2048, torch.bfloat16)


# Mixed batches, as a serving engine with chunked prefill produces them: sequences with one query token go to the
# single-token kernel (split key ranges), the rest to the prefill kernels, in one call.  Also: a batch of four or
# more without any single-token sequence, one made of nothing else but with max_seqlen_q > 1 passed, empty
# sequences in between, a non-causal batch, and the same batches with the routing switched off.
@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("Hq,Hk,D,block_size", [(32, 8, 128, 16), (8, 8, 64, 32), (12, 4, 128, 64)])
@pytest.mark.parametrize("mixed_env", [None, "0"])
def test_flash_attn_mixed_batches(gpu, fg_env, dtype, Hq, Hk, D, block_size, mixed_env):
    if mixed_env is None:
        fg_env.delenv("FG_ATTN_MIXED", raising=False)
    else:
        fg_env.setenv("FG_ATTN_MIXED", mixed_env)
    check(gpu, [(1, 700), (1, 33), (300, 300), (1, 4096), (64, 1000), (1, 1), (1, 2500), (17, 17)], Hq, Hk, D, block_size,
          2048, dtype)
    check(gpu, [(128, 128), (5, 900), (200, 1200), (33, 64)], Hq, Hk, D, block_size, 1024, dtype)
    check(gpu, [(1, 100), (1, 2000), (1, 3), (1, 513), (1, 64)], Hq, Hk, D, block_size, 1024, dtype)
    check(gpu, [(1, 40), (0, 0), (70, 70), (1, 0), (0, 50), (1, 900)], Hq, Hk, D, block_size, 512, dtype)
    check(gpu, [(1, 300), (40, 300), (1, 1000), (2, 77)], Hq, Hk, D, block_size, 512, dtype, causal=False)
    check(gpu, [(1, 300), (40, 300), (1, 1000), (2, 77)], Hq, Hk, D, block_size, 512, dtype, window=(128, 0))


# The lean kernel (head dim 64 / 128, power-of-two pages): its reference maximum moves lazily and is subtracted
# inside the matrix pipe, so feed it scores that keep growing along the keys (the reference has to move many
# times, by large steps), rows that see their first key late (windows), sequences longer than the 128-tile window
# of page ids it keeps in registers, and the plain grid order next to the XCD-grouped one.
@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("D,Hq,Hk", [(128, 8, 2), (64, 4, 4), (128, 3, 1)])
def test_flash_attn_lean_kernel_reference_moves(gpu, dtype, D, Hq, Hk):
    torch.manual_seed(5)
    lens = [(200, 900), (64, 64), (33, 700)]
    q, kc, vc, cu, sk, bt, qlens, klens = make_case(gpu, lens, Hq, Hk, D, 16, 512, dtype)
    # keys whose projection on a fixed direction grows with the slot index: scores rise along every sequence
    ramp = torch.linspace(0, 6, kc.shape[0] * kc.shape[1], device=gpu).view(kc.shape[0], kc.shape[1], 1, 1)
    kc = (kc.float() * 0.3 + ramp * torch.sign(torch.randn(1, 1, 1, D, device=gpu))).to(dtype)
    q = (q.float().abs() * 0.5).to(dtype)
    scale = D ** -0.5
    out, lse = flag_gems.ops.flash_attn_varlen_func(q, kc, vc, max(qlens), cu, max(klens), seqused_k=sk, softmax_scale=scale,
                                                    causal=True, block_table=bt, return_softmax_lse=True)
    ref, rlse = O.paged_attention(q, kc, vc, qlens, klens, bt, scale, causal=True, compute_dtype=torch.float32, return_lse=True)
    torch.testing.assert_close(out.float().cpu(), ref, atol=ATOL, rtol=RTOL)
    torch.testing.assert_close(lse.cpu(), rlse, atol=2e-2, rtol=2e-3)


@pytest.mark.parametrize("order", [None, "fn"])
def test_flash_attn_lean_kernel_long_sequences_and_grid_orders(gpu, fg_env, order):
    if order is None:
        fg_env.delenv("FG_ATTN_KERNEL")
    else:
        fg_env.setenv("FG_ATTN_KERNEL", order)
    # 8192 keys is 128 tiles: beyond it the page-id window is re-read; page 16 and page 128
    check(gpu, [(40, 9000), (600, 17000), (3, 8193), (130, 130)], 4, 2, 128, 16, 2048, torch.bfloat16)
    check(gpu, [(257, 12345), (64, 64)], 8, 8, 64, 128, 128, torch.float16)
    check(gpu, [(300, 9000)], 4, 1, 128, 16, 1024, torch.bfloat16, causal=False)
    check(gpu, [(500, 10000), (700, 700)], 4, 2, 128, 32, 512, torch.bfloat16, window=(300, 0))
    check(gpu, [(1, 1328), (5, 18), (129, 463), (70, 70)], 8, 2, 128, 16, 512, torch.bfloat16)


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("Hq,Hk,D,block_size", [(32, 8, 128, 16), (8, 8, 64, 32), (16, 2, 64, 16), (32, 32, 128, 64),
                                                 (4, 1, 128, 256), (8, 2, 128, 8), (8, 2, 96, 16)])
def test_flash_attn_decode(gpu, dtype, Hq, Hk, D, block_size):
    # ragged lengths around tile (32), page and range (4096) boundaries, an empty sequence, a long one that
    # needs several key ranges by itself
    check(gpu, [(1, 1), (1, 17), (1, 32), (1, 33), (1, 0), (1, 1000), (1, 4095), (1, 4097)], Hq, Hk, D, block_size, 1024, dtype)
    check(gpu, [(1, 9001)], Hq, Hk, D, block_size, 1024, dtype)           # one sequence: split for parallelism
    check(gpu, [(1, 100 + 37 * i) for i in range(70)], Hq, Hk, D, block_size, 1024, dtype)  # many short ones


def test_flash_attn_decode_variants(gpu):
    lens = [(1, 300), (1, 5000), (1, 64)]
    check(gpu, lens, 32, 8, 128, 16, 1024, torch.bfloat16, causal=False)
    check(gpu, lens, 32, 8, 128, 16, 1024, torch.bfloat16, window=(128, 0))     # left window: general kernel
    check(gpu, lens, 32, 8, 128, 16, 1024, torch.bfloat16, window=(-1, 5))
    check(gpu, lens, 32, 8, 128, 16, 1024, torch.bfloat16, alibi=True)          # ALiBi: general kernel
    check(gpu, lens, 32, 8, 128, 16, 1024, torch.bfloat16, softcap=30.0)
    # a sequence with no query at all among single-token ones
    check(gpu, [(1, 200), (0, 50), (1, 700)], 8, 2, 128, 16, 256, torch.float16)
    # without a workspace the library must still be right (unsplit, or the prefill kernels for long ranges)
    from flaggems_amd import _C
    q, kc, vc, cu, sk, bt, qlens, klens = make_case(gpu, [(1, 3000), (1, 6000)], 32, 8, 128, 16, 1024, torch.bfloat16)
    orig = _C.lib().fg_flash_attn_workspace_bytes
    try:
        _C.lib().fg_flash_attn_workspace_bytes = lambda *a: 0
        out = flag_gems.flash_attn_varlen_func(q, kc, vc, 1, cu, max(klens), seqused_k=sk, causal=True, block_table=bt)
    finally:
        _C.lib().fg_flash_attn_workspace_bytes = orig
    ref = O.paged_attention(q, kc, vc, qlens, klens, bt, 128 ** -0.5, compute_dtype=torch.float32)
    torch.testing.assert_close(out.float().cpu(), ref, atol=ATOL, rtol=RTOL)


# max_seqlen_k is an upper bound, not the longest length present (a caller may pass the model's limit, and one long
# sequence sets it for a whole batch): each sequence cuts its own key ranges from its own length on the device,
# and the merge must read exactly the ranges that sequence wrote.
@pytest.mark.parametrize("max_k", [4096, 32768, 131072])
@pytest.mark.parametrize("min_tiles", [None, "4", "64"])
def test_flash_attn_decode_max_seqlen_k_above_lengths(gpu, fg_env, max_k, min_tiles):
    if min_tiles is not None:
        fg_env.setenv("FG_DECODE_MIN_TILES", min_tiles)
    lens = [(1, n) for n in (2048, 1, 0, 31, 129, 511, 513, 2047, 2049, 3000, 4096, 640)] + [(1, 700 + 61 * i) for i in range(24)]
    q, kc, vc, cu, sk, bt, qlens, klens = make_case(gpu, lens, 32, 8, 128, 16, 1024, torch.bfloat16)
    wide = torch.zeros(bt.shape[0], max_k // 16, dtype=bt.dtype, device=bt.device)
    wide[:, :bt.shape[1]] = bt
    out, lse = flag_gems.ops.flash_attn_varlen_func(q, kc, vc, 1, cu, max_k, seqused_k=sk, causal=True, block_table=wide,
                                                    return_softmax_lse=True)
    ref, rlse = O.paged_attention(q, kc, vc, qlens, klens, bt, 128 ** -0.5, causal=True, compute_dtype=torch.float32,
                                  return_lse=True)
    torch.testing.assert_close(out.float().cpu(), ref, atol=ATOL, rtol=RTOL)
    lse = lse.cpu()
    fin = torch.isfinite(rlse)
    torch.testing.assert_close(lse[fin], rlse[fin], atol=1e-2, rtol=1e-3)
    assert (lse[~fin] == float("inf")).all()  # the sequence without keys: out = 0, lse = +inf
    # the same batch with one sequence that really is that long (bounded so the oracle stays quick)
    if max_k == 32768:
        check(gpu, lens[:8] + [(1, 32768)], 32, 8, 128, 16, 4096, torch.bfloat16)


# Dense attention through the same kernel: aten::_flash_attention_forward and scaled_dot_product_attention
# (reference: tests/test_attention_ops.py:540-575 test_flash_fwd_nonsquare_qk, :578-640 GQA and alibi, :296-330 sdpa).
def _dense_inputs(dev, batch, heads, heads_k, sq, sk, d, dtype):
    torch.manual_seed(1234567890)
    q = torch.empty(batch, heads, sq, d, dtype=dtype, device=dev).uniform_(-0.05, 0.05)
    k = torch.empty(batch, heads_k, sk, d, dtype=dtype, device=dev).uniform_(-0.05, 0.05)
    v = torch.empty(batch, heads_k, sk, d, dtype=dtype, device=dev).uniform_(-0.05, 0.05)
    return q, k, v


@pytest.mark.parametrize("batch,heads,sq,sk", [(1, 1, 128, 2048), (4, 8, 1024, 128), (4, 8, 17, 1030)])
@pytest.mark.parametrize("d", [32, 64, 96, 128, 192, 256])
@pytest.mark.parametrize("causal", [False, True])
@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
def test_flash_attention_forward_nonsquare(gpu, batch, heads, sq, sk, d, causal, dtype):
    q, k, v = _dense_inputs(gpu, batch, heads, heads, sq, sk, d, dtype)
    scale = float(1.0 / np.sqrt(d))
    # the caller holds (batch, heads, seq, d) tensors and passes transposed views, as torch's SDPA front end does
    out, lse, *_ = flag_gems.ops.flash_attention_forward(q.transpose(1, 2), k.transpose(1, 2), v.transpose(1, 2), None, None,
                                                         sq, sk, 0, causal, False, scale=scale)
    ref, rlse = O.dense_attention(q.transpose(1, 2), k.transpose(1, 2), v.transpose(1, 2), scale, causal=causal, return_lse=True)
    atol, rtol = O.gems_tolerance(dtype)
    torch.testing.assert_close(out.float().cpu(), ref, atol=max(atol, 2e-3 if dtype == torch.bfloat16 else 2e-4), rtol=rtol)
    fin = torch.isfinite(rlse)
    torch.testing.assert_close(lse.cpu()[fin], rlse[fin], atol=1e-3, rtol=1e-4)
    assert (lse.cpu()[~fin] == float("inf")).all()


@pytest.mark.parametrize("heads,heads_k", [(8, 2), (6, 3), (4, 1)])
@pytest.mark.parametrize("layout", ["bshd", "bhsd"])
@pytest.mark.parametrize("window,softcap", [((-1, -1), 0.0), ((64, 0), 0.0), ((30, 20), 0.0), ((-1, -1), 15.0)])
def test_flash_attention_forward_gqa_layouts_windows(gpu, heads, heads_k, layout, window, softcap):
    batch, sq, sk, d, dtype = 3, 200, 384, 128, torch.bfloat16
    q, k, v = _dense_inputs(gpu, batch, heads, heads_k, sq, sk, d, dtype)
    if layout == "bshd":
        q, k, v = (t.transpose(1, 2).contiguous() for t in (q, k, v))
    else:
        q, k, v = (t.transpose(1, 2) for t in (q, k, v))
    causal = window == (-1, -1)
    out, lse, *_ = flag_gems.ops.flash_attention_forward(q, k, v, None, None, sq, sk, 0, causal, False, scale=0.11, softcap=softcap,
                                                         window_size_left=window[0], window_size_right=window[1])
    ref, rlse = O.dense_attention(q, k, v, 0.11, causal=causal, window_size=window, softcap=softcap, return_lse=True)
    torch.testing.assert_close(out.float().cpu(), ref, atol=2e-3, rtol=1.6e-2)
    torch.testing.assert_close(lse.cpu(), rlse, atol=1e-3, rtol=1e-4)


def test_flash_attention_forward_dispatch_and_sdpa(gpu):
    dtype = torch.bfloat16
    q, k, v = _dense_inputs(gpu, 2, 8, 8, 256, 256, 128, dtype)
    ref = O.dense_attention(q.transpose(1, 2), k.transpose(1, 2), v.transpose(1, 2), 128 ** -0.5, causal=True)
    # the ATen operator, overridden inside use_gems()
    with flag_gems.use_gems():
        out, lse, *_ = torch.ops.aten._flash_attention_forward(q.transpose(1, 2), k.transpose(1, 2), v.transpose(1, 2), None, None,
                                                               256, 256, 0.0, True, False, scale=128 ** -0.5)
    torch.testing.assert_close(out.float().cpu(), ref, atol=2e-3, rtol=1.6e-2)
    assert lse.shape == (2, 8, 256) and lse.dtype == torch.float32
    # scaled_dot_product_attention: (batch, heads, seq, d) in and out, with and without GQA
    o = flag_gems.scaled_dot_product_attention(q, k, v, is_causal=True)
    assert o.shape == q.shape
    torch.testing.assert_close(o.transpose(1, 2).float().cpu(), ref, atol=2e-3, rtol=1.6e-2)
    qg, kg, vg = _dense_inputs(gpu, 2, 8, 2, 100, 333, 64, torch.float16)
    o = flag_gems.scaled_dot_product_attention(qg, kg, vg, scale=0.2, enable_gqa=True)
    refg = O.dense_attention(qg.transpose(1, 2), kg.transpose(1, 2), vg.transpose(1, 2), 0.2)
    torch.testing.assert_close(o.transpose(1, 2).float().cpu(), refg, atol=2e-4, rtol=1e-3)
    # what the kernel does not cover goes to torch's own implementation: an attention mask, a gradient
    mask = torch.rand(2, 8, 256, 256, device=gpu) > 0.5
    o = flag_gems.scaled_dot_product_attention(q, k, v, attn_mask=mask)
    torch.testing.assert_close(o, torch.nn.functional.scaled_dot_product_attention(q, k, v, attn_mask=mask))
    qr = q.clone().requires_grad_()
    flag_gems.scaled_dot_product_attention(qr, k, v, is_causal=True).sum().backward()
    assert qr.grad is not None and torch.isfinite(qr.grad).all()
    with pytest.raises(AssertionError):
        flag_gems.scaled_dot_product_attention(qg, kg, vg)  # different head counts need enable_gqa


def test_flash_attn_varlen_out_argument_and_views(gpu):
    q, kc, vc, cu, sk, bt, qlens, klens = make_case(gpu, [(40, 90), (17, 17)], 8, 2, 128, 16, 128, torch.bfloat16)
    out = torch.full_like(q, 7.0)
    r = flag_gems.flash_attn_varlen_func(q, kc, vc, max(qlens), cu, max(klens), seqused_k=sk, causal=True, block_table=bt, out=out)
    assert r.data_ptr() == out.data_ptr()
    ref = O.paged_attention(q, kc, vc, qlens, klens, bt, 128 ** -0.5, compute_dtype=torch.float32)
    torch.testing.assert_close(out.float().cpu(), ref, atol=ATOL, rtol=RTOL)
    # K and V as the two halves of one [2, pages, page, H, D] allocation; max_seqlen as 0-d tensors
    kv = torch.stack([kc, vc])
    k2, v2 = kv.unbind(0)
    r2 = flag_gems.flash_attn_varlen_func(q, k2, v2, torch.tensor(max(qlens)), cu, torch.tensor(max(klens)), seqused_k=sk,
                                          causal=True, block_table=bt)
    assert torch.equal(r2, out)


def test_flash_attn_golden(gpu):
    bf16 = torch.bfloat16
    q = torch.from_numpy(GOLD["attn_q"]).to(bf16).to(gpu)
    kc = torch.from_numpy(GOLD["attn_kc"]).to(bf16).to(gpu); vc = torch.from_numpy(GOLD["attn_vc"]).to(bf16).to(gpu)
    bt = torch.from_numpy(GOLD["attn_bt"]).to(gpu)
    qlens, klens = GOLD["attn_qlens"].tolist(), GOLD["attn_klens"].tolist()
    cu = torch.tensor([0] + qlens, dtype=torch.int32, device=gpu).cumsum(0, dtype=torch.int32)
    sk = torch.tensor(klens, dtype=torch.int32, device=gpu)
    out, lse = flag_gems.flash_attn_varlen_func(q, kc, vc, max(qlens), cu, max(klens), seqused_k=sk, softmax_scale=0.25, causal=True,
                                                block_table=bt, return_softmax_lse=True)
    torch.testing.assert_close(out.double().cpu(), torch.from_numpy(GOLD["attn_out"]), atol=ATOL, rtol=RTOL)
    torch.testing.assert_close(lse.double().cpu(), torch.from_numpy(GOLD["attn_lse"]), atol=1e-2, rtol=1e-3)


def test_prefill_benchmark_shape_properties(gpu):
    """The benchmark's GQA prefill shape (32 q heads / 8 kv heads / D 128 / page 16) on its two shortest
    sequences plus one long one against the oracle, and a permutation property on the full batch: the
    result must not depend on where the pages live."""
    torch.manual_seed(0)
    L = torch.randint(512, 4097, (16,), generator=torch.Generator().manual_seed(0)).tolist()
    assert sum(L) == 35846
    Hq, Hk, D, bs = 32, 8, 128, 16
    def run(lens, perm_seed):
        tot = sum(lens)
        g = torch.Generator().manual_seed(7)
        q = torch.randn(tot, Hq, D, generator=g).bfloat16().to(gpu)
        k = torch.randn(tot, Hk, D, generator=g).bfloat16().to(gpu); v = torch.randn(tot, Hk, D, generator=g).bfloat16().to(gpu)
        nblk = sum((l + bs - 1) // bs for l in lens)
        perm = torch.randperm(nblk, generator=torch.Generator().manual_seed(perm_seed))
        kc = torch.zeros(nblk, bs, Hk, D, dtype=torch.bfloat16, device=gpu); vc = torch.zeros_like(kc)
        bt = torch.zeros(len(lens), (max(lens) + bs - 1) // bs, dtype=torch.int32)
        slots = []; o = 0
        for i, l in enumerate(lens):
            n = (l + bs - 1) // bs
            bt[i, :n] = perm[o:o + n]; o += n
            t = torch.arange(l)
            slots.append(bt[i, t // bs].long() * bs + t % bs)
        slots = torch.cat(slots).to(gpu); bt = bt.to(gpu)
        flag_gems.reshape_and_cache_flash(k, v, kc, vc, slots, "auto", None, None)
        cu = torch.tensor([0] + lens, dtype=torch.int32, device=gpu).cumsum(0, dtype=torch.int32)
        sk = torch.tensor(lens, dtype=torch.int32, device=gpu)
        out = flag_gems.flash_attn_varlen_func(q, kc, vc, max(lens), cu, max(lens), seqused_k=sk, causal=True, block_table=bt)
        return out, q, kc, vc, bt
    sub = [L[11], L[7], L[2]]  # 538, 615, 1405
    out, q, kc, vc, bt = run(sub, 1)
    ref = O.paged_attention(q, kc, vc, sub, sub, bt, D ** -0.5, compute_dtype=torch.float32)
    torch.testing.assert_close(out.float().cpu(), ref, atol=ATOL, rtol=RTOL)
    full1 = run(L, 1)[0]
    full2 = run(L, 2)[0]
    assert torch.equal(full1, full2)
    assert torch.isfinite(full1.float()).all()


def test_decoder_layer_pipeline(gpu):
    """Llama-2-7B-shaped layer (hidden 4096, 32 heads x 128, FFN 11008, page 16) under flag_gems.enable()
    semantics at 2 x 96 tokens: every operator of the path chained as in the benchmark, against the same
    layer evaluated on the host in fp32."""
    torch.manual_seed(0)
    Hd, H, D, F, bs = 4096, 32, 128, 11008, 16
    B, S = 2, 96
    T = B * S
    bf16 = torch.bfloat16
    wqkv = (torch.randn(3 * Hd, Hd) * 0.02).to(bf16).to(gpu); wo = (torch.randn(Hd, Hd) * 0.02).to(bf16).to(gpu)
    wgu = (torch.randn(2 * F, Hd) * 0.02).to(bf16).to(gpu); wd = (torch.randn(Hd, F) * 0.02).to(bf16).to(gpu)
    n1 = torch.ones(Hd, dtype=bf16, device=gpu); n2 = torch.ones(Hd, dtype=bf16, device=gpu)
    h = torch.randn(T, Hd).to(bf16).to(gpu)
    pos = torch.arange(S).repeat(B).to(gpu)
    cos, sin = O.rope_cos_sin(2048, D, device=gpu)
    nblk = B * (S // bs)
    perm = torch.randperm(nblk)
    bt = perm.view(B, S // bs).int().to(gpu)
    t = torch.arange(S)
    slots = torch.cat([bt[i].cpu()[t // bs].long() * bs + t % bs for i in range(B)]).to(gpu)
    kc = torch.zeros(nblk, bs, H, D, dtype=bf16, device=gpu); vc = torch.zeros_like(kc)
    cu = torch.tensor([0, S, 2 * S], dtype=torch.int32, device=gpu); sk = torch.tensor([S, S], dtype=torch.int32, device=gpu)
    with flag_gems.use_gems():
        x = torch.nn.functional.rms_norm(h, [Hd], n1, 1e-5)
        qkv = torch.mm(x, wqkv.t())
        q, k, v = (qkv[:, i * Hd:(i + 1) * Hd].view(T, H, D) for i in range(3))
        flag_gems.apply_rotary_pos_emb(q, k, cos, sin, pos, False, inplace=True)
        flag_gems.reshape_and_cache_flash(k, v, kc, vc, slots, "auto", None, None)
        attn = flag_gems.flash_attn_varlen_func(q, kc, vc, S, cu, S, seqused_k=sk, causal=True, block_table=bt)
        o = torch.mm(attn.view(T, Hd), wo.t())
        resid = h.clone()
        y, resid = flag_gems.fused_add_rms_norm(o, resid, [Hd], n2, 1e-5)
        gu = torch.mm(y, wgu.t())
        act = flag_gems.silu_and_mul(gu[:, :F], gu[:, F:])
        out = torch.mm(act, wd.t()) + resid
    # host reference in fp32 with the same bf16 roundings at operator boundaries
    def r(t_): return t_.to(bf16).float()
    hf = h.float().cpu()
    xr = r(O.rms_norm(hf, n1.float().cpu(), 1e-5))
    qkvr = r(xr @ wqkv.float().cpu().t())
    qr, kr, vr = (qkvr[:, i * Hd:(i + 1) * Hd].view(T, H, D) for i in range(3))
    qr, kr = O.apply_rotary_pos_emb(qr, kr, cos, sin, pos, False); qr, kr = r(qr), r(kr)
    kcr, vcr = O.reshape_and_cache_flash(kr.to(bf16), vr.to(bf16), torch.zeros_like(kc).cpu(), torch.zeros_like(vc).cpu(), slots)
    ar = r(O.paged_attention(qr, kcr.float(), vcr.float(), [S, S], [S, S], bt, D ** -0.5))
    orr = r(ar.view(T, Hd) @ wo.float().cpu().t())
    yr, rr = O.fused_add_rms_norm(orr, hf, n2.float().cpu(), 1e-5); yr, rr = r(yr), r(rr)
    gur = r(yr @ wgu.float().cpu().t())
    actr = r(O.silu_and_mul(gur[:, :F], gur[:, F:]))
    outr = r(actr @ wd.float().cpu().t()) + rr
    # (the last GEMM's bf16 result, up to ~8 with an ulp of 0.06, meets a residual of opposite sign: one ulp of it
    # can be the whole difference at an output near zero)
    torch.testing.assert_close(out.float().cpu(), outr, atol=0.1, rtol=5e-2)
    assert (out.float().cpu() - outr).abs().mean().item() < 0.02
    torch.testing.assert_close(kc.float().cpu(), kcr.float(), atol=2e-2, rtol=2e-2)
