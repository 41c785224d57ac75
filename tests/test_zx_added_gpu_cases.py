"""GPU cases added after the last complete run of the GPU suite.  They collect behind the long-standing parity tests
(pytest takes files in alphabetical order) so that a problem in a case that has never run cannot hide, under `-x`, the
result of the ones that have; the tests of the entry point that allocates nothing still come last."""
import pytest
import torch

import flag_gems
from oracle import torch_ref as O
from helpers import gems_assert_close
from test_gpu_attention import ATOL, RTOL, make_case
from test_gpu_zgraph import _fresh_stream, _sk_inputs, _streamk_mm

pytestmark = pytest.mark.gpu


# The reference's single-token grid as it stands (tests/test_attention_ops.py:998-1085,
# test_flash_attn_varlen_func_swap_qg: every sequence has one query token, so the reference takes its "swap query
# groups and sequence" path, ops/flash_api.py:318-345): lengths [(1, 1328), (1, 18), (1, 463)], 8 query heads on 2 KV
# heads, head dim 128, pages of 32, 2048 pages, soft cap off and 10.0, both 16-bit types, causal, seed 1234567890.
@pytest.mark.parametrize("seq_lens", [[(1, 1328), (1, 18), (1, 463)]])
@pytest.mark.parametrize("num_heads", [(8, 2)])
@pytest.mark.parametrize("head_size", [128])
@pytest.mark.parametrize("block_size", [32])
@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("soft_cap", [None, 10.0])
@pytest.mark.parametrize("num_blocks", [2048])
def test_flash_attn_varlen_func_swap_qg(gpu, seq_lens, num_heads, head_size, block_size, dtype, soft_cap, num_blocks):
    q, kc, vc, cu, sk, bt, qlens, klens = make_case(gpu, seq_lens, num_heads[0], num_heads[1], head_size, block_size,
                                                    num_blocks, dtype)
    scale = head_size ** -0.5
    out = flag_gems.ops.flash_attn_varlen_func(
        q=q, k=kc, v=vc, cu_seqlens_q=cu, seqused_k=sk, max_seqlen_q=max(qlens), max_seqlen_k=max(klens),
        softmax_scale=scale, causal=True, window_size=(-1, -1), block_table=bt,
        softcap=soft_cap if soft_cap is not None else 0, fa_version=2,
    )
    assert out.shape == q.shape and out.dtype == dtype
    # the reference compares in the tensors' own dtype: its oracle rounds the probabilities to the value dtype
    ref = O.paged_attention(q, kc, vc, qlens, klens, bt, scale, causal=True, soft_cap=soft_cap)
    torch.testing.assert_close(out.cpu(), ref.to(dtype), atol=ATOL, rtol=RTOL)
    ref32 = O.paged_attention(q, kc, vc, qlens, klens, bt, scale, causal=True, soft_cap=soft_cap, compute_dtype=torch.float32)
    torch.testing.assert_close(out.float().cpu(), ref32, atol=ATOL, rtol=RTOL)


# The reference's own test of silu_and_mul differentiates it (tests/test_binary_pointwise_ops.py:1377-1403, shapes
# POINTWISE_SHAPES of tests/accuracy_utils.py:59-63 and the quick-mode shape, all float dtypes): output and both
# gradients against autograd through F.silu(a) * b on upcast copies.  Plus the halves of one gate-up tensor (views
# with a row stride) and broadcast operands.
@pytest.mark.parametrize("dtype", [torch.float16, torch.float32, torch.bfloat16])
@pytest.mark.parametrize("shape", [(), (1,), (2, 19, 7), (1024, 1024), (20, 320, 15), (16, 128, 64, 60), (16, 7, 57, 32, 29),
                                   "halves", "broadcast"], ids=lambda s: ("x".join(map(str, s)) or "scalar") if isinstance(s, tuple) else s)
def test_accuracy_silu_and_mul_with_gradients(gpu, shape, dtype):
    torch.manual_seed(0)
    if shape == "halves":
        gu = torch.randn(16, 22016, dtype=dtype, device=gpu, requires_grad=True)
        inputs, (a, b) = (gu,), (gu[:, :11008], gu[:, 11008:])
    elif shape == "broadcast":
        a = torch.randn(6, 1, 96, dtype=dtype, device=gpu, requires_grad=True)
        b = torch.randn(1, 5, 96, dtype=dtype, device=gpu, requires_grad=True)
        inputs = (a, b)
    else:
        a = torch.randn(shape, dtype=dtype, device=gpu, requires_grad=True)
        b = torch.randn(shape, dtype=dtype, device=gpu, requires_grad=True)
        inputs = (a, b)
    res = flag_gems.silu_and_mul(a, b)
    assert res.dtype == dtype and res.requires_grad
    out_grad = torch.randn_like(res)
    res_grads = torch.autograd.grad(res, inputs, out_grad)
    # the oracle: the same expression on fp64 CPU copies, differentiated by autograd
    ref_inputs = tuple(O.to_reference(t.detach(), True).requires_grad_(True) for t in inputs)
    ra, rb = (ref_inputs[0][:, :11008], ref_inputs[0][:, 11008:]) if shape == "halves" else ref_inputs
    ref = torch.nn.functional.silu(ra) * rb
    ref_grads = torch.autograd.grad(ref, ref_inputs, O.to_reference(out_grad, True))
    gems_assert_close(res.detach(), ref.detach(), dtype)
    for got, want in zip(res_grads, ref_grads):
        assert got.shape == want.shape and got.dtype == dtype
        if shape != "broadcast":
            gems_assert_close(got, want, dtype)
    if shape == "broadcast":
        # a broadcast operand's gradient is the sum, taken by torch in `dtype`, of 5 or 6 per-element gradients that
        # were each rounded to `dtype`: held to the reference's relative resolution of the sum of their magnitudes
        from flag_gems.testing import RESOLUTION

        ea, eb = torch.broadcast_tensors(*ref_inputs)
        da, db = O.silu_and_mul_grads(ea, eb, out_grad)
        for got, want, terms, axis in ((res_grads[0], ref_grads[0], da, 1), (res_grads[1], ref_grads[1], db, 0)):
            bound = RESOLUTION[dtype] * terms.abs().sum(axis, keepdim=True) + 1e-4
            assert ((got.cpu().double() - want).abs() <= 2 * bound).all()
    with torch.no_grad():
        assert not flag_gems.silu_and_mul(a, b).requires_grad


# A caller of the whole path: a Hugging Face Llama model (random weights, a configuration small enough for any machine)
# evaluated under flag_gems.use_gems(), as the reference's examples/model_llama_test.py does with downloaded weights.
# Its linear layers, softmax or attention, and bmm reach the library through the ATen overrides.  The oracle is the same
# model in fp32 on the CPU; the vendor's kernels in the model's dtype set the scale of an acceptable error.
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("attn", ["sdpa", "eager"])
def test_llama_model_under_use_gems(gpu, dtype, attn):
    transformers = pytest.importorskip("transformers")
    cfg = transformers.LlamaConfig(vocab_size=512, hidden_size=256, intermediate_size=704, num_hidden_layers=2,
                                   num_attention_heads=4, num_key_value_heads=2, max_position_embeddings=128,
                                   rms_norm_eps=1e-5, attn_implementation=attn)
    torch.manual_seed(0)
    model = transformers.LlamaForCausalLM(cfg).eval()
    ids = torch.randint(0, cfg.vocab_size, (2, 24))
    with torch.no_grad():
        want = model(ids).logits.float()
    model = model.to(dtype).to(gpu)
    with torch.no_grad():
        vendor = model(ids.to(gpu)).logits.float().cpu()
        with flag_gems.use_gems():
            got = model(ids.to(gpu)).logits
    assert got.dtype == dtype and got.shape == want.shape
    got = got.float().cpu()
    err_vendor = (vendor - want).abs().max().item()
    err_gems = (got - want).abs().max().item()
    assert err_gems <= 2.0 * err_vendor + 1e-2, (err_gems, err_vendor)
    agree = lambda t: (t.argmax(-1) == want.argmax(-1)).float().mean().item()
    assert agree(got) >= agree(vendor) - 0.05, (agree(got), agree(vendor))


def test_workspace_made_under_capture_then_used_eagerly(gpu):
    """The workspace of a stream is first made during a capture, so its clearing is only recorded; the next call on
    that stream is eager and comes before any replay.  It must not start from whatever the allocation held."""
    from flaggems_amd.ops import _gemm

    a1, w1 = _sk_inputs(gpu, 16, 1024, 4096, 5)
    a2, w2 = _sk_inputs(gpu, 384, 4096, 4096, 6)
    want1 = _streamk_mm(a1, w1.t())
    want2 = _streamk_mm(a2, w2.t())
    torch.cuda.synchronize()
    side = _fresh_stream(gpu)
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph, stream=side):
        got1 = _streamk_mm(a1, w1.t())
    entry = _gemm._workspaces[(gpu.index, side.cuda_stream)]
    assert entry[3] is False          # no clear of this buffer has run yet
    entry[0][:entry[2]].fill_(0xFF)   # what stale memory would look like to the ticket counters
    torch.cuda.synchronize()
    with torch.cuda.stream(side):
        eager = _streamk_mm(a2, w2.t())
    torch.cuda.synchronize()
    assert entry[3] is True
    assert torch.equal(eager, want2)
    for _ in range(2):
        got1.zero_()
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(got1, want1)
        with torch.cuda.stream(side):
            again = _streamk_mm(a2, w2.t())
        torch.cuda.synchronize()
        assert torch.equal(again, want2)
