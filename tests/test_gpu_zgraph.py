"""The operators of a decoding step captured in a HIP graph (what a serving engine does to shed launch
overhead) and replayed with new inputs: every replay must equal the eager result.  Covers the current-stream
plumbing, the cached stream-K workspace of the skinny GEMM and the split-KV scratch of single-token attention."""
import pytest
import torch

import flag_gems

pytestmark = pytest.mark.gpu


def _step(x, res, w_norm, w_qkv, w_gate_up, cos, sin, pos, kc, vc, slots, block_table, seqused, cu_q):
    tokens, hidden = x.shape
    h = x.clone()
    r = res.clone()
    flag_gems.fused_add_rms_norm(h, r, [hidden], w_norm, 1e-6)
    qkv = flag_gems.mm(h, w_qkv.t())  # skinny stream-K on the cached workspace
    q, k, v = qkv.view(tokens, 3, 4, 64).unbind(1)
    q, k = flag_gems.apply_rotary_pos_emb(q, k, cos, sin, pos)
    flag_gems.reshape_and_cache_flash(k, v, kc, vc, slots, "auto", None, None)
    att = flag_gems.flash_attn_varlen_func(q.contiguous(), kc, vc, 1, cu_q, 512, seqused_k=seqused, causal=True,
                                           block_table=block_table)
    gu = flag_gems.mm(att.reshape(tokens, 256), w_gate_up.t())
    act = flag_gems.silu_and_mul(gu[:, :512], gu[:, 512:])
    return flag_gems.softmax(act.float(), -1), r


def test_decode_step_in_hip_graph(gpu):
    torch.manual_seed(0)
    dt = torch.bfloat16
    tokens, hidden = 8, 256
    w_norm = (torch.rand(hidden, device=gpu) + 0.5).to(dt)
    w_qkv = (torch.randn(3 * 256, hidden, device=gpu) / 16).to(dt)
    w_gate_up = (torch.randn(1024, 256, device=gpu) / 16).to(dt)
    inv = 1.0 / (10000 ** (torch.arange(0, 64, 2, device=gpu).float() / 64))
    ang = torch.arange(1024, device=gpu).float()[:, None] * inv[None, :]
    cos, sin = ang.cos().to(dt), ang.sin().to(dt)
    num_blocks, bs = 512, 16
    kc = (torch.randn(num_blocks, bs, 4, 64, device=gpu) / 4).to(dt)
    vc = (torch.randn(num_blocks, bs, 4, 64, device=gpu) / 4).to(dt)
    block_table = torch.randperm(num_blocks, device=gpu)[: tokens * 32].view(tokens, 32).int()
    cu_q = torch.arange(tokens + 1, device=gpu, dtype=torch.int32)
    # static inputs of the graph
    x = torch.zeros(tokens, hidden, device=gpu, dtype=dt)
    res = torch.zeros_like(x)
    pos = torch.zeros(tokens, device=gpu, dtype=torch.long)
    seqused = torch.ones(tokens, device=gpu, dtype=torch.int32)
    slots = torch.zeros(tokens, device=gpu, dtype=torch.long)

    def fill(step):
        g = torch.Generator(device="cpu").manual_seed(step)
        x.copy_(torch.randn(tokens, hidden, generator=g).to(dt))
        res.copy_(torch.randn(tokens, hidden, generator=g).to(dt))
        lens = torch.randint(100, 500, (tokens,), generator=g)
        seqused.copy_(lens.int())
        pos.copy_(lens - 1)
        last = lens - 1
        slots.copy_(block_table.cpu()[torch.arange(tokens), last // bs].long() * bs + last % bs)

    args = (x, res, w_norm, w_qkv, w_gate_up, cos, sin, pos, kc, vc, slots, block_table, seqused, cu_q)
    fill(0)
    _step(*args)  # warm-up outside the capture: workspaces and function attributes exist afterwards
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        out_g, res_g = _step(*args)
    for step in range(1, 5):
        fill(step)
        kc_before, vc_before = kc.clone(), vc.clone()
        graph.replay()
        torch.cuda.synchronize()
        got, got_r = out_g.clone(), res_g.clone()
        kc_after, vc_after = kc.clone(), vc.clone()
        # the same step eagerly, from the same cache contents
        kc.copy_(kc_before); vc.copy_(vc_before)
        want, want_r = _step(*args)
        torch.cuda.synchronize()
        assert torch.equal(got, want), f"replay {step} differs from the eager step"
        assert torch.equal(got_r, want_r)
        assert torch.equal(kc_after, kc) and torch.equal(vc_after, vc)
