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


def _fresh_stream(gpu):
    """A side stream that has no GEMM workspace yet (torch hands streams out of a small pool)."""
    from flaggems_amd.ops import _gemm

    for _ in range(64):
        s = torch.cuda.Stream()
        if (gpu.index, s.cuda_stream) not in _gemm._workspaces:
            return s
    raise AssertionError("no unused stream left in torch's pool")


def _streamk_mm(a, b):
    from flaggems_amd import _C
    from flaggems_amd.ops import _gemm

    out = torch.empty(a.shape[0], b.shape[1], dtype=a.dtype, device=a.device)
    _gemm.gemm(a, b, None, out, schedule=_C.SCHED_STREAM_K)
    assert _gemm.last_schedule() == 2
    return out


def _sk_inputs(gpu, M, N, K, seed):
    g = torch.Generator(device="cpu").manual_seed(seed)
    a = (torch.randn(M, K, generator=g) / 8).to(torch.bfloat16).to(gpu)
    w = (torch.randn(N, K, generator=g) / 8).to(torch.bfloat16).to(gpu)
    return a, w


def test_workspace_survives_a_larger_eager_gemm_after_capture(gpu):
    """A captured decode GEMM (skinny stream-K, small share of the workspace), then an eager stream-K tile GEMM on
    the same stream that needs far more of it, then replays: the graph's recorded workspace address must still be
    the live buffer, so the replays equal the eager results."""
    from flaggems_amd.ops import _gemm

    a, w = _sk_inputs(gpu, 8, 512, 4096, 1)
    big_a, big_w = _sk_inputs(gpu, 384, 4096, 4096, 2)
    want = _streamk_mm(a, w.t())
    side = _fresh_stream(gpu)
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph, stream=side):
        got = _streamk_mm(a, w.t())
    key = (gpu.index, side.cuda_stream)
    buf = _gemm._workspaces[key][0]
    with torch.cuda.stream(side):
        big = _streamk_mm(big_a, big_w.t())  # eager, same stream: 128x128 stream-K tiles
    torch.cuda.synchronize()
    assert _gemm._workspaces[key][0] is buf and buf.data_ptr() == _gemm._workspaces[key][0].data_ptr()
    for _ in range(3):
        got.zero_()
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(got, want)
        with torch.cuda.stream(side):
            again = _streamk_mm(big_a, big_w.t())
        torch.cuda.synchronize()
        assert torch.equal(again, big)
    from oracle import torch_ref as O
    from helpers import gems_assert_close
    gems_assert_close(big[:16], O.mm(big_a[:16], big_w.t()), torch.bfloat16, reduce_dim=4096)


def test_two_graphs_on_one_stream_replayed_out_of_order(gpu):
    """The workspace of a stream is first made during a capture (its clearing is only recorded there); a second
    graph captured on the same stream is replayed BEFORE the first ever ran.  Each graph clears the ticket header
    itself, so both produce the eager result in either order."""
    from flaggems_amd.ops import _gemm

    a1, w1 = _sk_inputs(gpu, 16, 1024, 4096, 3)
    a2, w2 = _sk_inputs(gpu, 4, 768, 8192, 4)
    want1 = _streamk_mm(a1, w1.t())
    want2 = _streamk_mm(a2, w2.t())
    torch.cuda.synchronize()
    side = _fresh_stream(gpu)
    g1, g2 = torch.cuda.CUDAGraph(), torch.cuda.CUDAGraph()
    with torch.cuda.graph(g1, stream=side):
        got1 = _streamk_mm(a1, w1.t())
    with torch.cuda.graph(g2, stream=side):
        got2 = _streamk_mm(a2, w2.t())
    # poison the header the way stale memory would: a replay that did not clear it would mis-count its tickets
    entry = _gemm._workspaces[(gpu.index, side.cuda_stream)]
    entry[0][:entry[2]].fill_(0xFF)
    torch.cuda.synchronize()
    for order in ((g2, g1), (g1, g2), (g2, g2, g1)):
        got1.zero_(); got2.zero_()
        for g in order:
            g.replay()
            torch.cuda.synchronize()
        assert torch.equal(got1, want1) and torch.equal(got2, want2)
