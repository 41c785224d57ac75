"""Pins the CPU oracle: closed forms, invariants, brute force on tiny inputs, the committed golden
fixtures, and agreement of the plain-C restatements with independent Python loops.  A plausible
mistake in the oracle (dropped term, wrong sign or index, transposed operand) fails one of these.
Runs on the CPU."""
import math
import os

import numpy as np
import pytest
import torch

from oracle import cref
from oracle import torch_ref as O

GOLD = np.load(os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "golden_v1.npz"))


def t(name, dtype=None):
    x = torch.from_numpy(GOLD[name])
    return x.to(dtype) if dtype is not None else x


# ---------------------------------------------------------------------------------------------
# golden fixtures: the oracle of today reproduces the committed numbers
# ---------------------------------------------------------------------------------------------
def test_oracle_reproduces_golden():
    bf16, f16 = torch.bfloat16, torch.float16
    for tag, dt in (("bf16", bf16), ("f16", f16)):
        x, r, w = t(f"rms_{tag}_x", dt), t(f"rms_{tag}_r", dt), t(f"rms_{tag}_w", dt)
        torch.testing.assert_close(O.rms_norm(x, w, 1e-5).double(), t(f"rms_{tag}_y"), atol=0, rtol=0)
        y, s = O.fused_add_rms_norm(x, r, w, 1e-5)
        torch.testing.assert_close(y, t(f"fused_{tag}_y"), atol=1e-12, rtol=1e-12)
        torch.testing.assert_close(s, t(f"fused_{tag}_res"), atol=0, rtol=0)
    torch.testing.assert_close(O.softmax(t("softmax_bf16_x", bf16), -1), t("softmax_bf16_y"), atol=1e-12, rtol=1e-12,
                               equal_nan=True)
    a, b, bias = t("mm_f16_a", f16), t("mm_f16_b", f16), t("mm_f16_bias", f16)
    torch.testing.assert_close(O.mm(a, b), t("mm_f16_c"), atol=1e-12, rtol=1e-12)
    torch.testing.assert_close(O.addmm(bias, a, b, alpha=-0.999, beta=100.001), t("addmm_f16_c"), atol=1e-10, rtol=1e-12)
    q, k = t("rope_q", bf16), t("rope_k", bf16)
    for inter in (False, True):
        oq, ok = O.apply_rotary_pos_emb(q, k, t("rope_cos"), t("rope_sin"), t("rope_pos"), inter)
        torch.testing.assert_close(oq, t(f"rope_oq_{int(inter)}"), atol=1e-12, rtol=1e-12)
        torch.testing.assert_close(ok, t(f"rope_ok_{int(inter)}"), atol=1e-12, rtol=1e-12)
    torch.testing.assert_close(O.silu_and_mul(t("silu_a", f16), t("silu_b", f16)), t("silu_y"), atol=1e-12, rtol=1e-12)
    out, lse = O.paged_attention(t("attn_q", bf16), t("attn_kc", bf16), t("attn_vc", bf16), GOLD["attn_qlens"].tolist(),
                                 GOLD["attn_klens"].tolist(), t("attn_bt"), 0.25, causal=True,
                                 compute_dtype=torch.float64, return_lse=True)
    torch.testing.assert_close(out, t("attn_out"), atol=1e-12, rtol=1e-12)
    torch.testing.assert_close(lse.double(), t("attn_lse"), atol=1e-5, rtol=1e-6)


# ---------------------------------------------------------------------------------------------
# norms
# ---------------------------------------------------------------------------------------------
def test_rms_norm_closed_form_and_loops():
    # constant row, unit weight: y = c / sqrt(c^2 + eps)
    for c in (0.5, -3.0):
        x = torch.full((2, 16), c)
        y = O.rms_norm(x, torch.ones(16), 1e-3)
        assert torch.allclose(y, torch.full((2, 16), c / math.sqrt(c * c + 1e-3)), atol=1e-6)
    # independent numpy loop
    rng = np.random.default_rng(0)
    x = rng.standard_normal((3, 7)).astype(np.float32)
    w = rng.standard_normal(7).astype(np.float32)
    ref = np.stack([row / np.sqrt((row.astype(np.float64) ** 2).sum() / 7 + 1e-5) * w for row in x])
    assert np.allclose(O.rms_norm(torch.from_numpy(x), torch.from_numpy(w), 1e-5).numpy(), ref, atol=1e-5)
    # weight scales the output linearly; scaling x by a large factor leaves y (almost) unchanged
    y1 = O.rms_norm(torch.from_numpy(x), torch.from_numpy(w), 0.0)
    y2 = O.rms_norm(torch.from_numpy(x * 8), torch.from_numpy(w), 0.0)
    assert torch.allclose(y1, y2, atol=1e-5)


def test_fused_add_rms_norm_both_outputs():
    rng = np.random.default_rng(1)
    x = rng.standard_normal((4, 9)); r = rng.standard_normal((4, 9)); w = rng.standard_normal(9)
    y, s = O.fused_add_rms_norm(torch.from_numpy(x), torch.from_numpy(r), torch.from_numpy(w), 1e-6)
    assert np.allclose(s.numpy(), x + r)
    for i in range(4):
        row = x[i] + r[i]
        assert np.allclose(y[i].numpy(), row / math.sqrt((row ** 2).mean() + 1e-6) * w)
    # residual = 0 reduces to rms_norm of x
    y0, _ = O.fused_add_rms_norm(torch.from_numpy(x), torch.zeros(4, 9, dtype=torch.float64), torch.from_numpy(w), 1e-6)
    assert torch.allclose(y0.float(), O.rms_norm(torch.from_numpy(x).float(), torch.from_numpy(w).float(), 1e-6), atol=1e-5)
    # the scalar C port agrees
    xf, rf, wf = x.astype(np.float32).copy(), r.astype(np.float32).copy(), w.astype(np.float32)
    cref.fused_add_rms_norm_f32(xf, rf, wf, 1e-6)
    assert np.allclose(rf, (x + r).astype(np.float32), atol=1e-6) and np.allclose(xf, y.numpy(), atol=1e-5)


# ---------------------------------------------------------------------------------------------
# softmax
# ---------------------------------------------------------------------------------------------
def test_log_softmax_pinned():
    """Closed forms and a scalar loop: log_softmax(x) = x - log(sum(exp(x))); uniform rows give -log(N)."""
    import math
    x = torch.tensor([[0.0, math.log(2.0), math.log(5.0)], [3.0, 3.0, 3.0]], dtype=torch.float32)
    y = O.log_softmax(x, -1)
    assert torch.allclose(y[0], torch.tensor([-math.log(8.0), math.log(2.0 / 8.0), math.log(5.0 / 8.0)], dtype=torch.float64))
    assert torch.allclose(y[1], torch.full((3,), -math.log(3.0), dtype=torch.float64))
    g = torch.Generator().manual_seed(3)
    z = torch.randn(4, 5, 6, generator=g)
    for dim in range(3):
        got = O.log_softmax(z, dim)
        zz = z.double().movedim(dim, -1).contiguous()
        rows = []
        for row in zz.reshape(-1, zz.shape[-1]):
            lse = math.log(sum(math.exp(float(v)) for v in row))
            rows.append([float(v) - lse for v in row])
        want = torch.tensor(rows, dtype=torch.float64).reshape(zz.shape)
        assert torch.allclose(got, want.movedim(-1, dim), atol=1e-12)
        assert torch.allclose(got.exp(), O.softmax(z, dim), atol=1e-12)
    w = torch.tensor([[1.0, float("-inf"), 2.0]])
    assert O.log_softmax(w, -1)[0, 1] == float("-inf")


def test_reshape_and_cache_v0_layout_pinned():
    """Element by element against the index formula of the layout: key element (head h, feature f) of the token
    in slot s sits at key_cache[s // bs, h, f // x, s % bs, f % x], value at value_cache[s // bs, h, f, s % bs]."""
    g = torch.Generator().manual_seed(21)
    T, H, D, bs, nb, x = 5, 3, 8, 4, 6, 4
    key = torch.randn(T, H, D, generator=g); value = torch.randn(T, H, D, generator=g)
    kc = torch.randn(nb, H, D // x, bs, x, generator=g); vc = torch.randn(nb, H, D, bs, generator=g)
    slots = torch.tensor([7, -1, 0, 23, 12])
    nk, nv = O.reshape_and_cache(key, value, kc, vc, slots)
    touched_k = torch.zeros_like(kc, dtype=torch.bool); touched_v = torch.zeros_like(vc, dtype=torch.bool)
    for t, s in enumerate(slots.tolist()):
        if s < 0:
            continue
        for h in range(H):
            for f in range(D):
                assert nk[s // bs, h, f // x, s % bs, f % x] == key[t, h, f]
                assert nv[s // bs, h, f, s % bs] == value[t, h, f]
                touched_k[s // bs, h, f // x, s % bs, f % x] = True
                touched_v[s // bs, h, f, s % bs] = True
    assert torch.equal(nk[~touched_k], kc[~touched_k]) and torch.equal(nv[~touched_v], vc[~touched_v])
    assert int(touched_k.sum()) == 4 * H * D
    # the same tokens through the flash layout land in the same (block, offset, head, feature) cells
    fk, fv = O.reshape_and_cache_flash(key, value, torch.zeros(nb, bs, H, D), torch.zeros(nb, bs, H, D), slots)
    zk, zv = O.reshape_and_cache(key, value, torch.zeros_like(kc), torch.zeros_like(vc), slots)
    assert torch.equal(zk.permute(0, 3, 1, 2, 4).reshape(nb, bs, H, D), fk)
    assert torch.equal(zv.permute(0, 3, 1, 2), fv)


def test_softmax_backward_pinned():
    """Against the Jacobian written out element by element, and against central differences of the forward."""
    import math
    g = torch.Generator().manual_seed(11)
    x = torch.randn(3, 5, generator=g, dtype=torch.float64)
    dy = torch.randn(3, 5, generator=g, dtype=torch.float64)
    y = torch.softmax(x, -1)
    got = O.softmax_backward(dy, y, 1)
    got_log = O.log_softmax_backward(dy, torch.log_softmax(x, -1), 1)
    for r in range(3):
        for i in range(5):
            # d softmax_j / d x_i = y_j (delta_ij - y_i);  d log_softmax_j / d x_i = delta_ij - y_i
            want = sum(float(dy[r, j]) * float(y[r, j]) * ((1.0 if i == j else 0.0) - float(y[r, i])) for j in range(5))
            want_log = sum(float(dy[r, j]) * ((1.0 if i == j else 0.0) - float(y[r, i])) for j in range(5))
            assert math.isclose(float(got[r, i]), want, abs_tol=1e-12)
            assert math.isclose(float(got_log[r, i]), want_log, abs_tol=1e-12)
    h = 1e-6
    for i in range(5):
        e = torch.zeros(3, 5, dtype=torch.float64); e[:, i] = h
        fd = ((torch.softmax(x + e, -1) - torch.softmax(x - e, -1)) * dy).sum(-1) / (2 * h)
        assert torch.allclose(got[:, i], fd, atol=1e-8)
    # a middle axis is the same rule applied along that axis
    y3 = torch.softmax(torch.randn(2, 4, 3, generator=g, dtype=torch.float64), 1)
    d3 = torch.randn(2, 4, 3, generator=g, dtype=torch.float64)
    assert torch.allclose(O.softmax_backward(d3, y3, 1), O.softmax_backward(d3.transpose(1, 2), y3.transpose(1, 2), 2).transpose(1, 2))
    # gradients of a softmax sum to zero along the axis
    assert torch.allclose(got.sum(-1), torch.zeros(3, dtype=torch.float64), atol=1e-12)


def test_rms_norm_grads_pinned():
    """Closed form dx = inv * (g - xh * mean(xh * g)), dw = sum over rows of dy * xh, and central differences."""
    g = torch.Generator().manual_seed(12)
    x = torch.randn(4, 6, generator=g, dtype=torch.float64)
    w = torch.randn(6, generator=g, dtype=torch.float64)
    dy = torch.randn(4, 6, generator=g, dtype=torch.float64)
    eps = 1e-5
    dx, dw = O.rms_norm_grads(x, w, eps, dy)
    inv = torch.rsqrt(x.pow(2).mean(-1, keepdim=True) + eps)
    xh, gg = x * inv, dy * w
    assert torch.allclose(dx, inv * (gg - xh * (xh * gg).mean(-1, keepdim=True)), atol=1e-12)
    assert torch.allclose(dw, (dy * xh).sum(0), atol=1e-12)

    def f(xx, ww):
        return float(((ww * (xx * torch.rsqrt(xx.pow(2).mean(-1, keepdim=True) + eps))) * dy).sum())

    h = 1e-6
    for (r, c) in ((0, 0), (2, 5), (3, 1)):
        e = torch.zeros_like(x); e[r, c] = h
        assert abs((f(x + e, w) - f(x - e, w)) / (2 * h) - float(dx[r, c])) < 1e-7
    for c in (0, 3):
        e = torch.zeros_like(w); e[c] = h
        assert abs((f(x, w + e) - f(x, w - e)) / (2 * h) - float(dw[c])) < 1e-7
    # the forward these gradients belong to is the oracle's forward
    assert torch.allclose(w * xh, O.rms_norm(x, w, eps).double(), atol=1e-12)


def test_softmax_invariants():
    x = torch.randn(6, 11, generator=torch.Generator().manual_seed(2))
    x[0, 3] = float("-inf"); x[2] = float("-inf")
    y = O.softmax(x, -1)
    assert torch.allclose(y[[0, 1, 3, 4, 5]].sum(-1), torch.ones(5, dtype=torch.float64))
    assert y[0, 3] == 0 and torch.isnan(y[2]).all()
    assert torch.allclose(O.softmax(x[1:2] + 5.0, -1), y[1:2])  # shift invariance
    # brute force
    row = x[4].double()
    e = torch.tensor([math.exp(v - float(row.max())) for v in row.tolist()], dtype=torch.float64)
    assert torch.allclose(y[4], e / e.sum())
    # a middle axis
    z = torch.randn(3, 5, 4)
    assert torch.allclose(O.softmax(z, 1).sum(1), torch.ones(3, 4, dtype=torch.float64))


# ---------------------------------------------------------------------------------------------
# mm / addmm (library routines: only the argument roles can go wrong)
# ---------------------------------------------------------------------------------------------
def test_mm_addmm_roles():
    a = torch.tensor([[1.0, 2.0], [3.0, 4.0], [5.0, 6.0]]); b = torch.tensor([[1.0, 0.0, 2.0, 0.0], [0.0, 1.0, 0.0, 3.0]])
    assert torch.equal(O.mm(a, b), torch.tensor([[1, 2, 2, 6], [3, 4, 6, 12], [5, 6, 10, 18]], dtype=torch.float64))
    bias = torch.tensor([10.0, 20.0, 30.0, 40.0])
    assert torch.equal(O.addmm(bias, a, b, alpha=2, beta=0.5), 2 * O.mm(a, b) + 0.5 * bias.double())
    assert torch.equal(O.addmm(bias, a, b, alpha=0, beta=1), bias.double().expand(3, 4))


def test_bmm_pinned():
    """Scalar triple loop per matrix; matrix b of the result depends on matrix b of the inputs only."""
    g = torch.Generator().manual_seed(5)
    a = torch.randn(3, 4, 5, generator=g); b = torch.randn(3, 5, 2, generator=g)
    got = O.bmm(a, b)
    assert got.dtype == torch.float64 and got.shape == (3, 4, 2)
    for z in range(3):
        for i in range(4):
            for j in range(2):
                want = sum(float(a[z, i, k]) * float(b[z, k, j]) for k in range(5))
                assert abs(float(got[z, i, j]) - want) < 1e-12
        assert torch.equal(got[z], O.mm(a[z], b[z]))
    # (A.B)^T = B^T.A^T per matrix; permuting the batch permutes the result
    assert torch.allclose(O.bmm(b.transpose(1, 2), a.transpose(1, 2)), got.transpose(1, 2), atol=1e-12)
    perm = torch.tensor([2, 0, 1])
    assert torch.equal(O.bmm(a[perm], b[perm]), got[perm])


# ---------------------------------------------------------------------------------------------
# rope
# ---------------------------------------------------------------------------------------------
@pytest.mark.parametrize("inter", [False, True])
def test_rope_brute_force_and_invariants(inter):
    g = torch.Generator().manual_seed(3)
    q = torch.randn(2, 4, 3, 8, generator=g); k = torch.randn(2, 4, 1, 8, generator=g)
    cos, sin = O.rope_cos_sin(16, 8)
    assert torch.allclose(cos[:, 0], torch.cos(torch.arange(16.0))) and torch.allclose(sin[3, 1], torch.sin(torch.tensor(3.0 / 10000 ** 0.25)))
    pos = torch.randint(0, 16, (2, 4), generator=g)
    oq, ok = O.apply_rotary_pos_emb(q, k, cos, sin, pos, inter)
    for b in range(2):
        for s in range(4):
            p = int(pos[b, s])
            for (x, o) in ((q, oq), (k, ok)):
                for h in range(x.shape[2]):
                    for j in range(4):
                        i0, i1 = (2 * j, 2 * j + 1) if inter else (j, j + 4)
                        c, sn = float(cos[p, j]), float(sin[p, j])
                        x0, x1 = float(x[b, s, h, i0]), float(x[b, s, h, i1])
                        assert abs(float(o[b, s, h, i0]) - (x0 * c - x1 * sn)) < 1e-6
                        assert abs(float(o[b, s, h, i1]) - (x1 * c + x0 * sn)) < 1e-6
    # position 0 is the identity; rotations preserve the norm of every pair, hence of the head
    o0, _ = O.apply_rotary_pos_emb(q, k, cos, sin, torch.zeros(2, 4, dtype=torch.long), inter)
    assert torch.allclose(o0, q.double())
    assert torch.allclose(oq.norm(dim=-1), q.double().norm(dim=-1))
    # without position ids the position is the index along dim -3
    o1, _ = O.apply_rotary_pos_emb(q, k, cos, sin, None, inter)
    o2, _ = O.apply_rotary_pos_emb(q, k, cos, sin, torch.arange(4).expand(2, 4), inter)
    assert torch.allclose(o1, o2)


def test_silu_and_mul_closed_form():
    a = torch.tensor([0.0, 1.0, -2.0, 30.0]); b = torch.tensor([3.0, 2.0, 0.5, 1.0])
    ref = torch.tensor([0.0, 2.0 / (1 + math.exp(-1.0)), -1.0 / (1 + math.exp(2.0)), 30.0 / (1 + math.exp(-30.0))], dtype=torch.float64)
    assert torch.allclose(O.silu_and_mul(a, b), ref)


def test_silu_and_mul_grads_pinned():
    """Closed form (d silu(x)/dx = s + x s (1 - s), s the logistic function) on hand-picked points, and central
    differences of the pinned forward on random ones."""
    a = torch.tensor([0.0, 1.0, -2.0, 30.0]); b = torch.tensor([3.0, 2.0, 0.5, 1.0]); g = torch.tensor([1.0, -2.0, 4.0, 0.5])
    da, db = O.silu_and_mul_grads(a, b, g)
    sig = [1 / (1 + math.exp(-v)) for v in a.tolist()]
    want_da = [gi * bi * (s + x * s * (1 - s)) for gi, bi, s, x in zip(g.tolist(), b.tolist(), sig, a.tolist())]
    want_db = [gi * x * s for gi, s, x in zip(g.tolist(), sig, a.tolist())]
    assert torch.allclose(da, torch.tensor(want_da, dtype=torch.float64), atol=1e-12)
    assert torch.allclose(db, torch.tensor(want_db, dtype=torch.float64), atol=1e-12)
    assert da[0] == 0.5 * 3.0 and db[0] == 0.0             # at 0: silu' = 1/2, silu = 0
    torch.manual_seed(3)
    a, b, g = torch.randn(5, 7, dtype=torch.float64), torch.randn(5, 7, dtype=torch.float64), torch.randn(5, 7, dtype=torch.float64)
    da, db = O.silu_and_mul_grads(a, b, g)
    h = 1e-6
    num_da = (O.silu_and_mul(a + h, b) - O.silu_and_mul(a - h, b)) / (2 * h) * g
    num_db = (O.silu_and_mul(a, b + h) - O.silu_and_mul(a, b - h)) / (2 * h) * g
    assert torch.allclose(da, num_da, atol=1e-8) and torch.allclose(db, num_db, atol=1e-8)


# ---------------------------------------------------------------------------------------------
# paged attention
# ---------------------------------------------------------------------------------------------
def brute_attention(q, kc, vc, qlens, klens, bt, scale, causal, window=None, softcap=None, slopes=None):
    """Scalar loops: the definition itself."""
    H, Hk = q.shape[1], kc.shape[2]
    bs = kc.shape[1]
    outs, lses = [], []
    start = 0
    for i, (ql, kl) in enumerate(zip(qlens, klens)):
        o = torch.zeros(ql, H, q.shape[2], dtype=torch.float64)
        l = torch.zeros(H, ql, dtype=torch.float64)
        for r in range(ql):
            for h in range(H):
                kh = h // (H // Hk)
                logits = []
                for c in range(kl):
                    page = int(bt[i, c // bs])
                    kv = kc[page, c % bs, kh].double()
                    s = float((q[start + r, h].double() * kv).sum()) * scale
                    if softcap:
                        s = softcap * math.tanh(s / softcap)
                    rel = r + kl - ql
                    masked = (causal and c > rel)
                    if window is not None:
                        left, right = window
                        if left >= 0 and c < rel - left:
                            masked = True
                        if right >= 0 and not causal and c > rel + right:
                            masked = True
                    if slopes is not None:
                        s += float(slopes[i, h]) * ((c - kl + 1) if causal else -abs(rel - c))
                    logits.append(-math.inf if masked else s)
                m = max(logits) if logits else -math.inf
                if m == -math.inf:
                    l[h, r] = math.inf  # marks "no visible key"
                    continue
                w = [math.exp(v - m) for v in logits]
                z = sum(w)
                l[h, r] = m + math.log(z)
                for c in range(kl):
                    page = int(bt[i, c // bs])
                    o[r, h] += (w[c] / z) * vc[page, c % bs, kh].double()
        outs.append(o); lses.append(l)
        start += ql
    return torch.cat(outs), torch.cat(lses, dim=1)


def _tiny_attn(seed=4):
    g = torch.Generator().manual_seed(seed)
    qlens, klens = [1, 3, 6, 2], [7, 3, 4, 9]   # includes q_len > k_len (rows without any visible key)
    q = torch.randn(sum(qlens), 4, 8, generator=g)
    kc, vc = torch.randn(6, 4, 2, 8, generator=g), torch.randn(6, 4, 2, 8, generator=g)
    bt = torch.randint(0, 6, (4, 3), generator=g, dtype=torch.int32)
    return q, kc, vc, qlens, klens, bt


@pytest.mark.parametrize("causal,window,softcap,alibi", [
    (True, None, None, False), (False, None, None, False), (True, (2, 0), None, False),
    (False, (1, 2), None, False), (True, None, 5.0, False), (True, None, None, True), (False, None, None, True),
])
def test_paged_attention_vs_brute_force(causal, window, softcap, alibi):
    q, kc, vc, qlens, klens, bt = _tiny_attn()
    slopes = torch.tensor([[0.5, 0.25, 0.125, 0.0625]] * 4) if alibi else None
    bias = None
    if alibi:
        bias = torch.zeros(4, 4, max(qlens), max(klens))
        for i, (ql, kl) in enumerate(zip(qlens, klens)):
            bias[i, :, :ql, :kl] = O.alibi_bias(slopes[i:i + 1], ql, kl, causal)[0]
    ref, rlse = brute_attention(q, kc, vc, qlens, klens, bt, 0.3, causal, window, softcap, slopes)
    out, lse = O.paged_attention(q, kc, vc, qlens, klens, bt, 0.3, causal=causal, window=window, soft_cap=softcap,
                                 attn_bias=bias, compute_dtype=torch.float64, return_lse=True)
    assert torch.allclose(out, ref, atol=1e-9)
    fin = torch.isfinite(rlse)
    assert torch.allclose(lse.double()[fin], rlse[fin], atol=1e-5)
    assert (lse[~fin] == -math.inf).all()  # logsumexp of an empty row; the kernel reports +inf there


def test_paged_attention_special_cases():
    q, kc, vc, qlens, klens, bt = _tiny_attn(5)
    # one key: the output is that key's value row, whatever the scores
    out = O.paged_attention(q[:1], kc, vc, [1], [1], bt[:1], 1.0, causal=True, compute_dtype=torch.float64)
    for h in range(4):
        assert torch.allclose(out[0, h], vc[int(bt[0, 0]), 0, h // 2].double())
    # zero queries: uniform weights, the output is the mean of the visible values
    out = O.paged_attention(torch.zeros(1, 4, 8), kc, vc, [1], [7], bt[:1], 1.0, causal=True, compute_dtype=torch.float64)
    vals = torch.stack([vc[int(bt[0, c // 4]), c % 4] for c in range(7)]).double()
    assert torch.allclose(out[0, 0], vals[:, 0].mean(0)) and torch.allclose(out[0, 3], vals[:, 1].mean(0))
    # the sliding_window argument of the reference equals window=(w - 1, 0) under causal
    o1 = O.paged_attention(q, kc, vc, qlens, klens, bt, 0.3, causal=True, sliding_window=3, compute_dtype=torch.float64)
    o2 = O.paged_attention(q, kc, vc, qlens, klens, bt, 0.3, causal=True, window=(2, 0), compute_dtype=torch.float64)
    assert torch.allclose(o1, o2)


@pytest.mark.parametrize("causal,window,softcap", [
    (False, (-1, -1), 0.0), (True, (-1, -1), 0.0), (True, (2, 0), 0.0), (False, (1, 2), 0.0), (True, (-1, -1), 5.0),
    (False, (3, -1), 0.0),
])
@pytest.mark.parametrize("sq,sk", [(5, 8), (8, 8), (7, 4)])
def test_dense_attention_vs_brute_force(causal, window, softcap, sq, sk):
    """The dense oracle against the scalar loops above, by presenting the batch as a paged cache (page = 4 rows)."""
    g = torch.Generator().manual_seed(sq * 10 + sk)
    B, H, Hk, D, bs = 2, 4, 2, 8, 4
    q = torch.randn(B, sq, H, D, generator=g); k = torch.randn(B, sk, Hk, D, generator=g); v = torch.randn(B, sk, Hk, D, generator=g)
    pages = (sk + bs - 1) // bs
    kc = torch.zeros(B * pages, bs, Hk, D); vc = torch.zeros_like(kc)
    for b in range(B):
        for r in range(sk):
            kc[b * pages + r // bs, r % bs] = k[b, r]; vc[b * pages + r // bs, r % bs] = v[b, r]
    bt = torch.arange(B * pages, dtype=torch.int32).reshape(B, pages)
    win = None if window == (-1, -1) else window
    ref, rlse = brute_attention(q.reshape(B * sq, H, D), kc, vc, [sq] * B, [sk] * B, bt, 0.3, causal, win, softcap or None, None)
    out, lse = O.dense_attention(q, k, v, 0.3, causal=causal, window_size=window, softcap=softcap, return_lse=True)
    assert torch.allclose(out.double().reshape(B * sq, H, D), ref, atol=1e-5)
    lse_flat = lse.permute(1, 0, 2).reshape(H, B * sq).double()
    fin = torch.isfinite(rlse)
    assert torch.allclose(lse_flat[fin], rlse[fin], atol=1e-4)
    assert (lse_flat[~fin] == -math.inf).all()


def test_dense_attention_special_cases():
    g = torch.Generator().manual_seed(9)
    q = torch.randn(1, 3, 2, 8, generator=g); k = torch.randn(1, 5, 2, 8, generator=g); v = torch.randn(1, 5, 2, 8, generator=g)
    # one key: the output is that key's value row
    out = O.dense_attention(q, k[:, :1], v[:, :1], 1.0)
    assert torch.allclose(out, v[:, :1].expand(1, 3, 2, 8))
    # zero queries: uniform weights, the mean of the visible values (causal, bottom-right: row r sees keys 0..r+2)
    out = O.dense_attention(torch.zeros_like(q), k, v, 1.0, causal=True)
    for r in range(3):
        assert torch.allclose(out[0, r], v[0, : r + 3].mean(0), atol=1e-6)
    # softmax is shift-invariant: adding a constant vector to every key direction of q . k changes nothing
    out1 = O.dense_attention(q, k, v, 0.7)
    out2 = O.dense_attention(q, k, v, 0.7, window_size=(100, 100))  # a window wider than the sequence masks nothing
    assert torch.allclose(out1, out2)


# ---------------------------------------------------------------------------------------------
# byte / integer work: the C restatements
# ---------------------------------------------------------------------------------------------
def test_cache_scatter_c_vs_python_loop():
    rng = np.random.default_rng(6)
    for dtype, D, bs in ((np.float32, 5, 4), (np.uint16, 8, 2), (np.uint8, 3, 7)):
        nt, H, nb = 9, 2, 6
        packed = rng.integers(0, 250, size=(nt, 3, H, D)).astype(dtype)       # key/value are strided views
        key, val = packed[:, 1], packed[:, 2]
        kc = rng.integers(0, 250, size=(nb, bs, H, D)).astype(dtype); vc = kc[::-1].copy()
        slots = rng.permutation(nb * bs)[:nt].astype(np.int64); slots[4] = -1
        ek, ev = kc.copy(), vc.copy()
        for i, s in enumerate(slots):
            if s >= 0:
                ek[s // bs, s % bs] = key[i]; ev[s // bs, s % bs] = val[i]
        stride = 3 * H * D
        cref.reshape_and_cache_flash(packed.reshape(-1)[H * D:], packed.reshape(-1)[2 * H * D:], kc, vc, slots, stride, stride, bs * H * D)
        assert np.array_equal(kc, ek) and np.array_equal(vc, ev)
        # the torch loop of the reference's test agrees
        tk, tv = O.reshape_and_cache_flash(torch.from_numpy(key.astype(np.float32)), torch.from_numpy(val.astype(np.float32)),
                                           torch.from_numpy(ek.astype(np.float32)), torch.from_numpy(ev.astype(np.float32)),
                                           torch.from_numpy(slots))
        assert np.array_equal(tk.numpy(), ek.astype(np.float32))
    g = np.load(os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "golden_v1.npz"))
    kc, vc = g["cache_kc0"].copy(), g["cache_vc0"].copy()
    cref.reshape_and_cache_flash(g["cache_key"].reshape(-1), g["cache_val"].reshape(-1), kc, vc, g["cache_slots"], 16, 16, 64)
    assert np.array_equal(kc, g["cache_kc1"]) and np.array_equal(vc, g["cache_vc1"])
    assert np.array_equal(kc[1, 3], g["cache_key"][0]) and np.array_equal(kc[0, 0], g["cache_key"][1])  # slots 7 and 0


def test_virtual_to_cache():
    table = np.array([5, 0, 9, 2], dtype=np.int32)
    for virt in range(16 * 4):
        assert cref.virtual_to_cache(virt, table, 16, 1024) == (int(table[virt // 16]) * 16 + virt % 16) * 1024


def test_streamk_partition_rule_and_abi_agreement():
    import ctypes
    from flaggems_amd import _C

    # closed form: 32 tiles of 112 iterations over 256 programs -> 32 cooperative tiles, 14 iterations each
    coop, b, e = cref.streamk_partition(32, 112, 256)
    assert coop == 32 and (e - b == 14).all() and b[0] == 0 and e[-1] == 32 * 112
    for tiles, iters, workers in [(1, 1, 4), (5, 3, 4), (7, 10, 3), (300, 8, 256), (470, 4, 256), (256, 5, 256), (3, 7, 8), (100, 1, 7)]:
        coop, b, e = cref.streamk_partition(tiles, iters, workers)
        rem = tiles % workers
        expect = rem
        if tiles - rem > 0 and rem < workers * 0.5:
            expect = rem + workers
        elif tiles - rem > 0 and rem > workers * 0.8:
            expect = 0
        assert coop == expect
        # every (tile, iteration) unit of the cooperative tiles is covered exactly once, in order
        cover = np.zeros(coop * iters, dtype=np.int64)
        for w in range(workers):
            cover[b[w]:e[w]] += 1
            assert 0 <= e[w] - b[w] - (coop * iters) // workers <= 1
            if w:
                assert b[w] == e[w - 1]
        assert (cover == 1).all()
        # the product's host function gives the same split
        sk = ctypes.c_int64()
        pb = (ctypes.c_int64 * workers)(); pe = (ctypes.c_int64 * workers)()
        assert _C.lib().fg_streamk_partition(tiles, iters, workers, ctypes.byref(sk), pb, pe) == 0
        assert sk.value == coop and list(pb) == b.tolist() and list(pe) == e.tolist()


def test_decoder_layer_pinned():
    """The layer oracle against an independent composition of library routines (F.rms_norm,
    F.scaled_dot_product_attention, F.silu, the textbook rotation written with complex numbers) in fp32, where
    the oracle's per-operator rounding is the identity; and its q_rows restriction against the full result."""
    import torch.nn.functional as F

    torch.manual_seed(0)
    S, heads, D, Fd = 11, 4, 16, 40
    hid = heads * D
    h = torch.randn(S, hid)
    wqkv, wo = torch.randn(3 * hid, hid) / 8, torch.randn(hid, hid) / 8
    wgu, wd = torch.randn(2 * Fd, hid) / 8, torch.randn(hid, Fd) / 8
    n1, n2 = torch.rand(hid) + 0.5, torch.rand(hid) + 0.5
    pos = torch.arange(3, 3 + S)
    cos, sin = O.rope_cos_sin(64, D)
    got = O.decoder_layer(h, wqkv, wo, wgu, wd, n1, n2, pos, cos, sin, 1e-5, heads)

    def rope(t):  # pairs (i, i + D/2) rotated by pos * base^(-2i/D): complex multiplication
        ang = pos[:, None].double() * (1.0 / 10000 ** (torch.arange(0, D, 2).double() / D))[None, :]
        z = torch.complex(t[..., : D // 2].double(), t[..., D // 2:].double()) * torch.polar(torch.ones_like(ang), ang)[:, None, :]
        return torch.cat([z.real, z.imag], -1).float()

    x = F.rms_norm(h, [hid], n1, 1e-5)
    qkv = x @ wqkv.t()
    q, k, v = (qkv[:, i * hid:(i + 1) * hid].view(S, heads, D) for i in range(3))
    q, k = rope(q), rope(k)
    att = F.scaled_dot_product_attention(q.transpose(0, 1)[None], k.transpose(0, 1)[None], v.transpose(0, 1)[None],
                                         is_causal=True)[0].transpose(0, 1).reshape(S, hid)
    r = att @ wo.t() + h
    y = F.rms_norm(r, [hid], n2, 1e-5)
    gu = y @ wgu.t()
    want = (F.silu(gu[:, :Fd]) * gu[:, Fd:]) @ wd.t() + r
    torch.testing.assert_close(got["out"], want, atol=2e-4, rtol=2e-4)
    torch.testing.assert_close(got["k"], k, atol=1e-5, rtol=1e-5)
    torch.testing.assert_close(got["attn"].reshape(S, hid), att, atol=1e-5, rtol=1e-4)
    rows = torch.tensor([0, 4, 10])
    part = O.decoder_layer(h, wqkv, wo, wgu, wd, n1, n2, pos, cos, sin, 1e-5, heads, q_rows=rows)
    for name in ("q", "attn", "o", "y", "residual", "gate_up", "act", "out"):
        torch.testing.assert_close(part[name], got[name][rows], atol=1e-6, rtol=1e-6)
