"""CPU oracle for the floating-point operators of the path: PyTorch ATen on the host, restating the
expected-value computations of the reference's own accuracy tests.

TEST INFRASTRUCTURE ONLY.  Nothing in the product package may import this module; it is used by
tests/, by __graft_entry__.smoke() and by the cpu_baseline leg of bench.py, always as the checker
and never as the thing shipped or measured as the product.

Each function cites the reference test it follows (paths relative to the FlagGems tree).  The
reference holds no golden vectors for these operators (every expectation is computed live from
torch), so the pinning of this module is: (a) the torch library routines themselves for mm, addmm
and softmax, (b) closed forms and invariants checked in tests/test_oracle.py for the rest.
"""

import torch
import torch.nn.functional as F


def to_reference(t, upcast=False):
    """tests/accuracy_utils.py:175-186 with --ref cpu: move to the host, optionally widen to fp64."""
    if t is None:
        return None
    r = t.detach().to("cpu")
    if upcast and r.is_floating_point():
        r = r.to(torch.float64)
    return r


def mm(a, b):
    """tests/test_blas_ops.py:119-136: torch.mm on fp64 copies."""
    return torch.mm(to_reference(a, True), to_reference(b, True))


def addmm(bias, a, b, alpha=1, beta=1):
    """tests/test_blas_ops.py:24-60: torch.addmm on fp64 copies."""
    return torch.addmm(to_reference(bias, True), to_reference(a, True), to_reference(b, True), alpha=alpha, beta=beta)


def bmm(a, b):
    """tests/test_blas_ops.py:95-110: torch.bmm on fp64 copies."""
    return torch.bmm(to_reference(a, True), to_reference(b, True))


def softmax(x, dim):
    """tests/test_reduction_ops.py:507-523: F.softmax on an fp64 copy."""
    return F.softmax(to_reference(x, True), dim=dim)


def log_softmax(x, dim):
    """tests/test_reduction_ops.py:466-480: F.log_softmax on an fp64 copy."""
    return torch.nn.functional.log_softmax(to_reference(x, True), dim=dim)


def softmax_backward(grad, out, dim):
    """tests/test_reduction_ops.py:533-557: aten::_softmax_backward_data on fp64 copies
    (grad_in = out * (grad - sum(out * grad)))."""
    g, y = to_reference(grad, True), to_reference(out, True)
    return torch.ops.aten._softmax_backward_data(g, y, dim, g.dtype)


def log_softmax_backward(grad, out, dim):
    """tests/test_reduction_ops.py:487-503: aten::_log_softmax_backward_data on fp64 copies
    (grad_in = grad - exp(out) * sum(grad))."""
    g, y = to_reference(grad, True), to_reference(out, True)
    return torch.ops.aten._log_softmax_backward_data(g, y, dim, g.dtype)


def rms_norm_grads(x, weight, eps, grad):
    """tests/test_norm_ops.py:539-559: autograd through weight * (x * rsqrt(mean(x^2) + eps)), here on fp64
    copies.  Returns (dx, dweight)."""
    xr = to_reference(x, True).clone().requires_grad_(True)
    wr = to_reference(weight, True).clone().requires_grad_(True)
    y = wr * (xr * torch.rsqrt(xr.pow(2).mean(-1, keepdim=True) + eps))
    return torch.autograd.grad(y, (xr, wr), to_reference(grad, True))


def rms_norm(x, weight, eps):
    """tests/test_norm_ops.py:539-544: fp32 normalisation, cast to the input dtype, then the weight
    multiply (the test does not widen to fp64 for this operator)."""
    x = to_reference(x)
    weight = to_reference(weight)
    xf = x.to(torch.float32)
    var = xf.pow(2).mean(-1, keepdim=True)
    h = xf * torch.rsqrt(var + eps)
    return weight * h.to(x.dtype)


def fused_add_rms_norm(x, residual, weight, eps):
    """tests/test_norm_ops.py:614-618: fp64 sum, normalise, weight.  Returns (normed, new_residual)."""
    x = to_reference(x, True)
    r = to_reference(residual, True)
    w = to_reference(weight, True)
    s = x + r
    var = s.pow(2).mean(-1, keepdim=True)
    return s * torch.rsqrt(var + eps) * w, s


def rope_cos_sin(max_pos, dim, base=10000.0, dtype=torch.float32, device="cpu"):
    """tests/test_special_ops.py:106-112: inv_freq = base^(-2i/dim), cos/sin of the outer product."""
    inv_freq = 1.0 / (base ** (torch.arange(0, dim, 2, dtype=torch.float32, device=device) / dim))
    t = torch.arange(max_pos, dtype=torch.float32, device=device)
    freqs = torch.outer(t, inv_freq)
    return freqs.cos().to(dtype), freqs.sin().to(dtype)


def _rotate_half(x):
    h = x.shape[-1] // 2
    return torch.cat((-x[..., h:], x[..., :h]), dim=-1)


def _rotate_interleave(x):
    x1 = x[..., ::2]
    x2 = x[..., 1::2]
    return torch.stack((-x2, x1), dim=-1).flatten(-2)


def apply_rotary_pos_emb(q, k, cos, sin, position_ids=None, rotary_interleaved=False):
    """tests/test_special_ops.py:133-161: q, k in fp32, cos/sin widened to fp64 and expanded to the
    full head dim; q*cos + rotate(q)*sin.  Without position ids the position is the index along
    dim -3."""
    q = to_reference(q).float()
    k = to_reference(k).float()
    cos = to_reference(cos, True)
    sin = to_reference(sin, True)
    if position_ids is None:
        cos = cos[None, : q.size(-3), None, :]
        sin = sin[None, : q.size(-3), None, :]
    else:
        pid = to_reference(position_ids).long()
        cos = cos[pid].unsqueeze(-2)
        sin = sin[pid].unsqueeze(-2)
    if rotary_interleaved:
        cos = torch.repeat_interleave(cos, 2, dim=-1)
        sin = torch.repeat_interleave(sin, 2, dim=-1)
        rot = _rotate_interleave
    else:
        cos = torch.cat([cos, cos], dim=-1)
        sin = torch.cat([sin, sin], dim=-1)
        rot = _rotate_half
    return q * cos + rot(q) * sin, k * cos + rot(k) * sin


def silu_and_mul(a, b):
    """tests/test_binary_pointwise_ops.py:1377-1403: F.silu(a) * b on fp64 copies."""
    return F.silu(to_reference(a, True)) * to_reference(b, True)


def silu_and_mul_grads(a, b, grad):
    """tests/test_binary_pointwise_ops.py:1377-1403: autograd through F.silu(a) * b on fp64 copies.
    Returns (da, db)."""
    ar = to_reference(a, True).clone().requires_grad_(True)
    br = to_reference(b, True).clone().requires_grad_(True)
    return torch.autograd.grad(F.silu(ar) * br, (ar, br), to_reference(grad, True))


def alibi_bias(slopes, seqlen_q, seqlen_k, causal):
    """tests/test_attention_ops.py:804-816: slopes [batch, heads] -> bias broadcastable to
    [batch, heads, seqlen_q, seqlen_k]."""
    slopes = slopes.unsqueeze(-1).unsqueeze(-1)
    if causal:
        return torch.arange(-seqlen_k + 1, 1, dtype=torch.float32) * slopes
    row = torch.arange(seqlen_q, dtype=torch.long).unsqueeze(-1)
    col = torch.arange(seqlen_k, dtype=torch.long)
    rel = torch.abs(row + seqlen_k - seqlen_q - col)
    return -slopes * rel.to(slopes.dtype)


def paged_attention(query, key_cache, value_cache, query_lens, kv_lens, block_tables, scale, causal=True,
                    attn_bias=None, sliding_window=None, soft_cap=None, window=None, compute_dtype=None,
                    return_lse=False):
    """tests/test_attention_ops.py:819-881 (ref_paged_attn): per sequence, gather the pages named by
    the block table, scaled q . k^T per head (GQA by repeat_interleave), optional soft cap, causal
    mask triu(diagonal = kv_len - q_len + 1), optional sliding window, optional additive bias,
    softmax cast to v's dtype, weighted sum of v.

    Extensions used by this repo's tests: `causal=False`, a two-sided `window=(left, right)`,
    `compute_dtype` (run the arithmetic in a wider type than the inputs), and `return_lse`
    (log-sum-exp of the masked, biased logits: [heads, total_q])."""
    query = to_reference(query)
    key_cache = to_reference(key_cache)
    value_cache = to_reference(value_cache)
    block_tables = to_reference(block_tables).numpy()
    if compute_dtype is not None:
        query, key_cache, value_cache = (t.to(compute_dtype) for t in (query, key_cache, value_cache))
    _, block_size, num_kv_heads, head_size = key_cache.shape
    outputs, lses = [], []
    start = 0
    for i, (q_len, kv_len) in enumerate(zip(query_lens, kv_lens)):
        q = query[start : start + q_len].clone()
        q *= scale
        nblk = (kv_len + block_size - 1) // block_size
        idx = block_tables[i, :nblk]
        k = key_cache[idx].view(-1, num_kv_heads, head_size)[:kv_len]
        v = value_cache[idx].view(-1, num_kv_heads, head_size)[:kv_len]
        if q.shape[1] != k.shape[1]:
            k = torch.repeat_interleave(k, q.shape[1] // k.shape[1], dim=1)
            v = torch.repeat_interleave(v, q.shape[1] // v.shape[1], dim=1)
        attn = torch.einsum("qhd,khd->hqk", q, k)
        ones = torch.ones(q_len, kv_len)
        mask = torch.zeros(q_len, kv_len, dtype=torch.bool)
        if causal:
            mask |= torch.triu(ones, diagonal=kv_len - q_len + 1).bool()
        if sliding_window is not None:
            mask |= torch.triu(ones, diagonal=kv_len - (q_len + sliding_window) + 1).bool().logical_not()
        if window is not None:
            left, right = window
            if right >= 0 and not causal:
                mask |= torch.triu(ones, diagonal=kv_len - q_len + right + 1).bool()
            if left >= 0:
                mask |= torch.tril(ones, diagonal=kv_len - q_len - left - 1).bool()
        if soft_cap is not None:
            attn = soft_cap * torch.tanh(attn / soft_cap)
        attn.masked_fill_(mask, float("-inf"))
        if attn_bias is not None:
            attn = attn + attn_bias[i, :, :q_len, :kv_len].to(attn.dtype)
        lses.append(torch.logsumexp(attn.float(), dim=-1))
        probs = torch.softmax(attn, dim=-1).to(v.dtype)
        probs = torch.nan_to_num(probs, nan=0.0)  # rows with no visible key
        outputs.append(torch.einsum("hqk,khd->qhd", probs, v))
        start += q_len
    out = torch.cat(outputs, dim=0)
    if return_lse:
        return out, torch.cat(lses, dim=1)
    return out


def dense_attention(q, k, v, scale, causal=False, window_size=(-1, -1), softcap=0.0, return_lse=False):
    """tests/test_attention_ops.py:53-198 (construct_local_mask + attention_ref, the FlashAttention test
    reference): q (batch, seqlen_q, heads, d), k / v (batch, seqlen_k, heads_k, d); fp32 arithmetic; GQA
    by repeat_interleave; scores = scale * q . k^T, optional soft cap; keys col with
    col > row + seqlen_k - seqlen_q + right or col < row + seqlen_k - seqlen_q - left are masked
    (causal means right = 0: the mask is aligned to the bottom right corner); softmax; rows with no
    visible key give zeros.  `return_lse` adds the log-sum-exp of the masked scores, (batch, heads, seqlen_q)."""
    q, k, v = (to_reference(t).float() for t in (q, k, v))
    left, right = window_size
    if causal:
        right = 0
    seqlen_q, seqlen_k = q.shape[1], k.shape[1]
    g = q.shape[2] // k.shape[2]
    k = k.repeat_interleave(g, dim=2)
    v = v.repeat_interleave(g, dim=2)
    scores = torch.einsum("bthd,bshd->bhts", q * scale, k)
    if softcap > 0:
        scores = torch.tanh(scores / softcap) * softcap
    if left >= 0 or right >= 0:
        row = torch.arange(seqlen_q)[:, None]
        col = torch.arange(seqlen_k)[None, :]
        shift = seqlen_k - seqlen_q
        if left < 0:
            masked = col > row + shift + right
        else:
            hi = torch.minimum(row + shift + right, torch.tensor(seqlen_k)) if right >= 0 else torch.full_like(row, seqlen_k)
            masked = (col > hi) | (col < row + shift - left)
        scores = scores.masked_fill(masked, float("-inf"))
    lse = torch.logsumexp(scores, dim=-1)
    probs = torch.nan_to_num(torch.softmax(scores, dim=-1), nan=0.0)
    out = torch.einsum("bhts,bshd->bthd", probs, v)
    if return_lse:
        return out, lse
    return out


def reshape_and_cache_flash(key, value, key_cache, value_cache, slot_mapping):
    """tests/test_attention_ops.py:1459-1467: python loop scatter.  Returns updated clones."""
    key, value = to_reference(key), to_reference(value)
    kc, vc = to_reference(key_cache).clone(), to_reference(value_cache).clone()
    block_size = kc.shape[1]
    slots = to_reference(slot_mapping).tolist()
    for i, s in enumerate(slots):
        if s < 0:
            continue
        kc[s // block_size, s % block_size] = key[i]
        vc[s // block_size, s % block_size] = value[i]
    return kc, vc


def reshape_and_cache(key, value, key_cache, value_cache, slot_mapping):
    """tests/test_attention_ops.py:1304-1315: python loop scatter into key_cache
    [blocks, heads, head_size / x, block_size, x] and value_cache [blocks, heads, head_size, block_size].
    Returns updated clones."""
    key, value = to_reference(key), to_reference(value)
    kc, vc = to_reference(key_cache).clone(), to_reference(value_cache).clone()
    block_size = kc.shape[3]
    reshaped_key = key.reshape(key.shape[0], *kc[0, :, :, 0, :].shape)
    for i, s in enumerate(to_reference(slot_mapping).tolist()):
        if s < 0:
            continue
        kc[s // block_size, :, :, s % block_size, :] = reshaped_key[i]
        vc[s // block_size, :, :, s % block_size] = value[i]
    return kc, vc


def gems_tolerance(dtype, reduce_dim=1, atol=1e-4):
    """(atol, rtol) of src/flag_gems/testing/__init__.py:41-49."""
    rtol = {torch.float16: 1e-3, torch.bfloat16: 0.016, torch.float32: 1.3e-6, torch.float64: 1e-7}[dtype]
    return atol * reduce_dim, rtol


def decoder_layer(h, wqkv, wo, wgu, wd, n1, n2, positions, cos, sin, eps, heads, q_rows=None):
    """One Llama-style decoder layer over ONE causal sequence, evaluated on the host in fp32 from the operator
    oracles above, with every operator's result rounded to the input dtype where the device path stores a
    tensor (so that a comparison sees one rounding per operator, not an accumulation of them):
    rms_norm -> x.Wqkv^T -> rotary (neox) on q, k -> causal attention over the sequence's own keys ->
    .Wo^T -> fused_add_rms_norm with the layer input as residual -> .Wgu^T -> silu_and_mul -> .Wd^T -> + residual.
    The chain is the layer the benchmark configuration runs (hidden = heads * head_dim, MHA); it follows the
    reference's module layer, src/flag_gems/modules/{normalization,rotary_embedding,activation}.py, and the
    operator tests cited above for each step.  `q_rows` (a LongTensor of token indices) restricts everything
    behind the key/value projection to those query tokens; keys and values are always computed for the whole
    sequence.  Returns a dict of the intermediate tensors (fp32), restricted to q_rows where that applies."""
    dt = h.dtype
    rnd = lambda t: t.to(dt).float()
    h = to_reference(h)
    S, hidden = h.shape
    D = hidden // heads
    wqkv, wo, wgu, wd = (to_reference(w).float() for w in (wqkv, wo, wgu, wd))
    n1, n2 = to_reference(n1), to_reference(n2)
    cos, sin, positions = to_reference(cos), to_reference(sin), to_reference(positions)
    rows = torch.arange(S) if q_rows is None else to_reference(q_rows).long()
    x = rms_norm(h, n1, eps).float()                                   # [S, hidden], rounded by the oracle itself
    kv = rnd(x @ wqkv[hidden:].t())                                    # keys and values of every token
    k = kv[:, :hidden].view(S, heads, D)
    v = kv[:, hidden:].view(S, heads, D)
    q = rnd(x[rows] @ wqkv[:hidden].t()).view(len(rows), heads, D)
    q, _ = apply_rotary_pos_emb(q, q, cos, sin, positions[rows], False)
    k, _ = apply_rotary_pos_emb(k, k, cos, sin, positions, False)
    q, k = rnd(q), rnd(k)
    scale = D ** -0.5
    att = torch.empty(len(rows), heads, D)
    for i, r in enumerate(rows.tolist()):                              # causal: token r sees keys 0..r
        s = torch.einsum("hd,khd->hk", q[i] * scale, k[: r + 1])
        p = torch.softmax(s, dim=-1)
        att[i] = torch.einsum("hk,khd->hd", p, v[: r + 1])
    att = rnd(att)
    o = rnd(att.reshape(len(rows), hidden) @ wo.t())
    y, resid = fused_add_rms_norm(o, h[rows].float(), n2.float(), eps)
    y, resid = rnd(y), rnd(resid)
    gu = rnd(y @ wgu.t())
    F_ = wgu.shape[0] // 2
    act = rnd(silu_and_mul(gu[:, :F_], gu[:, F_:]))
    out = rnd(rnd(act @ wd.t()) + resid)
    return {"x": x, "k": k, "v": v, "q": q, "attn": att, "o": o, "y": y, "residual": resid, "gate_up": gu,
            "act": act, "out": out}
