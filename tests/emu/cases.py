"""Cases the interpreted device runs through the C-ABI: each builds seeded inputs with numpy, calls one entry point
and returns the arrays a checker needs (inputs and outputs).  No torch here: the process that runs these must not
have the real HIP runtime in its global symbol scope.  16-bit floats travel as bit patterns: bf16 as uint16, f16 as
numpy float16.
"""
import ctypes as C

import numpy as np

from device import BF16, F16, F32, E

DT = {"bf16": BF16, "f16": F16, "f32": F32}
ITEM = {"bf16": 2, "f16": 2, "f32": 4}


def bits(a, dtype):
    """fp32 array -> storage array of `dtype` (round to nearest even)."""
    a = np.asarray(a, np.float32)
    if dtype == "bf16":
        return E.bf16_round(a.ravel()).astype(np.uint16).reshape(a.shape)
    if dtype == "f16":
        with np.errstate(over="ignore"):
            return a.astype(np.float16)
    return a


def storage(dtype):
    return {"bf16": np.uint16, "f16": np.float16, "f32": np.float32}[dtype]


def P(x):
    return C.c_void_p(int(x))


def I64(x):
    return C.c_int64(int(x))


def I32(x):
    return C.c_int(int(x))


def F(x):
    return C.c_float(float(x))


class Strided:
    """A [rows, cols] matrix inside a wider allocation: row stride >= cols, the gap filled with a sentinel that a
    checker verifies untouched."""

    def __init__(self, dev, rows, cols, stride, dtype, data=None, name="buf"):
        self.rows, self.cols, self.stride, self.dtype = rows, cols, stride, dtype
        full = np.full((rows, stride), 0, dtype=storage(dtype))
        full.view(np.uint16 if ITEM[dtype] == 2 else np.uint32)[:] = 0x7B7B if ITEM[dtype] == 2 else 0x7B7B7B7B
        if data is not None:
            full[:, :cols] = data
        self.initial = full.copy()
        n = (rows - 1) * stride + cols if rows else 0       # the allocation ends with the last row's last element
        self.ptr = dev.upload(full.ravel()[:n], name) if n else dev.alloc(16, name)
        self.dev, self.n = dev, n

    def read(self):
        flat = np.zeros(self.rows * self.stride, dtype=storage(self.dtype))
        flat[:self.n] = self.dev.download(self.ptr, storage(self.dtype), (self.n,))
        full = flat.reshape(self.rows, self.stride)
        gap_ok = True
        if self.stride > self.cols and self.rows:
            a = full.view(np.uint16 if ITEM[self.dtype] == 2 else np.uint32)
            b = self.initial.view(a.dtype)
            gap = np.ones_like(a, dtype=bool)
            gap[:, :self.cols] = False
            gap.ravel()[self.n:] = False
            gap_ok = bool((a[gap] == b[gap]).all())
        return full[:, :self.cols].copy(), gap_ok


# ---------------------------------------------------------------------------------------------------------------
# row-wise operators
# ---------------------------------------------------------------------------------------------------------------
def rms_norm(dev, rng, dtype, M, N, weight=True, inv=True, xs=None, ys=None, eps=1e-5):
    xs, ys = xs or N, ys or N
    x = bits(rng.standard_normal((M, N)), dtype)
    w = bits(rng.standard_normal(N) * 0.5 + 1.0, dtype)
    X = Strided(dev, M, N, xs, dtype, x, "x")
    Y = Strided(dev, M, N, ys, dtype, None, "y")
    pw = dev.upload(w, "w") if weight else 0
    pi = dev.alloc(max(M, 1) * 4, "inv_rms") if inv else 0
    rc = dev.call("fg_rms_norm", P(X.ptr), P(pw), P(Y.ptr), P(pi), I64(M), I64(N), I64(xs), I64(ys), F(eps), I32(DT[dtype]), P(0))
    y, gap_ok = Y.read()
    out = {"rc": rc, "x": x, "w": w, "y": y, "gap_ok": gap_ok, "x_after": X.read()[0]}
    if inv:
        out["inv_rms"] = dev.download(pi, np.float32, (M,))
    return out


def fused_add_rms_norm(dev, rng, dtype, M, N, weight=True, xs=None, rs=None, eps=1e-5):
    xs, rs = xs or N, rs or N
    x = bits(rng.standard_normal((M, N)), dtype)
    r = bits(rng.standard_normal((M, N)), dtype)
    w = bits(rng.standard_normal(N) * 0.5 + 1.0, dtype)
    X = Strided(dev, M, N, xs, dtype, x, "x")
    R = Strided(dev, M, N, rs, dtype, r, "residual")
    pw = dev.upload(w, "w") if weight else 0
    rc = dev.call("fg_fused_add_rms_norm", P(X.ptr), P(R.ptr), P(pw), I64(M), I64(N), I64(xs), I64(rs), F(eps), I32(DT[dtype]), P(0))
    xo, g1 = X.read()
    ro, g2 = R.read()
    return {"rc": rc, "x": x, "residual": r, "w": w, "x_out": xo, "residual_out": ro, "gap_ok": g1 and g2}


def softmax(dev, rng, dtype, M, N, K, log=False, out_dtype=None, scale=3.0):
    out_dtype = out_dtype or dtype
    x = bits(rng.standard_normal((M, N, K)) * scale, dtype)
    px = dev.upload(x, "in")
    po = dev.alloc(max(M * N * K, 1) * ITEM[out_dtype], "out")
    rc = dev.call("fg_log_softmax" if log else "fg_softmax", P(px), P(po), I64(M), I64(N), I64(K), I32(DT[dtype]),
                  I32(DT[out_dtype]), P(0))
    return {"rc": rc, "x": x, "out": dev.download(po, storage(out_dtype), (M, N, K))}


def softmax_backward(dev, rng, dtype, M, N, K, log=False, grad_in_dtype=None):
    grad_in_dtype = grad_in_dtype or dtype
    z = rng.standard_normal((M, N, K)) * 2.0
    z = z - z.max(axis=1, keepdims=True)
    p = np.exp(z) / np.exp(z).sum(axis=1, keepdims=True)
    out = bits(np.log(p) if log else p, dtype)
    g = bits(rng.standard_normal((M, N, K)), dtype)
    po, pg = dev.upload(out, "out"), dev.upload(g, "grad_out")
    pi = dev.alloc(max(M * N * K, 1) * ITEM[grad_in_dtype], "grad_in")
    rc = dev.call("fg_log_softmax_backward" if log else "fg_softmax_backward", P(po), P(pg), P(pi), I64(M), I64(N), I64(K),
                  I32(DT[dtype]), I32(DT[grad_in_dtype]), P(0))
    return {"rc": rc, "out": out, "grad_out": g, "grad_in": dev.download(pi, storage(grad_in_dtype), (M, N, K))}


def rms_norm_backward(dev, rng, dtype, M, N, weight=True, dw=True, eps=1e-5):
    x = bits(rng.standard_normal((M, N)), dtype)
    dy = bits(rng.standard_normal((M, N)), dtype)
    w = bits(rng.standard_normal(N) * 0.5 + 1.0, dtype)
    xf = x.astype(np.float32) if dtype != "bf16" else (x.astype(np.uint32) << 16).view(np.float32)
    inv = (1.0 / np.sqrt((xf.astype(np.float64) ** 2).mean(axis=1) + eps)).astype(np.float32)
    px, pdy, pinv = dev.upload(x, "x"), dev.upload(dy, "dy"), dev.upload(inv, "inv_rms")
    pw = dev.upload(w, "w") if weight else 0
    pdx = dev.alloc(M * N * ITEM[dtype], "dx")
    dev.lib.fg_rms_norm_backward_partial_rows.restype = C.c_int64
    rows = int(dev.call("fg_rms_norm_backward_partial_rows", I64(M), I64(N), I32(DT[dtype]), I32(0))) if dw else 0
    ppart = dev.alloc(rows * N * 4 + 32, "dw_partial", fill=0x7B) if dw else 0
    rc = dev.call("fg_rms_norm_backward", P(px), P(pdy), P(pinv), P(pw), P(pdx), P(ppart), I64(rows), I64(M), I64(N),
                  I32(DT[dtype]), P(0))
    out = {"rc": rc, "x": x, "dy": dy, "w": w, "inv_rms": inv, "dx": dev.download(pdx, storage(dtype), (M, N)),
           "partial_rows": np.array(rows)}
    if dw and rc == 0:
        pdw = dev.alloc(N * ITEM[dtype], "dw")
        out["rc_dw"] = dev.call("fg_rms_norm_backward_dw", P(ppart), I64(rows), I64(N), P(pdw), I32(DT[dtype]), P(0))
        out["dw"] = dev.download(pdw, storage(dtype), (N,))
        out["dw_partial"] = dev.download(ppart, np.float32, (rows, N))
    return out


def transpose2d(dev, rng, elem_bytes, rows, cols, src_stride=None, dst_stride=None):
    src_stride, dst_stride = src_stride or cols, dst_stride or rows
    dtype = "bf16" if elem_bytes == 2 else "f32"
    data = rng.integers(0, 1 << 16, size=(rows, cols)).astype(np.uint16) if elem_bytes == 2 else \
        rng.standard_normal((rows, cols)).astype(np.float32)
    S = Strided(dev, rows, cols, src_stride, dtype, data, "src")
    D = Strided(dev, cols, rows, dst_stride, dtype, None, "dst")
    rc = dev.call("fg_transpose2d", P(S.ptr), P(D.ptr), I64(rows), I64(cols), I64(src_stride), I64(dst_stride), I32(elem_bytes), P(0))
    d, gap_ok = D.read()
    return {"rc": rc, "src": data, "dst": d, "gap_ok": gap_ok}


def silu_and_mul(dev, rng, dtype, rows, cols, a_stride=None, b_stride=None, o_stride=None):
    a_stride, b_stride, o_stride = a_stride or cols, b_stride or cols, o_stride or cols
    a = bits(rng.standard_normal((rows, cols)) * 2, dtype)
    b = bits(rng.standard_normal((rows, cols)), dtype)
    A, B = Strided(dev, rows, cols, a_stride, dtype, a, "a"), Strided(dev, rows, cols, b_stride, dtype, b, "b")
    O = Strided(dev, rows, cols, o_stride, dtype, None, "out")
    rc = dev.call("fg_silu_and_mul", P(A.ptr), P(B.ptr), P(O.ptr), I64(rows), I64(cols), I64(a_stride), I64(b_stride), I64(o_stride),
                  I32(DT[dtype]), P(0))
    o, gap_ok = O.read()
    return {"rc": rc, "a": a, "b": b, "out": o, "gap_ok": gap_ok}


def silu_and_mul_backward(dev, rng, dtype, rows, cols, a_stride=None, b_stride=None, g_stride=None, da_stride=None,
                          db_stride=None):
    a_stride, b_stride, g_stride = a_stride or cols, b_stride or cols, g_stride or cols
    da_stride, db_stride = da_stride or cols, db_stride or cols
    a = bits(rng.standard_normal((rows, cols)) * 2, dtype)
    b = bits(rng.standard_normal((rows, cols)), dtype)
    g = bits(rng.standard_normal((rows, cols)), dtype)
    A, B = Strided(dev, rows, cols, a_stride, dtype, a, "a"), Strided(dev, rows, cols, b_stride, dtype, b, "b")
    G = Strided(dev, rows, cols, g_stride, dtype, g, "g")
    DA, DB = Strided(dev, rows, cols, da_stride, dtype, None, "da"), Strided(dev, rows, cols, db_stride, dtype, None, "db")
    rc = dev.call("fg_silu_and_mul_backward", P(A.ptr), P(B.ptr), P(G.ptr), P(DA.ptr), P(DB.ptr), I64(rows), I64(cols),
                  I64(a_stride), I64(b_stride), I64(g_stride), I64(da_stride), I64(db_stride), I32(DT[dtype]), P(0))
    da, ok1 = DA.read()
    db, ok2 = DB.read()
    return {"rc": rc, "a": a, "b": b, "g": g, "da": da, "db": db, "gap_ok": ok1 and ok2}


def rope(dev, rng, dtype, n_tokens, Hq, Hk, D, interleaved=False, pos="i64", inplace=True, cs_dtype="f32", max_pos=64,
         seq_len=None, head_pad=0):
    """q [n_tokens, Hq, D] with `head_pad` unused elements behind every head (a slice of a wider projection)."""
    seq_len = seq_len or n_tokens
    hs = D + head_pad
    q = bits(rng.standard_normal((n_tokens, Hq, hs)), dtype)
    k = bits(rng.standard_normal((n_tokens, Hk, hs)), dtype)
    ang = rng.uniform(0, 6.28, size=(max_pos, D // 2))
    cos, sin = bits(np.cos(ang), cs_dtype), bits(np.sin(ang), cs_dtype)
    positions = rng.integers(0, max_pos, size=n_tokens)
    pq, pk = dev.upload(q, "q"), dev.upload(k, "k")
    pqo = pq if inplace else dev.alloc(q.nbytes, "q_out", fill=0x7B)
    pko = pk if inplace else dev.alloc(k.nbytes, "k_out", fill=0x7B)
    pc, ps = dev.upload(cos, "cos"), dev.upload(sin, "sin")
    ppos = 0
    if pos == "i64":
        ppos = dev.upload(positions.astype(np.int64), "pos")
    elif pos == "i32":
        ppos = dev.upload(positions.astype(np.int32), "pos")
    else:
        positions = np.arange(n_tokens) % seq_len
    arr = C.c_int64 * 3
    qs, ks = arr(Hq * hs, hs, 1), arr(Hk * hs, hs, 1)
    rc = dev.call("fg_rope", P(pqo), P(pko), P(pq), P(pk), P(pc), P(ps), P(ppos), I32(pos == "i64"), I64(n_tokens), I64(seq_len),
                  I32(Hq), I32(Hk), I32(D), qs, ks, qs, ks, I64(1), I64(D // 2), I64(D // 2), I64(max_pos), I32(interleaved),
                  I32(DT[dtype]), I32(DT[cs_dtype]), P(0))
    return {"rc": rc, "q": q, "k": k, "cos": cos, "sin": sin, "positions": positions.astype(np.int64),
            "q_out": dev.download(pqo, storage(dtype), q.shape), "k_out": dev.download(pko, storage(dtype), k.shape)}


def reshape_and_cache_flash(dev, rng, elem_bytes, num_tokens, H, D, block_size, num_blocks, slot_i64=True, token_pad=0,
                            block_pad=0):
    st = np.uint16 if elem_bytes == 2 else (np.uint8 if elem_bytes == 1 else np.uint32)
    ts = H * D + token_pad
    bs = block_size * H * D + block_pad
    key = rng.integers(0, 200, size=(num_tokens, ts)).astype(st)
    val = rng.integers(0, 200, size=(num_tokens, ts)).astype(st)
    slots = rng.permutation(num_blocks * block_size)[:num_tokens].astype(np.int64)
    if num_tokens > 2:
        slots[1] = -1
    kc = rng.integers(200, 250, size=(num_blocks, bs)).astype(st)
    vc = rng.integers(200, 250, size=(num_blocks, bs)).astype(st)
    pk, pv = dev.upload(key.ravel()[:(num_tokens - 1) * ts + H * D], "key"), dev.upload(val.ravel()[:(num_tokens - 1) * ts + H * D], "value")
    pkc, pvc = dev.upload(kc.ravel()[:(num_blocks - 1) * bs + block_size * H * D], "key_cache"), \
        dev.upload(vc.ravel()[:(num_blocks - 1) * bs + block_size * H * D], "value_cache")
    ps = dev.upload(slots if slot_i64 else slots.astype(np.int32), "slot_mapping")
    rc = dev.call("fg_reshape_and_cache_flash", P(pk), P(pv), P(pkc), P(pvc), P(ps), I32(slot_i64), I64(num_tokens), I32(H), I32(D),
                  I32(block_size), I64(ts), I64(ts), I64(bs), I32(elem_bytes), P(0))
    n = (num_blocks - 1) * bs + block_size * H * D
    kco, vco = kc.copy(), vc.copy()
    kco.ravel()[:n] = dev.download(pkc, st, (n,))
    vco.ravel()[:n] = dev.download(pvc, st, (n,))
    return {"rc": rc, "key": key, "value": val, "slots": slots, "key_cache_before": kc, "value_cache_before": vc,
            "key_cache": kco, "value_cache": vco, "dims": np.array([H, D, block_size, ts, bs])}


def reshape_and_cache(dev, rng, elem_bytes, num_tokens, H, D, block_size, x, num_blocks, slot_i64=True):
    st = np.uint16 if elem_bytes == 2 else np.uint32
    key = rng.integers(0, 200, size=(num_tokens, H, D)).astype(st)
    val = rng.integers(0, 200, size=(num_tokens, H, D)).astype(st)
    slots = rng.permutation(num_blocks * block_size)[:num_tokens].astype(np.int64)
    if num_tokens > 2:
        slots[1] = -1
        slots[2] = num_blocks * block_size + 3       # past the last block: skipped
    kc = rng.integers(200, 250, size=(num_blocks, H, D // x, block_size, x)).astype(st)
    vc = rng.integers(200, 250, size=(num_blocks, H, D, block_size)).astype(st)
    pk, pv, pkc, pvc = dev.upload(key, "key"), dev.upload(val, "value"), dev.upload(kc, "key_cache"), dev.upload(vc, "value_cache")
    ps = dev.upload(slots if slot_i64 else slots.astype(np.int32), "slot_mapping")
    rc = dev.call("fg_reshape_and_cache", P(pk), P(pv), P(pkc), P(pvc), P(ps), I32(slot_i64), I64(num_tokens), I32(H), I32(D),
                  I32(block_size), I32(x), I64(num_blocks), I64(H * D), I64(H * D), I32(elem_bytes), P(0))
    return {"rc": rc, "key": key, "value": val, "slots": slots, "key_cache_before": kc, "value_cache_before": vc,
            "key_cache": dev.download(pkc, st, kc.shape), "value_cache": dev.download(pvc, st, vc.shape)}


# ---------------------------------------------------------------------------------------------------------------
# GEMM
# ---------------------------------------------------------------------------------------------------------------
def gemm(dev, rng, dtype, M, N, K, b_layout="kn", bias=None, alpha=1.0, beta=1.0, schedule=0, c_dtype=None, entry="fg_gemm",
         a_pad=0):
    """b_layout "kn": B row-major [K, N]; "nk": B stored [N, K] (K-contiguous, the weight layout).
    bias: None, "row" ([N] broadcast over rows), "full" ([M, N])."""
    c_dtype = c_dtype or dtype
    a = bits(rng.standard_normal((M, K + a_pad)) * 0.5, dtype)
    b = bits(rng.standard_normal((K, N)) * 0.5, dtype)
    pa = dev.upload(a.ravel()[:(M - 1) * (K + a_pad) + K], "A")
    if b_layout == "kn":
        pb, sbk, sbn = dev.upload(b, "B"), N, 1
    else:
        pb, sbk, sbn = dev.upload(np.ascontiguousarray(b.T), "B"), 1, K
    pc = dev.alloc(M * N * ITEM[c_dtype], "C", fill=0x7B)
    pbias, sim, sin_ = 0, 0, 0
    bias_arr = np.zeros(0, np.float32)
    if bias == "row":
        bias_arr = bits(rng.standard_normal(N), dtype)
        pbias, sim, sin_ = dev.upload(bias_arr, "bias"), 0, 1
    elif bias == "full":
        bias_arr = bits(rng.standard_normal((M, N)), dtype)
        pbias, sim, sin_ = dev.upload(bias_arr, "bias"), N, 1
    used = C.c_int(-1)
    out = {}
    if entry == "fg_gemm":
        dev.lib.fg_gemm_workspace_bytes.restype = C.c_size_t
        need = int(dev.call("fg_gemm_workspace_bytes", I64(M), I64(N), I64(K), I32(DT[dtype]), I32(schedule), I32(0)))
        pws = dev.alloc(need + 256, "workspace") if need else 0
        rc = dev.call("fg_gemm", P(pa), P(pb), P(pbias), P(pc), I64(M), I64(N), I64(K), I64(K + a_pad), I64(1), I64(sbk), I64(sbn),
                      I64(sim), I64(sin_), I64(N), I64(1), F(alpha), F(beta), I32(DT[dtype]), I32(DT[c_dtype]), I32(DT[dtype]),
                      I32(schedule), P(pws), C.c_size_t(need), C.byref(used), P(0))
        out["workspace_bytes"] = np.array(need)
        if need:   # the header (ticket counters) must read zero again after the launch
            hdr = C.c_size_t(0)
            mx = C.c_size_t(0)
            dev.call("fg_gemm_workspace_layout", I32(0), C.byref(mx), C.byref(hdr))
            out["header_after"] = dev.download(pws, np.uint8, (min(int(hdr.value), need),))
    else:
        rc = dev.call("fg_gemm_skinny_static", P(pa), P(pb), P(pbias), P(pc), I64(M), I64(N), I64(K), I64(K + a_pad), I64(1),
                      I64(sbk), I64(sbn), I64(sim), I64(sin_), I64(N), I64(1), F(alpha), F(beta), I32(DT[dtype]), I32(DT[c_dtype]),
                      I32(DT[dtype]), P(0))
    out.update({"rc": rc, "a": a[:, :K].copy(), "b": b, "bias": bias_arr, "c": dev.download(pc, storage(c_dtype), (M, N)),
                "schedule_used": np.array(used.value)})
    return out


def bmm(dev, rng, dtype, batch, M, N, K):
    a = bits(rng.standard_normal((batch, M, K)) * 0.5, dtype)
    b = bits(rng.standard_normal((batch, K, N)) * 0.5, dtype)
    pa, pb = dev.upload(a, "A"), dev.upload(b, "B")
    pc = dev.alloc(batch * M * N * ITEM[dtype], "C", fill=0x7B)
    rc = dev.call("fg_bmm", P(pa), P(pb), P(pc), I64(batch), I64(M), I64(N), I64(K), I64(M * K), I64(K), I64(1), I64(K * N), I64(N),
                  I64(1), I64(M * N), I64(N), I64(1), I32(DT[dtype]), P(0))
    return {"rc": rc, "a": a, "b": b, "c": dev.download(pc, storage(dtype), (batch, M, N))}


# ---------------------------------------------------------------------------------------------------------------
# attention over a paged KV cache
# ---------------------------------------------------------------------------------------------------------------
class FgFlashParams(C.Structure):
    _fields_ = [("q", C.c_void_p), ("k_cache", C.c_void_p), ("v_cache", C.c_void_p), ("out", C.c_void_p), ("lse", C.c_void_p),
                ("cu_seqlens_q", C.c_void_p), ("seqused_k", C.c_void_p), ("block_table", C.c_void_p), ("alibi_slopes", C.c_void_p),
                ("q_row_stride", C.c_int64), ("q_head_stride", C.c_int64), ("o_row_stride", C.c_int64), ("o_head_stride", C.c_int64),
                ("k_page_stride", C.c_int64), ("k_row_stride", C.c_int64), ("k_head_stride", C.c_int64),
                ("v_page_stride", C.c_int64), ("v_row_stride", C.c_int64), ("v_head_stride", C.c_int64),
                ("block_table_stride", C.c_int64), ("alibi_batch_stride", C.c_int64), ("total_q", C.c_int64),
                ("batch", C.c_int32), ("Hq", C.c_int32), ("Hk", C.c_int32), ("D", C.c_int32), ("page_size", C.c_int32),
                ("max_seqlen_q", C.c_int32), ("max_seqlen_k", C.c_int32), ("is_causal", C.c_int32),
                ("window_left", C.c_int32), ("window_right", C.c_int32), ("softmax_scale", C.c_float), ("softcap", C.c_float),
                ("dtype", C.c_int32), ("workspace", C.c_void_p), ("workspace_bytes", C.c_int64)]


def attention(dev, rng, dtype, q_lens, k_lens, Hq, Hk, D, page_size, causal=True, window=(-1, -1), softcap=0.0, alibi=False,
              lse=True, workspace=True, spare_pages=2):
    """Sequences of q_lens[i] queries over k_lens[i] cached keys, pages handed out in a shuffled order."""
    batch = len(q_lens)
    total_q = int(sum(q_lens))
    pages_per = [(k + page_size - 1) // page_size for k in k_lens]
    num_pages = sum(pages_per) + spare_pages
    max_pages = max(pages_per)
    q = bits(rng.standard_normal((total_q, Hq, D)), dtype)
    kc = bits(rng.standard_normal((num_pages, page_size, Hk, D)), dtype)
    vc = bits(rng.standard_normal((num_pages, page_size, Hk, D)), dtype)
    order = rng.permutation(num_pages)
    table = np.zeros((batch, max_pages), dtype=np.int32)
    at = 0
    for i, n in enumerate(pages_per):
        table[i, :n] = order[at:at + n]
        at += n
    cu = np.concatenate([[0], np.cumsum(q_lens)]).astype(np.int32)
    used = np.asarray(k_lens, dtype=np.int32)
    slopes = (rng.uniform(0.05, 0.5, size=(batch, Hq))).astype(np.float32)
    p = FgFlashParams()
    p.q, p.k_cache, p.v_cache = dev.upload(q, "q"), dev.upload(kc, "k_cache"), dev.upload(vc, "v_cache")
    p.out = dev.alloc(q.nbytes, "out", fill=0x7B)
    p.lse = dev.alloc(Hq * total_q * 4, "lse", fill=0x7B) if lse else 0
    p.cu_seqlens_q, p.seqused_k, p.block_table = dev.upload(cu, "cu_seqlens_q"), dev.upload(used, "seqused_k"), dev.upload(table, "block_table")
    p.alibi_slopes = dev.upload(slopes, "alibi_slopes") if alibi else 0
    p.q_row_stride, p.q_head_stride, p.o_row_stride, p.o_head_stride = Hq * D, D, Hq * D, D
    p.k_page_stride = p.v_page_stride = page_size * Hk * D
    p.k_row_stride = p.v_row_stride = Hk * D
    p.k_head_stride = p.v_head_stride = D
    p.block_table_stride, p.alibi_batch_stride, p.total_q = max_pages, Hq if alibi else 0, total_q
    p.batch, p.Hq, p.Hk, p.D, p.page_size = batch, Hq, Hk, D, page_size
    p.max_seqlen_q, p.max_seqlen_k = int(max(q_lens)), int(max(k_lens))
    p.is_causal, p.window_left, p.window_right = int(causal), window[0], window[1]
    p.softmax_scale, p.softcap, p.dtype = float(D) ** -0.5, softcap, DT[dtype]
    dev.lib.fg_flash_attn_workspace_bytes.restype = C.c_size_t
    need = int(dev.call("fg_flash_attn_workspace_bytes", C.byref(p), I32(0))) if workspace else 0
    p.workspace = dev.alloc(need, "workspace", fill=0x7B) if need else 0
    p.workspace_bytes = need
    rc = dev.call("fg_flash_attn_varlen_fwd", C.byref(p), P(0))
    out = {"rc": rc, "q": q, "k_cache": kc, "v_cache": vc, "block_table": table, "q_lens": np.asarray(q_lens), "k_lens": np.asarray(k_lens),
           "out": dev.download(p.out, storage(dtype), q.shape), "slopes": slopes, "workspace_bytes": np.array(need)}
    if lse:
        out["lse"] = dev.download(p.lse, np.float32, (Hq, total_q))
    return out


# ---------------------------------------------------------------------------------------------------------------
# the interpreter's own guard: a call whose buffers are too small must be reported, not absorbed
# ---------------------------------------------------------------------------------------------------------------
def short_buffer(dev, rng, which):
    """fg_rms_norm on [4, 2048] bf16 with one operand allocated 16 bytes short; returns the interpreter's message."""
    M, N = 4, 2048
    x = bits(rng.standard_normal((M, N)), "bf16")
    w = bits(np.ones(N), "bf16")
    px = dev.upload(x.ravel()[:M * N - (8 if which == "x" else 0)], "x")
    pw = dev.upload(w[:N - (8 if which == "w" else 0)], "w")
    py = dev.alloc((M * N - (8 if which == "y" else 0)) * 2, "y")
    try:
        rc = dev.call("fg_rms_norm", P(px), P(pw), P(py), P(0), I64(M), I64(N), I64(N), I64(N), F(1e-5), I32(BF16), P(0))
        return {"rc": rc, "caught": np.array("")}
    except E.EmuError as exc:
        return {"rc": 0, "caught": np.array(str(exc).splitlines()[0])}


# ---------------------------------------------------------------------------------------------------------------
# full-size problems, a few workgroups of the launch each
# ---------------------------------------------------------------------------------------------------------------
def _only(dev, picks):
    """Run only the listed workgroups of every launch (linear ids, x fastest; negative ids count from the end)."""
    def choose(name, grid):
        total = grid[0] * grid[1] * grid[2]
        out = []
        for p in picks:
            i = p % total
            out.append((i % grid[0], (i // grid[0]) % grid[1], i // (grid[0] * grid[1])))
        return out
    dev.group_filter = choose


def _untouched(arr):
    """Elements still holding the 0x7B fill."""
    raw = arr.view(np.uint16 if arr.dtype.itemsize == 2 else np.uint32)
    return raw == (0x7B7B if arr.dtype.itemsize == 2 else 0x7B7B7B7B)


def gemm_sampled(dev, rng, dtype, M, N, K, groups, b_layout="nk", bias=None, alpha=1.0, beta=1.0):
    """fg_gemm at full size with only `groups` of its workgroups run; returns the rows of A, columns of B and the block
    of C those workgroups produced."""
    scale = 1.0 / np.sqrt(K)
    a = bits(rng.standard_normal((M, K), dtype=np.float32) * scale, dtype)
    b = bits(rng.standard_normal((K, N), dtype=np.float32) * scale, dtype)
    pa = dev.upload(a, "A")
    if b_layout == "kn":
        pb, sbk, sbn = dev.upload(b, "B"), N, 1
    else:
        pb, sbk, sbn = dev.upload(np.ascontiguousarray(b.T), "B"), 1, K
    pc = dev.alloc(M * N * ITEM[dtype], "C", fill=0x7B)
    pbias, sin_, bias_arr = 0, 0, np.zeros(N, np.float32)
    if bias == "row":
        bias_arr = bits(rng.standard_normal(N) * 0.02, dtype)
        pbias, sin_ = dev.upload(bias_arr, "bias"), 1
    dev.lib.fg_gemm_workspace_bytes.restype = C.c_size_t
    need = int(dev.call("fg_gemm_workspace_bytes", I64(M), I64(N), I64(K), I32(DT[dtype]), I32(0), I32(0)))
    pws = dev.alloc(need + 256, "workspace") if need else 0
    used = C.c_int(-1)
    _only(dev, groups)
    try:
        rc = dev.call("fg_gemm", P(pa), P(pb), P(pbias), P(pc), I64(M), I64(N), I64(K), I64(K), I64(1), I64(sbk), I64(sbn),
                      I64(0), I64(sin_), I64(N), I64(1), F(alpha), F(beta), I32(DT[dtype]), I32(DT[dtype]), I32(DT[dtype]),
                      I32(0), P(pws), C.c_size_t(need), C.byref(used), P(0))
    finally:
        dev.group_filter = None
    c = dev.download(pc, storage(dtype), (M, N))
    done = ~_untouched(c)
    rows, cols = np.nonzero(done.any(axis=1))[0], np.nonzero(done.any(axis=0))[0]
    return {"rc": rc, "a": a[rows], "b": b[:, cols], "bias": bias_arr[cols] if bias else np.zeros(0, np.float32),
            "c": c[np.ix_(rows, cols)], "done": done[np.ix_(rows, cols)], "rows": rows, "cols": cols,
            "schedule_used": np.array(used.value)}


def attention_sampled(dev, rng, dtype, q_len, k_len, Hq, Hk, D, page_size, groups):
    """One causal sequence at full length, only `groups` of the launch's workgroups run."""
    _only(dev, groups)
    try:
        out = attention(dev, rng, dtype, [q_len], [k_len], Hq, Hk, D, page_size, causal=True, lse=True)
    finally:
        dev.group_filter = None
    out["done"] = ~_untouched(out["out"])
    return out


def rows_sampled(dev, rng, op, dtype, M, N, groups, masked=0.0, K=1, eps=1e-6):
    """softmax / fused_add_rms_norm at full size, only `groups` of the workgroups run; returns the rows they wrote."""
    edge = min(64, M // 2)          # rows at either end of the matrix hold data, the rest (never read here) zeros

    def ends(make):
        full = np.zeros((M, N), dtype=storage(dtype))
        full[:edge], full[M - edge:] = make(), make()
        return full
    if op == "softmax":
        def scores():
            v = rng.standard_normal((edge, N), dtype=np.float32) * 2.0
            if masked:
                v[rng.random((edge, N)) < masked] = -np.inf
            return bits(v, dtype)
        xb = ends(scores)
        px = dev.upload(xb, "in")
        po = dev.alloc(M * N * ITEM[dtype], "out", fill=0x7B)
        _only(dev, groups)
        try:
            rc = dev.call("fg_softmax", P(px), P(po), I64(M), I64(N), I64(1), I32(DT[dtype]), I32(DT[dtype]), P(0))
        finally:
            dev.group_filter = None
        o = dev.download(po, storage(dtype), (M, N))
        rows = np.nonzero((~_untouched(o)).any(axis=1))[0]
        return {"rc": rc, "x": xb[rows].reshape(len(rows), N, 1), "out": o[rows].reshape(len(rows), N, 1), "rows": rows}
    xb = ends(lambda: bits(rng.standard_normal((edge, N), dtype=np.float32), dtype))
    rb = ends(lambda: bits(rng.standard_normal((edge, N), dtype=np.float32), dtype))
    w = bits(rng.uniform(0.5, 1.5, N), dtype)
    px, pr, pw = dev.upload(xb, "x"), dev.upload(rb, "residual"), dev.upload(w, "w")
    _only(dev, groups)
    try:
        rc = dev.call("fg_fused_add_rms_norm", P(px), P(pr), P(pw), I64(M), I64(N), I64(N), I64(N), F(eps), I32(DT[dtype]), P(0))
    finally:
        dev.group_filter = None
    xo, ro = dev.download(px, storage(dtype), (M, N)), dev.download(pr, storage(dtype), (M, N))
    rows = np.nonzero((xo.view(np.uint16 if ITEM[dtype] == 2 else np.uint32) != xb.view(np.uint16 if ITEM[dtype] == 2 else np.uint32)).any(axis=1))[0]
    return {"rc": rc, "x": xb[rows], "residual": rb[rows], "w": w, "x_out": xo[rows], "residual_out": ro[rows], "rows": rows,
            "gap_ok": np.array(True)}


def static_first_call_under_capture(dev, rng):
    """fg_gemm_skinny_static in a process that has made no call yet: refused while the stream is being captured (the
    lookup of the scratch array's address must not happen then), accepted eagerly, and from then on under capture too."""
    kw = dict(dtype="bf16", M=8, N=128, K=1024, b_layout="nk", entry="fg_gemm_skinny_static")
    out = {}
    dev.shim.shim_set_capturing(1)
    first = gemm(dev, rng, **kw)
    out["rc_first_under_capture"] = np.array(first["rc"])
    out["message"] = np.array(dev.last_error())
    out["launches_first"] = np.array(len(dev.launches))
    dev.shim.shim_set_capturing(0)
    eager = gemm(dev, rng, **kw)
    dev.shim.shim_set_capturing(1)
    again = gemm(dev, rng, **kw)
    dev.shim.shim_set_capturing(0)
    out["rc"] = np.array(eager["rc"] or again["rc"])
    for k in ("a", "b", "c"):
        out[k], out[k + "_captured"] = eager[k], again[k]
    out["bias"] = eager["bias"]
    out["schedule_used"] = eager["schedule_used"]
    return out


# ---------------------------------------------------------------------------------------------------------------
# operands of more than 4 GiB: offsets that no longer fit 32 bits.  The buffers are virtual (zero pages until touched);
# only the workgroups that work at the far end run.
# ---------------------------------------------------------------------------------------------------------------
def _poke(dev, ptr, byte_offset, array):
    raw = np.ascontiguousarray(array).view(np.uint8).ravel()
    dev.mem.view(ptr)[byte_offset:byte_offset + raw.size] = raw


def _peek(dev, ptr, byte_offset, dtype, shape):
    n = int(np.prod(shape)) * np.dtype(dtype).itemsize
    return dev.mem.view(ptr)[byte_offset:byte_offset + n].view(dtype).reshape(shape).copy()


def huge_cache_and_attention(dev, rng, dtype="bf16", num_pages=210000, page_size=16, Hq=8, Hk=8, D=128, k_len=300, q_len=1):
    """A paged cache of 6.4 GiB per tensor: tokens are scattered into its LAST pages by fg_reshape_and_cache_flash and
    attended from there by fg_flash_attn_varlen_fwd (page offsets beyond 4 GiB on both paths)."""
    page_elems = page_size * Hk * D
    cache_bytes = num_pages * page_elems * 2
    assert cache_bytes > 6 * 2 ** 30
    pk, pv = dev.alloc(cache_bytes, "k_cache"), dev.alloc(cache_bytes, "v_cache")
    pages = (k_len + page_size - 1) // page_size
    table = (num_pages - 1 - rng.permutation(pages * 2)[:pages]).astype(np.int32).reshape(1, pages)     # among the last pages
    key = bits(rng.standard_normal((k_len, Hk, D)), dtype)
    val = bits(rng.standard_normal((k_len, Hk, D)), dtype)
    slots = (table[0, np.arange(k_len) // page_size].astype(np.int64) * page_size + np.arange(k_len) % page_size)
    pkey, pval, pslots = dev.upload(key, "key"), dev.upload(val, "value"), dev.upload(slots, "slot_mapping")
    rc1 = dev.call("fg_reshape_and_cache_flash", P(pkey), P(pval), P(pk), P(pv), P(pslots), I32(1), I64(k_len), I32(Hk), I32(D),
                   I32(page_size), I64(Hk * D), I64(Hk * D), I64(page_elems), I32(2), P(0))
    # what landed in the pages of the table, gathered back in key order
    got_k = np.stack([_peek(dev, pk, int(s) * Hk * D * 2, np.uint16, (Hk, D)) for s in slots])
    got_v = np.stack([_peek(dev, pv, int(s) * Hk * D * 2, np.uint16, (Hk, D)) for s in slots])
    q = bits(rng.standard_normal((q_len, Hq, D)), dtype)
    p = FgFlashParams()
    p.q, p.k_cache, p.v_cache = dev.upload(q, "q"), pk, pv
    p.out = dev.alloc(q.nbytes, "out", fill=0x7B)
    p.lse = dev.alloc(Hq * q_len * 4, "lse", fill=0x7B)
    p.cu_seqlens_q = dev.upload(np.array([0, q_len], np.int32), "cu_seqlens_q")
    p.seqused_k = dev.upload(np.array([k_len], np.int32), "seqused_k")
    p.block_table = dev.upload(table, "block_table")
    p.q_row_stride, p.q_head_stride, p.o_row_stride, p.o_head_stride = Hq * D, D, Hq * D, D
    p.k_page_stride = p.v_page_stride = page_elems
    p.k_row_stride = p.v_row_stride = Hk * D
    p.k_head_stride = p.v_head_stride = D
    p.block_table_stride, p.total_q = pages, q_len
    p.batch, p.Hq, p.Hk, p.D, p.page_size = 1, Hq, Hk, D, page_size
    p.max_seqlen_q, p.max_seqlen_k, p.is_causal, p.window_left, p.window_right = q_len, k_len, 1, -1, -1
    p.softmax_scale, p.softcap, p.dtype = float(D) ** -0.5, 0.0, DT[dtype]
    rc2 = dev.call("fg_flash_attn_varlen_fwd", C.byref(p), P(0))
    # a dense two-page cache for the checker: page i of the sequence becomes page i
    dense_k = np.zeros((pages, page_size, Hk, D), np.uint16)
    dense_v = np.zeros((pages, page_size, Hk, D), np.uint16)
    dense_k.reshape(-1, Hk, D)[:k_len], dense_v.reshape(-1, Hk, D)[:k_len] = key, val
    return {"rc": rc1 or rc2, "key": key, "value": val, "got_k": got_k, "got_v": got_v, "q": q, "k_cache": dense_k, "v_cache": dense_v,
            "block_table": np.arange(pages, dtype=np.int32).reshape(1, pages), "q_lens": np.array([q_len]), "k_lens": np.array([k_len]),
            "out": dev.download(p.out, storage(dtype), q.shape), "lse": dev.download(p.lse, np.float32, (Hq, q_len)),
            "slopes": np.zeros((1, Hq), np.float32), "min_byte_offset": np.array(int(slots.min()) * Hk * D * 2)}


def huge_rows(dev, rng, op, dtype="bf16", M=1400000, N=2048):
    """A row-wise operator on a matrix of more than 4 GiB, the last workgroup only: its rows lie beyond 2^32 bytes and
    (for 16-bit types at this size) beyond 2^31 elements."""
    item = ITEM[dtype]
    assert M * N * item > 5 * 2 ** 30 and M * N > 2 ** 31
    edge = 8
    tail = (M - edge) * N * item
    x = bits(rng.standard_normal((edge, N)), dtype)
    px = dev.alloc(M * N * item, "x")
    _poke(dev, px, tail, x)
    out = {"x": x}
    _only(dev, [-1])
    try:
        if op == "softmax":
            po = dev.alloc(M * N * item, "out")
            out["rc"] = dev.call("fg_softmax", P(px), P(po), I64(M), I64(N), I64(1), I32(DT[dtype]), I32(DT[dtype]), P(0))
            out["out"] = _peek(dev, po, tail, storage(dtype), (edge, N))
        elif op == "fused_add_rms_norm":
            r = bits(rng.standard_normal((edge, N)), dtype)
            w = bits(rng.uniform(0.5, 1.5, N), dtype)
            pr, pw = dev.alloc(M * N * item, "residual"), dev.upload(w, "w")
            _poke(dev, pr, tail, r)
            out["rc"] = dev.call("fg_fused_add_rms_norm", P(px), P(pr), P(pw), I64(M), I64(N), I64(N), I64(N), F(1e-5), I32(DT[dtype]), P(0))
            out.update(residual=r, w=w, x_out=_peek(dev, px, tail, storage(dtype), (edge, N)),
                       residual_out=_peek(dev, pr, tail, storage(dtype), (edge, N)))
        elif op == "silu_and_mul":
            b = bits(rng.standard_normal((edge, N)), dtype)
            pb, po = dev.alloc(M * N * item, "b"), dev.alloc(M * N * item, "out")
            _poke(dev, pb, tail, b)
            out["rc"] = dev.call("fg_silu_and_mul", P(px), P(pb), P(po), I64(M), I64(N), I64(N), I64(N), I64(N), I32(DT[dtype]), P(0))
            out.update(b=b, out=_peek(dev, po, tail, storage(dtype), (edge, N)))
    finally:
        dev.group_filter = None
    return out


def huge_gemm(dev, rng, dtype="bf16", M=2500000, N=1024, K=1024, b_layout="nk"):
    """C = A.B with A [M, K] and C [M, N] of more than 4 GiB each: the last workgroup of the launch, whose rows of A and C
    start beyond 2^32 bytes."""
    item = ITEM[dtype]
    assert M * K * item > 4 * 2 ** 30 and M * N * item > 4 * 2 ** 30
    edge = 256
    a_tail = bits(rng.standard_normal((edge, K)) * 0.1, dtype)
    b = bits(rng.standard_normal((K, N)) * 0.1, dtype)
    pa = dev.alloc(M * K * item, "A")
    _poke(dev, pa, (M - edge) * K * item, a_tail)
    pb = dev.upload(np.ascontiguousarray(b.T) if b_layout == "nk" else b, "B")
    sbk, sbn = (1, K) if b_layout == "nk" else (N, 1)
    pc = dev.alloc(M * N * item, "C")
    used = C.c_int(-1)
    _only(dev, [-1])
    try:
        rc = dev.call("fg_gemm", P(pa), P(pb), P(0), P(pc), I64(M), I64(N), I64(K), I64(K), I64(1), I64(sbk), I64(sbn), I64(0), I64(0),
                      I64(N), I64(1), F(1.0), F(0.0), I32(DT[dtype]), I32(DT[dtype]), I32(DT[dtype]), I32(1), P(0), C.c_size_t(0),
                      C.byref(used), P(0))
    finally:
        dev.group_filter = None
    c_tail = _peek(dev, pc, (M - edge) * N * item, storage(dtype), (edge, N))
    done = c_tail.view(np.uint16) != 0
    rows, cols = np.nonzero(done.any(axis=1))[0], np.nonzero(done.any(axis=0))[0]
    return {"rc": rc, "a": a_tail[rows], "b": b[:, cols], "c": c_tail[np.ix_(rows, cols)], "done": done[np.ix_(rows, cols)],
            "bias": np.zeros(0, np.float32), "rows": rows, "cols": cols, "schedule_used": np.array(used.value)}


def huge_rope(dev, rng, dtype="bf16", n_tokens=600000, Hq=32, Hk=8, D=128, max_pos=64):
    """In-place rotation of q [n_tokens, Hq, D] of 4.9 GiB: the last workgroup, i.e. the last tokens."""
    item = ITEM[dtype]
    assert n_tokens * Hq * D * item > 4 * 2 ** 30
    edge = 4
    q = bits(rng.standard_normal((edge, Hq, D)), dtype)
    k = bits(rng.standard_normal((edge, Hk, D)), dtype)
    ang = rng.uniform(0, 6.28, size=(max_pos, D // 2))
    cos, sin = bits(np.cos(ang), "f32"), bits(np.sin(ang), "f32")
    positions = np.zeros(n_tokens, dtype=np.int64)
    positions[-edge:] = rng.integers(0, max_pos, size=edge)
    pq, pk = dev.alloc(n_tokens * Hq * D * item, "q"), dev.alloc(n_tokens * Hk * D * item, "k")
    q_tail, k_tail = (n_tokens - edge) * Hq * D * item, (n_tokens - edge) * Hk * D * item
    _poke(dev, pq, q_tail, q)
    _poke(dev, pk, k_tail, k)
    pc, ps, ppos = dev.upload(cos, "cos"), dev.upload(sin, "sin"), dev.upload(positions, "pos")
    arr = C.c_int64 * 3
    qs, ks = arr(Hq * D, D, 1), arr(Hk * D, D, 1)
    _only(dev, [-1])
    try:
        rc = dev.call("fg_rope", P(pq), P(pk), P(pq), P(pk), P(pc), P(ps), P(ppos), I32(1), I64(n_tokens), I64(n_tokens), I32(Hq), I32(Hk),
                      I32(D), qs, ks, qs, ks, I64(1), I64(D // 2), I64(D // 2), I64(max_pos), I32(0), I32(DT[dtype]), I32(F32), P(0))
    finally:
        dev.group_filter = None
    return {"rc": rc, "q": q, "k": k, "cos": cos, "sin": sin, "positions": positions[-edge:],
            "q_out": _peek(dev, pq, q_tail, storage(dtype), q.shape), "k_out": _peek(dev, pk, k_tail, storage(dtype), k.shape)}


def bmm_per_matrix(dev, rng, dtype="bf16", batch=32, M=2048, N=2048, K=128, matrices=(0, 31), groups=(0, 1, -1)):
    """The launches fg_bmm makes for a batch of `batch` matrices (one data-parallel fg_gemm per matrix on
    base + z * stride), for the listed matrices only and a few workgroups of each: the attention-sized batch that
    fg_bmm itself turns away."""
    item = ITEM[dtype]
    a = bits(rng.standard_normal((batch, M, K)) * 0.2, dtype)
    b = bits(rng.standard_normal((batch, K, N)) * 0.2, dtype)
    pa, pb = dev.upload(a, "A"), dev.upload(b, "B")
    pc = dev.alloc(batch * M * N * item, "C")
    rcs = []
    _only(dev, list(groups))
    try:
        for z in matrices:
            rcs.append(dev.call("fg_gemm", P(pa + z * M * K * item), P(pb + z * K * N * item), P(0), P(pc + z * M * N * item), I64(M),
                                I64(N), I64(K), I64(K), I64(1), I64(N), I64(1), I64(0), I64(0), I64(N), I64(1), F(1.0), F(0.0),
                                I32(DT[dtype]), I32(DT[dtype]), I32(DT[dtype]), I32(1), P(0), C.c_size_t(0), None, P(0)))
    finally:
        dev.group_filter = None
    out = {"rc": np.array(max(rcs, key=abs))}
    for z in matrices:
        c = _peek(dev, pc, z * M * N * item, storage(dtype), (M, N))
        done = c.view(np.uint16) != 0
        rows, cols = np.nonzero(done.any(axis=1))[0], np.nonzero(done.any(axis=0))[0]
        out.update({"a%d" % z: a[z][rows], "b%d" % z: b[z][:, cols], "c%d" % z: c[np.ix_(rows, cols)], "done%d" % z: done[np.ix_(rows, cols)]})
    # nothing outside the listed matrices was written
    others = [z for z in range(batch) if z not in matrices]
    out["others_untouched"] = np.array(all(not _peek(dev, pc, z * M * N * item, np.uint8, (4096,)).any() for z in others))
    return out
