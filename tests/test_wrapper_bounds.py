"""What the Python wrappers hand over the C ABI stays inside memory the caller owns.

A kernel trusts its arguments: a stride taken from the wrong tensor, a row count from before a reshape or a pointer to
a temporary that has already been freed reads or writes outside an allocation, which on a GPU ends in a memory fault.
These tests run the operator wrappers on CPU tensors with a stand-in for the native library that launches nothing and
records every call.  `Tensor.data_ptr` is wrapped for the duration, so every pointer that reaches the C ABI is known
together with the storage it points into; for each recorded call the footprint that the header's contract
(include/fg_mi355.h) gives the pointer's operand, from the sizes and element strides passed with it, must lie inside
that storage, and index operands (slot mapping, sequence bounds, block table) must only name rows and pages that exist.
No GPU, no kernel: the native side of the same contract is covered by the GPU parity tests.
"""
import ctypes

import pytest
import torch

import flag_gems
from flaggems_amd import _C

ESIZE = {_C.FG_F16: 2, _C.FG_BF16: 2, _C.FG_F32: 4}


class Recorder:
    """Stand-in for the loaded library: records (name, args), answers the few queries with fixed device facts."""

    def __init__(self):
        self.calls = []

    def __getattr__(self, name):
        def call(*args):
            self.calls.append((name, args))
            if name == "fg_last_error":
                return b""
            if name in ("fg_gemm_workspace_bytes", "fg_flash_attn_workspace_bytes"):
                return 0
            if name == "fg_rms_norm_backward_partial_rows":
                return min(args[0], 8)
            if name == "fg_device_info":
                for ref, value in zip(args[1:], (256, 163840, 0x950)):
                    if ref is not None:
                        ref._obj.value = value
            if name == "fg_stream_capture_id":
                args[1]._obj.value = 0
            return 0

        return call


class Harness:
    def __init__(self, monkeypatch):
        self.rec = Recorder()
        self.ranges = {}      # data_ptr value -> (storage begin, storage end), the widest seen
        self.keep = []        # tensors whose pointer was taken stay alive until the checks have run
        real = torch.Tensor.data_ptr
        harness = self

        def data_ptr(t):
            p = real(t)
            st = t.untyped_storage()
            harness.keep.append(t)
            harness.ranges[p] = (st.data_ptr(), st.data_ptr() + st.nbytes())
            return p

        monkeypatch.setattr(torch.Tensor, "data_ptr", data_ptr)
        monkeypatch.setattr(torch.Tensor, "is_cuda", property(lambda t: True))
        monkeypatch.setattr(_C, "lib", lambda: self.rec)
        monkeypatch.setattr(_C, "current_stream", lambda device: 0)
        monkeypatch.setattr(_C, "device_guard", lambda device: _C._NO_GUARD)
        monkeypatch.setattr(_C, "_dev_info", {})
        from flaggems_amd.ops import _gemm

        monkeypatch.setattr(_gemm, "_workspaces", {})
        monkeypatch.setattr(_gemm, "_layouts", {})

    # ---- footprint arithmetic --------------------------------------------------------------------------------
    def inside(self, what, ptr, esize, dims, offset=0):
        """Operand at `ptr` (+ `offset` elements): dims = [(count, stride in elements), ...]; every element must lie
        inside the storage the pointer was taken from."""
        if ptr is None or ptr == 0:
            return
        ptr = int(ptr.value) if hasattr(ptr, "value") else int(ptr)
        assert ptr in self.ranges, "%s: pointer %#x did not come from a tensor's data_ptr()" % (what, ptr)
        if any(c <= 0 for c, _ in dims):
            return
        lo = offset + sum((c - 1) * s for c, s in dims if s < 0)
        hi = offset + sum((c - 1) * s for c, s in dims if s > 0)
        begin, end = self.ranges[ptr]
        assert begin <= ptr + lo * esize, "%s: reaches %d bytes below its storage" % (what, begin - (ptr + lo * esize))
        assert ptr + (hi + 1) * esize <= end, "%s: reaches %d bytes past its storage (dims %s)" % (
            what, ptr + (hi + 1) * esize - end, dims)

    @staticmethod
    def read(ptr, ctype, n):
        ptr = int(ptr.value) if hasattr(ptr, "value") else int(ptr)
        return list((ctype * n).from_address(ptr)) if n > 0 else []

    # ---- one checker per entry point -------------------------------------------------------------------------
    def check_all(self):
        names = []
        for name, a in self.rec.calls:
            fn = getattr(self, "chk_" + name, None)
            if fn is not None:
                fn(*a)
                names.append(name)
        return names

    def chk_fg_rms_norm(self, x, w, y, inv_rms, M, N, xs, ys, eps, dtype, stream):
        e = ESIZE[dtype]
        self.inside("rms_norm x", x, e, [(M, xs), (N, 1)])
        self.inside("rms_norm w", w, e, [(N, 1)])
        self.inside("rms_norm y", y, e, [(M, ys), (N, 1)])
        self.inside("rms_norm inv_rms", inv_rms, 4, [(M, 1)])

    def chk_fg_fused_add_rms_norm(self, x, res, w, M, N, xs, rs, eps, dtype, stream):
        e = ESIZE[dtype]
        self.inside("fused x", x, e, [(M, xs), (N, 1)])
        self.inside("fused residual", res, e, [(M, rs), (N, 1)])
        self.inside("fused w", w, e, [(N, 1)])

    def chk_fg_softmax(self, inp, out, M, N, K, in_dt, out_dt, stream):
        self.inside("softmax in", inp, ESIZE[in_dt], [(M * N * K, 1)])
        self.inside("softmax out", out, ESIZE[out_dt], [(M * N * K, 1)])

    chk_fg_log_softmax = chk_fg_softmax

    def chk_fg_softmax_backward(self, out, gout, gin, M, N, K, dtype, gin_dt, stream):
        self.inside("softmax_backward out", out, ESIZE[dtype], [(M * N * K, 1)])
        self.inside("softmax_backward grad_out", gout, ESIZE[dtype], [(M * N * K, 1)])
        self.inside("softmax_backward grad_in", gin, ESIZE[gin_dt], [(M * N * K, 1)])

    chk_fg_log_softmax_backward = chk_fg_softmax_backward

    def chk_fg_rms_norm_backward(self, x, dy, inv_rms, w, dx, dwp, prow, M, N, dtype, stream):
        e = ESIZE[dtype]
        for what, p in (("x", x), ("dy", dy), ("dx", dx)):
            self.inside("rms_norm_backward " + what, p, e, [(M * N, 1)])
        self.inside("rms_norm_backward inv_rms", inv_rms, 4, [(M, 1)])
        self.inside("rms_norm_backward w", w, e, [(N, 1)])
        if dwp is not None:
            assert 1 <= prow <= M
            self.inside("rms_norm_backward dw_partial", dwp, 4, [(prow * N, 1)])

    def chk_fg_rms_norm_backward_dw(self, dwp, prow, N, dw, dtype, stream):
        self.inside("rms_norm_backward_dw partial", dwp, 4, [(prow * N, 1)])
        self.inside("rms_norm_backward_dw dw", dw, ESIZE[dtype], [(N, 1)])

    def chk_fg_transpose2d(self, src, dst, rows, cols, srs, drs, eb, stream):
        self.inside("transpose src", src, eb, [(rows, srs), (cols, 1)])
        self.inside("transpose dst", dst, eb, [(cols, drs), (rows, 1)])

    def chk_fg_silu_and_mul(self, a, b, out, rows, cols, ars, brs, ors, dtype, stream):
        e = ESIZE[dtype]
        self.inside("silu a", a, e, [(rows, ars), (cols, 1)])
        self.inside("silu b", b, e, [(rows, brs), (cols, 1)])
        self.inside("silu out", out, e, [(rows, ors), (cols, 1)])

    def chk_fg_silu_and_mul_backward(self, a, b, g, da, db, rows, cols, ars, brs, grs, dars, dbrs, dtype, stream):
        e = ESIZE[dtype]
        for what, ptr, rs in (("a", a, ars), ("b", b, brs), ("grad_out", g, grs), ("grad_a", da, dars), ("grad_b", db, dbrs)):
            self.inside("silu backward " + what, ptr, e, [(rows, rs), (cols, 1)])

    def chk_fg_gemm(self, A, B, bias, C, M, N, K, sam, sak, sbk, sbn, sim, sin_, scm, scn, alpha, beta, ab, cdt, bdt,
                    schedule, ws, ws_bytes, used, stream):
        self.inside("gemm A", A, ESIZE[ab], [(M, sam), (K, sak)])
        self.inside("gemm B", B, ESIZE[ab], [(K, sbk), (N, sbn)])
        self.inside("gemm bias", bias, ESIZE[bdt], [(M, sim), (N, sin_)])
        self.inside("gemm C", C, ESIZE[cdt], [(M, scm), (N, scn)])
        if ws is not None and ws_bytes:
            self.inside("gemm workspace", ws, 1, [(ws_bytes, 1)])

    def chk_fg_bmm(self, A, B, C, batch, M, N, K, sab, sam, sak, sbb, sbk, sbn, scb, scm, scn, dtype, stream):
        e = ESIZE[dtype]
        self.inside("bmm A", A, e, [(batch, sab), (M, sam), (K, sak)])
        self.inside("bmm B", B, e, [(batch, sbb), (K, sbk), (N, sbn)])
        self.inside("bmm C", C, e, [(batch, scb), (M, scm), (N, scn)])

    def chk_fg_rope(self, qo, ko, q, k, cos, sin, pos, pos_i64, n_tok, seq_len, Hq, Hk, D, qs, ks, qos, kos, pos_stride,
                    cos_stride, sin_stride, max_pos, interleaved, dtype, cs_dtype, stream):
        e = ESIZE[dtype]
        for what, p, H, st in (("q", q, Hq, qs), ("k", k, Hk, ks), ("q_out", qo, Hq, qos), ("k_out", ko, Hk, kos)):
            st = list(st)
            self.inside("rope " + what, p, e, [(n_tok, st[0]), (H, st[1]), (D, st[2])])
        self.inside("rope cos", cos, ESIZE[cs_dtype], [(max_pos, cos_stride), (D // 2, 1)])
        self.inside("rope sin", sin, ESIZE[cs_dtype], [(max_pos, sin_stride), (D // 2, 1)])
        if pos is not None:
            self.inside("rope positions", pos, 8 if pos_i64 else 4, [(n_tok, pos_stride)])
            vals = self.read(pos, ctypes.c_int64 if pos_i64 else ctypes.c_int32, (n_tok - 1) * pos_stride + 1)[::pos_stride]
            assert all(0 <= v < max_pos for v in vals), "rope: a position outside the cos/sin table"
        else:
            assert 0 < seq_len <= max_pos, "rope: token_index %% seq_len would leave the cos/sin table"

    def chk_fg_reshape_and_cache_flash(self, key, value, kc, vc, slots, slot_i64, n_tok, H, D, bs, ks, vs, blk, eb, stream):
        self.inside("cache key", key, eb, [(n_tok, ks), (H * D, 1)])
        self.inside("cache value", value, eb, [(n_tok, vs), (H * D, 1)])
        self.inside("cache slot_mapping", slots, 8 if slot_i64 else 4, [(n_tok, 1)])
        vals = [v for v in self.read(slots, ctypes.c_int64 if slot_i64 else ctypes.c_int32, n_tok) if v >= 0]
        for what, cache in (("key_cache", kc), ("value_cache", vc)):
            for v in (min(vals), max(vals)) if vals else ():
                row = int(cache) + ((v // bs) * blk + (v % bs) * H * D) * eb
                begin, end = self.ranges[int(cache)]
                assert begin <= row and row + H * D * eb <= end, "cache scatter: slot %d lies outside %s" % (v, what)

    def chk_fg_reshape_and_cache(self, key, value, kc, vc, slots, slot_i64, n_tok, H, D, bs, x, nblk, ks, vs, eb, stream):
        self.inside("cache(v0) key", key, eb, [(n_tok, ks), (H * D, 1)])
        self.inside("cache(v0) value", value, eb, [(n_tok, vs), (H * D, 1)])
        self.inside("cache(v0) slot_mapping", slots, 8 if slot_i64 else 4, [(n_tok, 1)])
        self.inside("cache(v0) key_cache", kc, eb, [(nblk * H * D * bs, 1)])
        self.inside("cache(v0) value_cache", vc, eb, [(nblk * H * D * bs, 1)])
        assert D % x == 0

    def chk_fg_flash_attn_varlen_fwd(self, pref, stream):
        p = pref._obj
        e = ESIZE[p.dtype]
        B = p.batch
        self.inside("attn cu_seqlens_q", p.cu_seqlens_q, 4, [(B + 1, 1)])
        self.inside("attn seqused_k", p.seqused_k, 4, [(B, 1)])
        cu = self.read(ctypes.cast(p.cu_seqlens_q, ctypes.c_void_p), ctypes.c_int32, B + 1)
        sk = self.read(ctypes.cast(p.seqused_k, ctypes.c_void_p), ctypes.c_int32, B)
        assert cu[0] == 0 and all(b >= a for a, b in zip(cu, cu[1:])) and cu[-1] <= p.total_q
        assert max(b - a for a, b in zip(cu, cu[1:])) <= p.max_seqlen_q and max(sk) <= p.max_seqlen_k
        self.inside("attn q", p.q, e, [(p.total_q, p.q_row_stride), (p.Hq, p.q_head_stride), (p.D, 1)])
        self.inside("attn out", p.out, e, [(p.total_q, p.o_row_stride), (p.Hq, p.o_head_stride), (p.D, 1)])
        self.inside("attn lse", ctypes.cast(p.lse, ctypes.c_void_p), 4, [(p.Hq * p.total_q, 1)])
        pages = [(n + p.page_size - 1) // p.page_size for n in sk]
        if max(pages) > 0:
            self.inside("attn block_table", ctypes.cast(p.block_table, ctypes.c_void_p), 4,
                        [(B, p.block_table_stride), (max(pages), 1)])
            # rows a kernel may read: every row of a sequence's pages but, in its last page, only those below its
            # length (the kernels clamp keys past the end to the last one; a dense K/V presented as pages of
            # consecutive rows has nothing behind the last row of its last batch)
            used = {}
            base = ctypes.cast(p.block_table, ctypes.c_void_p).value
            for b, n in enumerate(pages):
                ids = self.read(base + 4 * b * p.block_table_stride, ctypes.c_int32, n)
                for j, page in enumerate(ids):
                    assert page >= 0
                    rows = p.page_size if j + 1 < n else (sk[b] - 1) % p.page_size + 1
                    used[page] = max(used.get(page, 0), rows)
            for what, cache, ps, rs, hs in (("k_cache", p.k_cache, p.k_page_stride, p.k_row_stride, p.k_head_stride),
                                            ("v_cache", p.v_cache, p.v_page_stride, p.v_row_stride, p.v_head_stride)):
                for page, rows in used.items():
                    self.inside("attn %s page %d" % (what, page), cache, e, [(rows, rs), (p.Hk, hs), (p.D, 1)],
                                offset=page * ps)
        if p.alibi_slopes:
            self.inside("attn alibi", ctypes.cast(p.alibi_slopes, ctypes.c_void_p), 4,
                        [(B if p.alibi_batch_stride else 1, p.alibi_batch_stride), (p.Hq, 1)])
        assert p.Hq % p.Hk == 0 and p.D % 8 == 0


@pytest.fixture
def hx(monkeypatch):
    return Harness(monkeypatch)


bf16 = torch.bfloat16


def _r(*shape, dtype=bf16):
    return torch.randn(*shape).to(dtype)


# ---- GEMM family ---------------------------------------------------------------------------------------------
@pytest.mark.parametrize("dtype", [torch.float16, bf16, torch.float32])
def test_mm_addmm_bmm_operands(hx, dtype):
    a, b = _r(33, 72, dtype=dtype), _r(72, 40, dtype=dtype)
    w = _r(40, 72, dtype=dtype)
    big = _r(64, 200, dtype=dtype)
    flag_gems.mm(a, b)
    flag_gems.mm(a, w.t())                              # B = W^T, consumed as it is
    flag_gems.mm(w.t()[:, :33].t()[:, :72], b)          # a view of a view
    flag_gems.mm(b.t(), a.t())                          # both column-major
    flag_gems.mm(big[:33, 5:77], b)                     # row-strided slice
    flag_gems.mm(big[::2, ::2][:33, :72], b)            # both strides > 1: copied first
    out = torch.empty(50, 64, dtype=dtype)[:33, :40]
    torch.ops.aten.mm.out  # (the override takes the same path)
    flag_gems.mm_out(a, b, out=out)                     # strided out
    flag_gems.addmm(_r(40, dtype=dtype), a, b)          # bias broadcast over rows
    flag_gems.addmm(_r(33, 1, dtype=dtype), a, b, alpha=0.5, beta=-2.0)
    flag_gems.addmm(_r(33, 40, dtype=dtype), a, b)
    flag_gems.addmm(torch.tensor(1.5).to(dtype), a, b)  # scalar bias
    flag_gems.addmm(_r(64, 80, dtype=dtype)[:33, ::2], a.t().contiguous().t(), b)
    flag_gems.bmm(_r(3, 17, 24, dtype=dtype), _r(3, 24, 9, dtype=dtype))
    flag_gems.bmm(_r(3, 24, 17, dtype=dtype).transpose(1, 2), _r(9, 3, 24, dtype=dtype).permute(1, 2, 0))
    flag_gems.bmm(_r(1, 17, 24, dtype=dtype), _r(1, 24, 9, dtype=dtype))
    done = hx.check_all()
    assert done.count("fg_gemm") >= 13 and done.count("fg_bmm") == 2


def test_mm_skinny_and_column_major_a_take_their_helpers(hx):
    # a column-major A in front of a wide output is transposed first (fg_transpose2d), then multiplied
    a = _r(512, 300).t()                # [300, 512] column-major
    w = _r(1024, 512)
    flag_gems.mm(a, w.t())
    flag_gems.mm(_r(8, 4096), _r(512, 4096).t())        # skinny: asks for a workspace size (0 from the stand-in)
    done = hx.check_all()
    assert "fg_gemm" in done


# ---- row-wise operators --------------------------------------------------------------------------------------
@pytest.mark.parametrize("dtype", [torch.float16, bf16, torch.float32])
def test_rowwise_operands(hx, dtype):
    x = _r(6, 5, 64, dtype=dtype)
    w = _r(64, dtype=dtype)
    flag_gems.softmax(x, -1)
    flag_gems.softmax(x, 1)                              # middle axis
    flag_gems.softmax(x, 0, half_to_float=dtype != torch.float32)
    flag_gems.softmax(x.transpose(0, 2), -1)             # made contiguous first
    flag_gems.log_softmax(x, -1)
    flag_gems.log_softmax(x, 1)
    flag_gems.rms_norm(x, [64], w, 1e-5)
    flag_gems.rms_norm(x, [5, 64], _r(5, 64, dtype=dtype), 1e-5)
    flag_gems.rms_norm(x[:, ::2], [64], w, 1e-5)
    y = flag_gems.softmax(x, -1)
    flag_gems.softmax_backward(_r(6, 5, 64, dtype=dtype), y, -1, dtype)
    flag_gems.log_softmax_backward(_r(6, 5, 64, dtype=dtype), y, 1, dtype)
    xr, rr = _r(30, 64, dtype=dtype), _r(30, 64, dtype=dtype)
    flag_gems.fused_add_rms_norm(xr, rr, [64], w, 1e-6)
    flag_gems.fused_add_rms_norm(_r(60, 64, dtype=dtype)[::2], _r(30, 128, dtype=dtype)[:, :64], [64], w, 1e-6)
    gu = _r(30, 256, dtype=dtype)
    flag_gems.silu_and_mul(gu[:, :128], gu[:, 128:])      # halves of one gate-up tensor
    flag_gems.silu_and_mul_out(gu[:, :128], gu[:, 128:], torch.empty(30, 200, dtype=dtype)[:, :128])
    done = hx.check_all()
    for name in ("fg_softmax", "fg_log_softmax", "fg_rms_norm", "fg_fused_add_rms_norm", "fg_silu_and_mul",
                 "fg_softmax_backward", "fg_log_softmax_backward"):
        assert name in done, name


def test_silu_and_mul_autograd_operands(hx):
    gu = _r(30, 256).requires_grad_()
    y = flag_gems.silu_and_mul(gu[:, :128], gu[:, 128:])       # halves of one gate-up tensor, saved as views
    y.backward(_r(60, 128)[::2])                               # a gradient with gaps between its rows
    a, b = _r(4, 1, 64).requires_grad_(), _r(1, 5, 64).requires_grad_()
    flag_gems.silu_and_mul(a, b).sum().backward()              # broadcast operands, an expanded (stride-0) gradient
    assert gu.grad.shape == (30, 256) and a.grad.shape == (4, 1, 64) and b.grad.shape == (1, 5, 64)
    done = hx.check_all()
    assert done.count("fg_silu_and_mul") == 2 and done.count("fg_silu_and_mul_backward") == 2


def test_silu_and_mul_gradient_without_the_kernel(hx, monkeypatch):
    """A library built without the gradient kernel answers FG_ERR_UNSUPPORTED: the operator asks once, then takes the
    gradient from torch's elementwise operations (checked here against the oracle) and does not ask again; any other
    error code is raised."""
    import importlib

    mod = importlib.import_module("flaggems_amd.fused.silu_and_mul")   # (the package re-exports a function of that name)
    from oracle import torch_ref as O

    real = hx.rec.__getattr__
    answers = {"fg_silu_and_mul_backward": -2}

    def lib_attr(name):
        call = real(name)
        if name in answers:
            def refused(*args):
                call(*args)
                return answers[name]
            return refused
        if name == "fg_last_error":
            return lambda: b"refused"
        return call

    monkeypatch.setattr(type(hx.rec), "__getattr__", lambda self, name: lib_attr(name))
    monkeypatch.setattr(mod, "_grad_kernel_built", None)
    a, b, g = _r(7, 40, dtype=torch.float32), _r(7, 40, dtype=torch.float32), _r(7, 40, dtype=torch.float32)
    for _ in range(2):
        da, db = mod._grads(a, b, g)
        want_a, want_b = O.silu_and_mul_grads(a, b, g)
        torch.testing.assert_close(da.double(), want_a, atol=1e-5, rtol=1e-5)
        torch.testing.assert_close(db.double(), want_b, atol=1e-5, rtol=1e-5)
    assert [n for n, _ in hx.rec.calls].count("fg_silu_and_mul_backward") == 1 and mod._grad_kernel_built is False
    monkeypatch.setattr(mod, "_grad_kernel_built", None)
    answers["fg_silu_and_mul_backward"] = -3
    with pytest.raises(RuntimeError, match="fg_silu_and_mul_backward failed"):
        mod._grads(a, b, g)


def test_rms_norm_autograd_operands(hx):
    x = _r(12, 96).requires_grad_()
    w = _r(96).requires_grad_()
    y = flag_gems.rms_norm(x, [96], w, 1e-5)
    y.backward(_r(12, 96))
    done = hx.check_all()
    assert "fg_rms_norm_backward" in done and "fg_rms_norm_backward_dw" in done


# ---- rotary embedding and the cache scatter ------------------------------------------------------------------
@pytest.mark.parametrize("interleaved", [False, True])
def test_rope_operands(hx, interleaved):
    T, Hq, Hk, D, max_pos = 10, 8, 2, 64, 32
    qkv = _r(T, (Hq + 2 * Hk) * D)
    q = qkv[:, :Hq * D].view(T, Hq, D)                   # views into a fused projection: token stride 768
    k = qkv[:, Hq * D:(Hq + Hk) * D].view(T, Hk, D)
    cos, sin = _r(max_pos, D // 2, dtype=torch.float32), _r(max_pos, D // 2, dtype=torch.float32)
    pos = torch.randint(0, max_pos, (T,))
    flag_gems.apply_rotary_pos_emb(q, k, cos, sin, pos, interleaved, inplace=True)
    flag_gems.apply_rotary_pos_emb(q, k, cos, sin, pos.int(), interleaved)
    cache = _r(max_pos, D, dtype=torch.float32)          # one table, cos and sin halves: row stride D
    c2, s2 = cache.chunk(2, -1)
    flag_gems.apply_rotary_pos_emb(q, k, c2, s2, pos, interleaved)
    q4, k4 = _r(2, 5, Hq, D), _r(2, 5, Hk, D)            # no positions: token index modulo the sequence length
    flag_gems.apply_rotary_pos_emb(q4, k4, cos, sin, None, interleaved)
    flag_gems.apply_rotary_pos_emb(_r(T, Hq, 96), _r(T, Hk, 96), _r(max_pos, 48), _r(max_pos, 48), pos, interleaved)
    done = hx.check_all()
    assert done.count("fg_rope") == 5


def test_cache_scatter_operands(hx):
    T, H, D, bs, nblk = 11, 4, 32, 16, 6
    kv = _r(T + 3, 2 * H * D)
    key, value = kv[:, :H * D].view(-1, H, D), kv[:, H * D:].view(-1, H, D)   # strided token rows, padded token count
    both = torch.zeros(2, nblk, bs, H, D, dtype=bf16)
    kc, vc = both.unbind(0)
    slots = torch.randperm(nblk * bs)[:T]
    slots[3] = -1                                         # a padding token
    flag_gems.reshape_and_cache_flash(key, value, kc, vc, slots, "auto", None, None)
    flag_gems.reshape_and_cache_flash(key, value, kc, vc, slots.int(), "auto", None, None)
    last = torch.tensor([nblk * bs - 1, 0])
    flag_gems.reshape_and_cache_flash(key[:2], value[:2], kc, vc, last, "auto", None, None)
    x = 8
    kc0 = torch.zeros(nblk, H, D // x, bs, x, dtype=bf16)
    vc0 = torch.zeros(nblk, H, D, bs, dtype=bf16)
    flag_gems.reshape_and_cache(key, value, kc0, vc0, slots, "auto", None, None)
    done = hx.check_all()
    assert done.count("fg_reshape_and_cache_flash") == 3 and done.count("fg_reshape_and_cache") == 1


# ---- attention ------------------------------------------------------------------------------------------------
def _paged_case(lens, Hq, Hk, D, bs, nblk, dtype=bf16):
    qlens = [a for a, _ in lens]
    klens = [b for _, b in lens]
    q = _r(sum(qlens), Hq, D, dtype=dtype)
    both = _r(2, nblk, bs, Hk, D, dtype=dtype)
    kc, vc = both.unbind(0)
    cu = torch.tensor([0] + qlens, dtype=torch.int32).cumsum(0, dtype=torch.int32)
    sk = torch.tensor(klens, dtype=torch.int32)
    bt = torch.randint(0, nblk, (len(lens), (max(klens) + bs - 1) // bs), dtype=torch.int32)
    return q, kc, vc, cu, sk, bt, max(qlens), max(klens)


def test_paged_attention_operands(hx):
    q, kc, vc, cu, sk, bt, mq, mk = _paged_case([(1, 1328), (5, 18), (129, 463)], 8, 2, 128, 32, 64)
    flag_gems.flash_attn_varlen_func(q, kc, vc, mq, cu, mk, seqused_k=sk, causal=True, block_table=bt)
    flag_gems.flash_attn_varlen_func(q, kc, vc, mq, cu, mk, seqused_k=sk, causal=True, block_table=bt, softcap=10.0,
                                     window_size=(64, 0), return_softmax_lse=True,
                                     alibi_slopes=torch.rand(3, 8, dtype=torch.float32))
    out = torch.empty(q.shape[0], 8, 256, dtype=bf16)[:, :, :128]       # out= with padded heads
    flag_gems.flash_attn_varlen_func(q, kc, vc, mq, cu, mk, seqused_k=sk, causal=True, block_table=bt, out=out)
    wide = torch.zeros(3, 4096 // 32, dtype=torch.int32)                # max_seqlen_k above every length
    wide[:, :bt.shape[1]] = bt
    flag_gems.flash_attn_varlen_func(q, kc, vc, mq, cu, 4096, seqused_k=sk, causal=True, block_table=wide)
    q1, kc, vc, cu1, sk1, bt1, mq1, mk1 = _paged_case([(1, 700), (1, 3), (1, 0), (1, 129)], 32, 8, 128, 16, 64)
    flag_gems.flash_attn_varlen_func(q1, kc, vc, 1, cu1, mk1, seqused_k=sk1, causal=True, block_table=bt1)
    qkv = _r(q1.shape[0], 3 * 32 * 128)                                  # q as a view into a fused projection
    flag_gems.flash_attn_varlen_func(qkv[:, :32 * 128].view(-1, 32, 128), kc, vc, 1, cu1, mk1, seqused_k=sk1,
                                     causal=True, block_table=bt1)
    done = hx.check_all()
    assert done.count("fg_flash_attn_varlen_fwd") == 6


@pytest.mark.parametrize("layout", ["bshd", "bhsd"])
def test_dense_attention_operands(hx, layout):
    B, Hq, Hk, Sq, Sk, D = 3, 8, 2, 17, 70, 64
    if layout == "bshd":
        q, k, v = _r(B, Sq, Hq, D), _r(B, Sk, Hk, D), _r(B, Sk, Hk, D)
    else:
        q, k, v = _r(B, Hq, Sq, D).transpose(1, 2), _r(B, Hk, Sk, D).transpose(1, 2), _r(B, Hk, Sk, D).transpose(1, 2)
    flag_gems.ops.flash_attention_forward(q, k, v, None, None, Sq, Sk, 0.0, True, False, scale=D ** -0.5)
    flag_gems.ops.flash_attention_forward(q, k, v, None, None, Sq, Sk, 0.0, False, False, scale=D ** -0.5,
                                          window_size_left=30, window_size_right=20)
    qs, ks, vs = _r(B, Hq, 40, D), _r(B, Hq, 40, D), _r(B, Hq, 40, D)
    flag_gems.scaled_dot_product_attention(qs, ks, vs, is_causal=True)
    done = hx.check_all()
    assert done.count("fg_flash_attn_varlen_fwd") == 3


def test_the_checks_notice_a_wrong_stride_a_long_row_and_a_foreign_pointer(hx):
    x = _r(8, 64)
    y = torch.empty_like(x)
    half = x[:, :32]                      # 32 columns at row stride 64
    lib = _C.lib()
    lib.fg_rms_norm(half.data_ptr(), None, y.data_ptr(), None, 8, 32, 64, 64, 1e-5, _C.FG_BF16, 0)
    assert hx.check_all() == ["fg_rms_norm"]
    hx.rec.calls.clear()
    lib.fg_rms_norm(half.data_ptr(), None, y.data_ptr(), None, 8, 64, 64, 64, 1e-5, _C.FG_BF16, 0)   # N of the parent
    assert hx.check_all() == ["fg_rms_norm"]      # still inside x's storage: a view's overrun into its parent is legal
    hx.rec.calls.clear()
    lib.fg_rms_norm(x.data_ptr(), None, y.data_ptr(), None, 8, 64, 128, 64, 1e-5, _C.FG_BF16, 0)      # doubled stride
    with pytest.raises(AssertionError, match="past its storage"):
        hx.check_all()
    hx.rec.calls.clear()
    lib.fg_rms_norm(x.data_ptr(), None, y.data_ptr(), None, 9, 64, 64, 64, 1e-5, _C.FG_BF16, 0)       # one row too many
    with pytest.raises(AssertionError, match="past its storage"):
        hx.check_all()
    hx.rec.calls.clear()
    lib.fg_rms_norm(x.data_ptr() + 2, None, y.data_ptr(), None, 8, 64, 64, 64, 1e-5, _C.FG_BF16, 0)   # not a data_ptr()
    with pytest.raises(AssertionError, match="did not come from"):
        hx.check_all()


def test_repeated_calls_take_the_short_host_path(hx):
    """Decode-size calls are host-bound unless the wrapper stays short: the workspace query of a GEMM shape is asked
    of the library once, attention hands out its dropout placeholders instead of allocating them, and rotary
    embedding on (tokens, heads, dim) tensors in place returns its arguments without making views."""
    from flaggems_amd.ops import _gemm

    _gemm._ws_need.clear()
    a, w = _r(8, 256), _r(64, 256)
    for _ in range(3):
        flag_gems.mm(a, w.t())
    flag_gems.mm(_r(9, 256), w.t())
    names = [n for n, _ in hx.rec.calls]
    assert names.count("fg_gemm") == 4 and names.count("fg_gemm_workspace_bytes") == 2
    _gemm._ws_need.clear()

    q1, kc, vc, cu1, sk1, bt1, _, mk1 = _paged_case([(1, 70), (1, 3)], 8, 2, 64, 16, 16)
    from flaggems_amd.ops.attention import mha_varlan_fwd

    r1 = mha_varlan_fwd(q1, kc, vc, None, cu1, cu1, sk1, None, bt1, None, 1, mk1, 0.0, 0.125, False, True, -1, -1, 0.0, False, None)
    r2 = mha_varlan_fwd(q1, kc, vc, None, cu1, cu1, sk1, None, bt1, None, 1, mk1, 0.0, 0.125, False, True, -1, -1, 0.0, False, None)
    assert all(x is y for x, y in zip(r1[5:], r2[5:])) and r1[0] is not r2[0] and r1[4] is not r2[4]

    q, k = _r(5, 8, 64), _r(5, 2, 64)
    cos, sin = _r(16, 32, dtype=torch.float32), _r(16, 32, dtype=torch.float32)
    pos = torch.arange(5)
    qo, ko = flag_gems.apply_rotary_pos_emb(q, k, cos, sin, pos, False, inplace=True)
    assert qo is q and ko is k
    qo, ko = flag_gems.apply_rotary_pos_emb(q, k, cos, sin, pos, False)
    assert qo.shape == q.shape and qo.data_ptr() != q.data_ptr()
    hx.check_all()
