"""GPU parity of every operator under torch.ops.flag_gems (the schemas of the reference's C extension,
src/flag_gems/csrc/cstub.cpp:26-129) against the CPU oracle, with the reference's tolerance rule."""
import pytest
import torch

import flag_gems  # noqa: F401  (defines the namespace)
from helpers import gems_assert_close
from oracle import torch_ref as O

pytestmark = pytest.mark.gpu
FG = torch.ops.flag_gems
DTYPES = [torch.float16, torch.bfloat16, torch.float32]


@pytest.mark.parametrize("dtype", DTYPES)
def test_custom_op_blas(gpu, dtype):
    torch.manual_seed(0)
    a = torch.randn(130, 264, device=gpu, dtype=dtype)
    b = torch.randn(264, 72, device=gpu, dtype=dtype)
    bias = torch.randn(72, device=gpu, dtype=dtype)
    gems_assert_close(FG.mm(a, b), O.mm(a, b), dtype, reduce_dim=264)
    gems_assert_close(FG.addmm(bias, a, b), O.addmm(bias, a, b), dtype, reduce_dim=264)
    gems_assert_close(FG.addmm(bias, a, b, beta=0.5, alpha=-2.0), O.addmm(bias, a, b, beta=0.5, alpha=-2.0), dtype,
                      reduce_dim=264)
    a3 = torch.randn(3, 65, 136, device=gpu, dtype=dtype)
    b3 = torch.randn(3, 136, 40, device=gpu, dtype=dtype)
    gems_assert_close(FG.bmm(a3, b3), O.bmm(a3, b3), dtype, reduce_dim=136)


@pytest.mark.parametrize("dtype", DTYPES)
def test_custom_op_softmax_and_backward(gpu, dtype):
    torch.manual_seed(1)
    x = torch.randn(37, 5, 300, device=gpu, dtype=dtype)
    for dim in (-1, 1):
        y = FG.softmax(x, dim)
        gems_assert_close(y, O.softmax(x, dim), dtype)
        g = torch.randn_like(y)
        gems_assert_close(FG.softmax_backward(g, y, dim, dtype), O.softmax_backward(g, y, dim), dtype,
                          reduce_dim=x.shape[dim])
    if dtype != torch.float32:
        y32 = FG.softmax(x, -1, True)
        assert y32.dtype == torch.float32
        gems_assert_close(y32, O.softmax(x, -1).float(), torch.float32)


@pytest.mark.parametrize("dtype", DTYPES)
def test_custom_op_norms(gpu, dtype):
    torch.manual_seed(2)
    x = torch.randn(4, 33, 1024, device=gpu, dtype=dtype)
    r = torch.randn_like(x)
    w = (torch.rand(1024, device=gpu) + 0.5).to(dtype)
    gems_assert_close(FG.rms_norm(x, w, 1e-5), O.rms_norm(x, w, 1e-5), dtype)
    ry, rr = O.fused_add_rms_norm(x, r, w, 1e-6)
    xp, rp = x.data_ptr(), r.data_ptr()
    assert FG.fused_add_rms_norm(x, r, w, 1e-6) is None
    assert x.data_ptr() == xp and r.data_ptr() == rp
    gems_assert_close(x, ry, dtype)  # the arguments themselves hold the results
    gems_assert_close(r, rr, dtype)
    # rows that are not dense (a column slice): the arguments are still the ones mutated
    big_x = torch.randn(16, 2048, device=gpu, dtype=dtype)
    big_r = torch.randn_like(big_x)
    xs, rs = big_x[:, :1024], big_r[:, 1024:]
    keep_x, keep_r = big_x[:, 1024:].clone(), big_r[:, :1024].clone()
    ry, rr = O.fused_add_rms_norm(xs, rs, w, 1e-6)
    FG.fused_add_rms_norm(xs, rs, w, 1e-6)
    gems_assert_close(big_x[:, :1024], ry, dtype)
    gems_assert_close(big_r[:, 1024:], rr, dtype)
    assert torch.equal(big_x[:, 1024:], keep_x) and torch.equal(big_r[:, :1024], keep_r)
    with pytest.raises(RuntimeError, match="same shape"):
        FG.fused_add_rms_norm(x, r[:2], w, 1e-6)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("interleaved", [False, True])
def test_custom_op_rotary(gpu, dtype, interleaved):
    torch.manual_seed(3)
    T, Hq, Hk, D = 77, 8, 2, 128
    q = torch.randn(T, Hq, D, device=gpu, dtype=dtype)
    k = torch.randn(T, Hk, D, device=gpu, dtype=dtype)
    cos, sin = O.rope_cos_sin(512, D, device=gpu)
    pos = torch.randint(0, 512, (T,), device=gpu)
    rq, rk = O.apply_rotary_pos_emb(q, k, cos, sin, pos, interleaved)
    oq, ok = FG.rotary_embedding(q, k, cos, sin, pos, interleaved)
    assert oq.data_ptr() != q.data_ptr()
    gems_assert_close(oq, rq, dtype)
    gems_assert_close(ok, rk, dtype)
    assert FG.rotary_embedding_inplace(q, k, cos, sin, pos, interleaved) is None
    gems_assert_close(q, rq, dtype)
    gems_assert_close(k, rk, dtype)


def test_custom_op_cache_and_attention(gpu):
    torch.manual_seed(4)
    dtype = torch.bfloat16
    Hq, Hk, D, bs, nblk = 8, 2, 128, 16, 64
    lens = [150, 1, 97]
    T = sum(lens)
    q = torch.randn(T, Hq, D, device=gpu, dtype=dtype)
    k = torch.randn(T, Hk, D, device=gpu, dtype=dtype)
    v = torch.randn(T, Hk, D, device=gpu, dtype=dtype)
    perm = torch.randperm(nblk)
    pages = (max(lens) + bs - 1) // bs
    bt = torch.zeros(len(lens), pages, dtype=torch.int32)
    slots, o = [], 0
    for i, l in enumerate(lens):
        n = (l + bs - 1) // bs
        bt[i, :n] = perm[o:o + n]
        o += n
        t = torch.arange(l)
        slots.append(bt[i, t // bs].long() * bs + t % bs)
    slots = torch.cat(slots).to(gpu)
    bt = bt.to(gpu)
    kc = torch.zeros(nblk, bs, Hk, D, dtype=dtype, device=gpu)
    vc = torch.zeros_like(kc)
    ek, ev = O.reshape_and_cache_flash(k, v, kc, vc, slots)
    assert FG.reshape_and_cache_flash(k, v, kc, vc, slots, "auto", None, None) is None
    assert torch.equal(kc.cpu(), ek) and torch.equal(vc.cpu(), ev)  # bit-exact
    cu = torch.tensor([0] + lens, dtype=torch.int32, device=gpu).cumsum(0, dtype=torch.int32)
    sk = torch.tensor(lens, dtype=torch.int32, device=gpu)
    out, lse = FG.flash_attn_varlen_func(q, kc, vc, max(lens), cu, max(lens), None, sk, None, 0.0, None, True, None,
                                         0.0, None, False, False, bt, False, None, None, None, None, None, 2)
    ref, rlse = O.paged_attention(q, kc, vc, lens, lens, bt, D ** -0.5, compute_dtype=torch.float32, return_lse=True)
    torch.testing.assert_close(out.float().cpu(), ref, atol=2e-2, rtol=1e-2)
    assert lse.shape == (Hq, T) and lse.dtype == torch.float32  # returned whatever return_softmax_lse says
    torch.testing.assert_close(lse.cpu(), rlse, atol=1e-2, rtol=1e-3)
    # keyword form with a window and a caller-provided output
    mine = torch.empty_like(q)
    out2, _ = FG.flash_attn_varlen_func(q, kc, vc, max(lens), cu, max(lens), seqused_k=sk, causal=True,
                                        window_size=[40, 0], block_table=bt, out=mine)
    assert out2.data_ptr() == mine.data_ptr()
    ref2 = O.paged_attention(q, kc, vc, lens, lens, bt, D ** -0.5, window=(40, 0), compute_dtype=torch.float32)
    torch.testing.assert_close(mine.float().cpu(), ref2, atol=2e-2, rtol=1e-2)
    with pytest.raises(RuntimeError):
        FG.flash_attn_varlen_func(q, kc, vc, max(lens), cu, max(lens), seqused_k=sk, block_table=bt, fa_version=3)
