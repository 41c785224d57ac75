"""GPU parity of mm / addmm (data-parallel and stream-K schedules) against the CPU oracle.
Shapes, scalars and layouts follow tests/test_blas_ops.py:17-136 of the reference."""
import pytest
import torch

import flag_gems
from flaggems_amd import _C
from flaggems_amd.ops import _gemm
from oracle import torch_ref as O

from helpers import FLOAT_DTYPES, MNK_SHAPES, SCALARS, gems_assert_close

pytestmark = pytest.mark.gpu

EXTRA_SHAPES = [(256, 256, 256), (300, 520, 264), (1024, 768, 512), (64, 4096, 136)]


def _operand(rows, cols, dtype, dev, transposed):
    if transposed:
        return torch.randn(cols, rows, dtype=dtype, device=dev).t()
    return torch.randn(rows, cols, dtype=dtype, device=dev)


@pytest.mark.parametrize("dtype", FLOAT_DTYPES)
@pytest.mark.parametrize("M,N,K", MNK_SHAPES + EXTRA_SHAPES)
@pytest.mark.parametrize("b_col_major", [False, True])
@pytest.mark.parametrize("a_col_major", [False, True])
def test_mm(gpu, M, N, K, dtype, a_col_major, b_col_major):
    torch.manual_seed(0)
    a = _operand(M, K, dtype, gpu, a_col_major)
    b = _operand(K, N, dtype, gpu, b_col_major)
    ref = O.mm(a, b)
    with flag_gems.use_gems():
        res = torch.mm(a, b)
    gems_assert_close(res, ref, dtype, reduce_dim=K)
    out = torch.empty(M, N, dtype=dtype, device=gpu)
    with flag_gems.use_gems():
        torch.mm(a, b, out=out)
    gems_assert_close(out, ref, dtype, reduce_dim=K)


@pytest.mark.parametrize("dtype", FLOAT_DTYPES)
@pytest.mark.parametrize("M,N,K", MNK_SHAPES + EXTRA_SHAPES[:2])
@pytest.mark.parametrize("scalar", SCALARS)
@pytest.mark.parametrize("b_col_major", [False, True])
def test_addmm(gpu, M, N, K, scalar, dtype, b_col_major):
    torch.manual_seed(0)
    a = torch.randn(M, K, dtype=dtype, device=gpu)
    b = _operand(K, N, dtype, gpu, b_col_major)
    for bias in (torch.randn(N, dtype=dtype, device=gpu), torch.randn(M, N, dtype=dtype, device=gpu)):
        ref = O.addmm(bias, a, b, alpha=scalar, beta=scalar)
        with flag_gems.use_gems():
            res = torch.addmm(bias, a, b, alpha=scalar, beta=scalar)
        gems_assert_close(res, ref, dtype, reduce_dim=K)
    out = torch.empty(M, N, dtype=dtype, device=gpu)
    with flag_gems.use_gems():
        torch.addmm(bias, a, b, alpha=scalar, beta=scalar, out=out)
    gems_assert_close(out, ref, dtype, reduce_dim=K)


BMM_LAYOUTS = ["contiguous", "b_transposed", "a_transposed", "broadcast_b", "batch_inner"]


@pytest.mark.parametrize("dtype", FLOAT_DTYPES)
@pytest.mark.parametrize("M,N,K", MNK_SHAPES + EXTRA_SHAPES[:3] + [(256, 512, 128), (77, 40, 24)])
@pytest.mark.parametrize("layout", BMM_LAYOUTS)
def test_bmm(gpu, M, N, K, dtype, layout):
    """tests/test_blas_ops.py:95-110 of the reference (batch 4), plus operand layouts the kernels take
    without a copy: transposed matrices, one matrix broadcast over the batch, batch as the middle dim."""
    torch.manual_seed(0)
    batch = 4
    a = torch.randn(batch, M, K, dtype=dtype, device=gpu)
    b = torch.randn(batch, K, N, dtype=dtype, device=gpu)
    if layout == "b_transposed":
        b = torch.randn(batch, N, K, dtype=dtype, device=gpu).transpose(1, 2)
    elif layout == "a_transposed":
        a = torch.randn(batch, K, M, dtype=dtype, device=gpu).transpose(1, 2)
    elif layout == "broadcast_b":
        b = torch.randn(K, N, dtype=dtype, device=gpu).expand(batch, K, N)
    elif layout == "batch_inner":
        a = torch.randn(M, batch, K, dtype=dtype, device=gpu).transpose(0, 1)
        b = torch.randn(K, batch, N, dtype=dtype, device=gpu).transpose(0, 1)
    ref = O.bmm(a, b)
    with flag_gems.use_gems():
        res = torch.bmm(a, b)
    assert res.shape == (batch, M, N) and res.is_contiguous()
    gems_assert_close(res, ref, dtype, reduce_dim=K)


def test_bmm_special_cases(gpu):
    torch.manual_seed(2)
    a = torch.randn(3, 33, 40, device=gpu); b = torch.randn(3, 40, 17, device=gpu)
    # every matrix of the batch equals the 2-D product of its operands, bit for bit (same kernel, same order)
    res = flag_gems.bmm(a, b)
    for z in range(3):
        assert torch.equal(res[z], flag_gems.mm(a[z], b[z]))
    # batch of one, empty extents, K == 0
    gems_assert_close(flag_gems.bmm(a[:1], b[:1]), O.bmm(a[:1], b[:1]), torch.float32, reduce_dim=40)
    assert flag_gems.bmm(a[:0], b[:0]).shape == (0, 33, 17)
    assert flag_gems.bmm(a[:, :0], b).shape == (3, 0, 17)
    z = flag_gems.bmm(a[:, :, :0], b[:, :0])
    assert z.shape == (3, 33, 17) and not z.any()
    # dtypes the kernels do not cover stay on the vendor library, also under the override
    with flag_gems.use_gems():
        d = torch.bmm(a.double(), b.double())
        m = torch.mm(a[0].double(), b[0].double())
    assert d.dtype == torch.float64 and torch.allclose(d.cpu(), O.bmm(a, b), atol=1e-10)
    assert torch.allclose(m.cpu(), O.mm(a[0], b[0]), atol=1e-10)
    with pytest.raises(AssertionError):
        flag_gems.bmm(a, b[:2])
    # a large aligned batch on the direct-to-LDS kernels (attention-like shapes), against the oracle
    q = torch.randn(16, 512, 128, device=gpu, dtype=torch.bfloat16)
    k = torch.randn(16, 512, 128, device=gpu, dtype=torch.bfloat16)
    s = flag_gems.bmm(q, k.transpose(1, 2))
    gems_assert_close(s, O.bmm(q, k.transpose(1, 2)), torch.bfloat16, reduce_dim=128)
    v = torch.randn(16, 512, 128, device=gpu, dtype=torch.bfloat16)
    gems_assert_close(flag_gems.bmm(s, v), O.bmm(s, v), torch.bfloat16, reduce_dim=512)


def test_bmm_large_batches_stay_on_the_vendor_kernel(gpu):
    """Batches beyond the verified envelope (more than 16 matrices or 2^24 output elements) are handed to
    the vendor kernel by the wrapper; the result still has to match the oracle."""
    import importlib

    bmm_mod = importlib.import_module("flaggems_amd.ops.bmm")  # (the package attribute of that name is the function)

    assert bmm_mod._within_verified_envelope(16, 512, 512)
    assert not bmm_mod._within_verified_envelope(32, 2048, 2048)
    assert not bmm_mod._within_verified_envelope(17, 8, 8)
    torch.manual_seed(5)
    a = torch.randn(20, 96, 64, device=gpu, dtype=torch.bfloat16)
    b = torch.randn(20, 64, 40, device=gpu, dtype=torch.bfloat16)
    with flag_gems.use_gems():
        res = torch.bmm(a, b)
    gems_assert_close(res, O.bmm(a, b), torch.bfloat16, reduce_dim=64)


@pytest.mark.skip(reason="fg_bmm on 32 x 2048x2048x128 bf16 (one 128x128-tile launch per matrix, 268 MB output) once "
                         "ended in a GPU memory fault; no cause has been shown on the host, so the case is not run "
                         "on a GPU and ops.bmm routes such batches to the vendor kernel")
def test_bmm_attention_sized_batch_native(gpu):
    torch.manual_seed(6)
    a = torch.randn(32, 2048, 128, device=gpu, dtype=torch.bfloat16)
    b = torch.randn(32, 128, 2048, device=gpu, dtype=torch.bfloat16)
    from flaggems_amd import _C
    out = torch.empty(32, 2048, 2048, device=gpu, dtype=torch.bfloat16)
    rc = _C.lib().fg_bmm(a.data_ptr(), b.data_ptr(), out.data_ptr(), 32, 2048, 2048, 128, *a.stride(), *b.stride(),
                         *out.stride(), _C.dtype_id(a.dtype), _C.current_stream(gpu))
    assert rc == 0
    idx = torch.randint(0, 2048, (64,))
    gems_assert_close(out[:, idx], O.bmm(a[:, idx], b), torch.bfloat16, reduce_dim=128)


def test_addmm_special_cases(gpu):
    torch.manual_seed(1)
    a = torch.randn(33, 40, device=gpu); b = torch.randn(40, 17, device=gpu); bias = torch.randn(17, device=gpu)
    # alpha = 0: out = beta * bias exactly (fp32)
    res = flag_gems.addmm(bias, a, b, alpha=0, beta=3)
    assert torch.equal(res, (bias * 3).expand(33, 17))
    # identity B
    eye = torch.eye(40, device=gpu)
    assert torch.equal(flag_gems.mm(a, eye), a)
    # mixed dtypes promote to the higher one
    res = flag_gems.mm(a.half(), b.bfloat16())
    assert res.dtype == torch.bfloat16
    # empty and K == 0
    assert flag_gems.mm(a[:0], b).shape == (0, 17)
    assert torch.equal(flag_gems.mm(a[:, :0], b[:0]), torch.zeros(33, 17, device=gpu))
    # scalar (0-d) and column bias broadcast through zero strides
    for bb in (torch.tensor(2.0, device=gpu), torch.randn(33, 1, device=gpu)):
        gems_assert_close(flag_gems.addmm(bb, a, b), O.addmm(bb, a, b), torch.float32, reduce_dim=40)
    # dtypes without a kernel go to the vendor library and still give the right answer
    with flag_gems.use_gems():
        r64 = torch.mm(a.double(), b.double())
    assert r64.dtype == torch.float64 and torch.allclose(r64.cpu(), O.mm(a, b))


SK_CASES = [
    # (M, N, K, schedule)               skinny stream-K kernel (M <= 16) ...
    (16, 4096, 14336, _C.SCHED_AUTO), (1, 4096, 4096, _C.SCHED_AUTO), (7, 1000, 2048, _C.SCHED_AUTO),
    (16, 152, 1024, _C.SCHED_AUTO), (3, 11008, 4096, _C.SCHED_STREAM_K), (13, 128, 40960, _C.SCHED_AUTO),
    # ... few columns (every tile split between many workgroups), ragged N with several tiles per workgroup,
    # K a multiple of 8 but not of 64, K an odd multiple of 64
    (16, 24, 2048, _C.SCHED_AUTO), (2, 8200, 1024, _C.SCHED_AUTO), (5, 1000, 1032, _C.SCHED_AUTO),
    (9, 4096, 1088, _C.SCHED_AUTO),
    # ... wide outputs (32-column tiles when B = W^T): whole tiles per workgroup, split tiles, a ragged last tile
    (16, 12288, 4096, _C.SCHED_AUTO), (5, 8192, 1088, _C.SCHED_AUTO), (16, 32000, 4096, _C.SCHED_AUTO),
    (7, 8456, 2048, _C.SCHED_AUTO),
    # ... 17 to 64 rows (two and four row blocks in the LDS-staged kernel when B = W^T): narrow and wide outputs, ragged N,
    # every tile split between workgroups, K an odd multiple of 64
    (32, 4096, 4096, _C.SCHED_AUTO), (64, 8192, 4096, _C.SCHED_AUTO), (17, 1000, 2048, _C.SCHED_STREAM_K),
    (48, 8456, 1088, _C.SCHED_STREAM_K), (33, 152, 1024, _C.SCHED_STREAM_K), (64, 4096, 14336, _C.SCHED_AUTO),
    (24, 11008, 4096, _C.SCHED_AUTO), (64, 12288, 4096, _C.SCHED_AUTO),
    # ... and wide outputs with 17 to 64 rows (one copy of A per workgroup, eight column tiles in lockstep)
    (24, 32000, 4096, _C.SCHED_STREAM_K), (64, 22016, 4096, _C.SCHED_STREAM_K), (40, 9000, 1024, _C.SCHED_STREAM_K),
    # ... and the tile stream-K kernel: few tiles / ragged waves / K and M,N tails
    (384, 384, 4096, _C.SCHED_STREAM_K), (1000, 1300, 2048, _C.SCHED_STREAM_K), (2048, 2304, 1024, _C.SCHED_STREAM_K),
    (495, 5333, 71, _C.SCHED_STREAM_K), (640, 640, 8192, _C.SCHED_AUTO), (128, 128, 64, _C.SCHED_STREAM_K),
    # ... and the same schedule on the direct-to-LDS main loop (aligned operands, K a multiple of 64): less than
    # a wave of tiles (chosen automatically), ragged edges with bias, full waves in front of the shared tiles
    (512, 4096, 4096, _C.SCHED_AUTO), (256, 4096, 1024, _C.SCHED_STREAM_K), (1000, 1304, 2048, _C.SCHED_STREAM_K),
    (3000, 4104, 1024, _C.SCHED_STREAM_K), (130, 136, 64, _C.SCHED_STREAM_K),
    # ... tiles cut into equal parts on fewer workgroups than CUs (96 tiles in halves, 24 tiles in eighths, 43 K steps
    # per tile left whole), and K steps that no divisor spreads well (equal shares across tile boundaries)
    (384, 4096, 4096, _C.SCHED_STREAM_K), (384, 1024, 8192, _C.SCHED_AUTO), (1024, 2048, 2752, _C.SCHED_STREAM_K),
    (200, 1000, 2752, _C.SCHED_STREAM_K),
]


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("M,N,K,schedule", SK_CASES)
@pytest.mark.parametrize("b_col_major", [False, True])
def test_stream_k(gpu, M, N, K, schedule, dtype, b_col_major):
    torch.manual_seed(2)
    a = torch.randn(M, K, dtype=dtype, device=gpu) / K ** 0.5
    b = _operand(K, N, dtype, gpu, b_col_major) / K ** 0.5
    bias = torch.randn(N, dtype=dtype, device=gpu).broadcast_to(M, N)
    ref = O.mm(a, b) * 0.5 + bias.double().cpu() * 2.0
    c = torch.empty(M, N, dtype=dtype, device=gpu)
    _gemm.gemm(a, b, bias, c, 0.5, 2.0, schedule=schedule)
    assert _gemm.last_schedule() == _C.SCHED_STREAM_K
    gems_assert_close(c, ref, dtype, reduce_dim=K)
    # same answer as the data-parallel schedule up to fp32 re-association, and bit-identical run to run
    d = torch.empty_like(c)
    _gemm.gemm(a, b, bias, d, 0.5, 2.0, schedule=_C.SCHED_DATA_PARALLEL)
    assert _gemm.last_schedule() == _C.SCHED_DATA_PARALLEL
    gems_assert_close(d, ref, dtype, reduce_dim=K)
    for _ in range(10):
        e = torch.empty_like(c)
        _gemm.gemm(a, b, bias, e, 0.5, 2.0, schedule=schedule)
        assert torch.equal(c, e)


# The direct-to-LDS stream-K kernel normally cuts tiles into equal parts; with FG_GEMM_SK_EVEN set it deals equal
# shares of the K steps to all CUs instead, so shares cross tile boundaries (two partial tiles per workgroup,
# three or four contributors per tile).
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("M,N,K", [(384, 4096, 4096), (640, 4096, 2752), (1000, 1304, 2048), (3000, 4104, 1024), (200, 1000, 2752)])
@pytest.mark.parametrize("b_col_major", [False, True])
def test_stream_k_equal_shares(gpu, fg_env, M, N, K, dtype, b_col_major):
    fg_env.setenv("FG_GEMM_SK_EVEN", "1")
    torch.manual_seed(4)
    a = torch.randn(M, K, dtype=dtype, device=gpu) / K ** 0.5
    b = _operand(K, N, dtype, gpu, b_col_major) / K ** 0.5
    bias = torch.randn(N, dtype=dtype, device=gpu).broadcast_to(M, N)
    ref = O.mm(a, b) * 0.5 + bias.double().cpu() * 2.0
    c = torch.empty(M, N, dtype=dtype, device=gpu)
    _gemm.gemm(a, b, bias, c, 0.5, 2.0, schedule=_C.SCHED_STREAM_K)
    assert _gemm.last_schedule() == _C.SCHED_STREAM_K
    gems_assert_close(c, ref, dtype, reduce_dim=K)
    for _ in range(10):
        e = torch.empty_like(c)
        _gemm.gemm(a, b, bias, e, 0.5, 2.0, schedule=_C.SCHED_STREAM_K)
        assert torch.equal(c, e)


def test_stream_k_needs_workspace(gpu):
    a = torch.randn(8, 2048, dtype=torch.bfloat16, device=gpu); b = torch.randn(2048, 256, dtype=torch.bfloat16, device=gpu)
    c = torch.empty(8, 256, dtype=torch.bfloat16, device=gpu)
    rc = _C.lib().fg_gemm(a.data_ptr(), b.data_ptr(), None, c.data_ptr(), 8, 256, 2048, 2048, 1, 256, 1, 0, 0, 256, 1,
                          1.0, 0.0, _C.FG_BF16, _C.FG_BF16, _C.FG_BF16, _C.SCHED_STREAM_K, None, 0, None, None)
    assert rc == -4 and "workspace" in _C.last_error()


# Shapes with enough 256x256 tiles to take the direct-to-LDS kernel (first three), and neighbours that
# miss one of its preconditions (K = 72 takes its zero-padded last K step, N not a multiple of 8 the
# register-staged kernel instead); ragged M and N edges in both.
LARGE_TILE_SHAPES = [(3857, 4104, 64), (4100, 4104, 256), (4096, 4096, 192), (4096, 4096, 72), (3900, 4100, 128)]


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("M,N,K", LARGE_TILE_SHAPES)
@pytest.mark.parametrize("b_col_major", [False, True])
def test_mm_addmm_large_tiles(gpu, M, N, K, dtype, b_col_major):
    torch.manual_seed(M + K)
    a = torch.randn(M, K, dtype=dtype, device=gpu)
    b = _operand(K, N, dtype, gpu, b_col_major)
    rows = torch.tensor([0, 1, 31, 32, 127, 128, 255, 256, 2047, 2048, M - 258, M - 257, M - 2, M - 1], device=gpu)
    cols = torch.tensor([0, 7, 8, 63, 64, 255, 256, 257, N // 2, N - 257, N - 256, N - 9, N - 8, N - 1], device=gpu)
    c = flag_gems.mm(a, b)
    gems_assert_close(c[rows], O.mm(a[rows], b), dtype, reduce_dim=K)
    gems_assert_close(c[:, cols], O.mm(a, b[:, cols]), dtype, reduce_dim=K)
    for bias in (torch.randn(N, dtype=dtype, device=gpu), torch.randn(M, N, dtype=dtype, device=gpu)):
        d = flag_gems.addmm(bias, a, b, alpha=0.5, beta=2.0)
        brow = bias if bias.dim() == 1 else bias[rows]
        bcol = bias[cols] if bias.dim() == 1 else bias[:, cols]
        gems_assert_close(d[rows], O.addmm(brow, a[rows], b, alpha=0.5, beta=2.0), dtype, reduce_dim=K)
        gems_assert_close(d[:, cols], O.addmm(bcol, a, b[:, cols], alpha=0.5, beta=2.0), dtype, reduce_dim=K)
    # an output view whose row stride is not a multiple of 16 bytes (no vector stores possible)
    wide = torch.empty(M, N + 3, dtype=dtype, device=gpu)
    out = wide[:, :N]
    with flag_gems.use_gems():
        torch.mm(a, b, out=out)
    gems_assert_close(out[rows], O.mm(a[rows], b), dtype, reduce_dim=K)
    gems_assert_close(out[:, cols], O.mm(a, b[:, cols]), dtype, reduce_dim=K)


# K a multiple of 8 but not of 64: the direct-to-LDS kernels copy the chunks of the last K step that lie past K from a
# buffer of zeros.  Two to 44 K steps, 8 to 56 valid k in the last one, both tiles (the large shapes fill the machine
# with 256x256 tiles), ragged M and N edges.  The operands are views into larger tensors whose memory behind every row
# (and behind the last row) holds NaN: a chunk read from there instead of the zeros poisons its row or column.
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("M,N,K", [(300, 520, 72), (1100, 2824, 136), (2040, 1032, 1000), (513, 4104, 2744), (4100, 4104, 200),
                                   (3900, 4096, 120)])
@pytest.mark.parametrize("b_col_major", [False, True])
def test_mm_addmm_k_not_a_multiple_of_64(gpu, M, N, K, dtype, b_col_major):
    torch.manual_seed(M + K)
    pad = 64 - K % 64
    a_full = torch.full((M + 1, K + pad), float("nan"), dtype=dtype, device=gpu)
    a = a_full[:M, :K]
    a.copy_(torch.randn(M, K, device=gpu))
    if b_col_major:
        b_full = torch.full((N + 1, K + pad), float("nan"), dtype=dtype, device=gpu)
        b_full[:N, :K] = torch.randn(N, K, device=gpu).to(dtype)
        b = b_full[:N, :K].t()
    else:
        b_full = torch.full((K + pad, N), float("nan"), dtype=dtype, device=gpu)
        b_full[:K] = torch.randn(K, N, device=gpu).to(dtype)
        b = b_full[:K]
    rows = torch.tensor([0, 1, 15, 16, 127, 128, 255, 256, M // 2, M - 129, M - 2, M - 1], device=gpu)
    cols = torch.tensor([0, 7, 8, 15, 16, 255, 256, N // 2, N - 257, N - 9, N - 8, N - 1], device=gpu)
    c = flag_gems.mm(a, b)
    assert torch.isfinite(c).all()
    gems_assert_close(c[rows], O.mm(a[rows], b), dtype, reduce_dim=K)
    gems_assert_close(c[:, cols], O.mm(a, b[:, cols]), dtype, reduce_dim=K)
    bias = torch.randn(N, dtype=dtype, device=gpu)
    d = flag_gems.addmm(bias, a, b, alpha=0.5, beta=2.0)
    gems_assert_close(d[rows], O.addmm(bias, a[rows], b, alpha=0.5, beta=2.0), dtype, reduce_dim=K)
    assert torch.equal(flag_gems.mm(a, b), c)


# The direct-to-LDS kernel exists for five tile sizes; the library picks by how the tile count fills the
# machine.  Each is forced in turn on ragged shapes (edge tiles in M and N; one to four K steps, which is fewer
# than or as many as the LDS ring has stages, and seventeen) and, with no forcing, on shapes whose automatic
# choice is the 128x128 and the 256x128 tile.  The smaller tiles run with a ring of three or four stages.
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("tile", ["256x256", "192x256", "256x128", "128x256", "128x128", None])
@pytest.mark.parametrize("M,N,K", [(1024, 4096, 128), (1100, 4104, 64), (2040, 4104, 256), (1537, 2824, 192), (1100, 2824, 1088)])
@pytest.mark.parametrize("b_col_major", [False, True])
def test_mm_addmm_tile_sizes(gpu, fg_env, M, N, K, dtype, tile, b_col_major):
    if tile is None:
        fg_env.delenv("FG_GEMM_TILE", raising=False)
    else:
        fg_env.setenv("FG_GEMM_TILE", tile)
    torch.manual_seed(M + K)
    a = torch.randn(M, K, dtype=dtype, device=gpu)
    b = _operand(K, N, dtype, gpu, b_col_major)
    rows = torch.tensor([0, 1, 31, 32, 63, 64, 127, 128, 255, 256, 511, 512, M // 2, M - 130, M - 129, M - 2, M - 1], device=gpu)
    cols = torch.tensor([0, 7, 8, 63, 64, 127, 128, 255, 256, 257, N // 2, N - 137, N - 129, N - 9, N - 8, N - 1], device=gpu)
    c = flag_gems.mm(a, b)
    gems_assert_close(c[rows], O.mm(a[rows], b), dtype, reduce_dim=K)
    gems_assert_close(c[:, cols], O.mm(a, b[:, cols]), dtype, reduce_dim=K)
    bias = torch.randn(N, dtype=dtype, device=gpu)
    d = flag_gems.addmm(bias, a, b, alpha=0.5, beta=2.0)
    gems_assert_close(d[rows], O.addmm(bias, a[rows], b, alpha=0.5, beta=2.0), dtype, reduce_dim=K)
    gems_assert_close(d[:, cols], O.addmm(bias[cols], a, b[:, cols], alpha=0.5, beta=2.0), dtype, reduce_dim=K)
    # every tile size accumulates each output element over K in the same order: identical bits
    fg_env.setenv("FG_GEMM_TILE", "256x256")
    assert torch.equal(flag_gems.mm(a, b), c)


@pytest.mark.parametrize("tile", ["256x256", "128x128", None])
@pytest.mark.parametrize("M,N,K", [(8192, 8192, 64), (4096, 3072, 128), (6144, 5120, 64), (2048, 9216, 64), (4096, 11008, 64),
                                   (10240, 1024, 64), (256, 12288, 192)])
def test_mm_every_tile_is_written_once(gpu, fg_env, M, N, K, tile):
    """The workgroup id -> output tile map is a bijection on every kind of tile grid it treats differently (multiples of
    the 8 x 4 sub-blocks with whole and partial rounds, an odd number of sub-block rows, a single row of them, grids that
    are not multiples): an output pre-filled with NaN holds the whole product afterwards, checked against the oracle."""
    if tile is None:
        fg_env.delenv("FG_GEMM_TILE", raising=False)
    else:
        fg_env.setenv("FG_GEMM_TILE", tile)
    torch.manual_seed(N + K)
    dtype = torch.bfloat16
    a = torch.randn(M, K, dtype=dtype, device=gpu)
    b = _operand(K, N, dtype, gpu, True)
    c = torch.full((M, N), float("nan"), dtype=dtype, device=gpu)
    flag_gems.mm_out(a, b, out=c)
    assert not torch.isnan(c).any()
    gems_assert_close(c, O.mm(a, b), dtype, reduce_dim=K)


def test_mm_full_size_properties(gpu):
    """8192^3 bf16 (the benchmark shape): sampled rows against the oracle, plus linearity in A."""
    torch.manual_seed(3)
    n = 8192
    a = torch.randn(n, n, dtype=torch.bfloat16, device=gpu) / n ** 0.5
    b = torch.randn(n, n, dtype=torch.bfloat16, device=gpu) / n ** 0.5
    for bb in (b, b.t()):
        c = flag_gems.mm(a, bb)
        rows = torch.tensor([0, 1, 255, 256, 4095, 4097, 8190, 8191], device=gpu)
        gems_assert_close(c[rows], O.mm(a[rows], bb), torch.bfloat16, reduce_dim=n)
        # doubling A doubles C exactly (power-of-two scaling commutes with every rounding)
        assert torch.equal(flag_gems.mm(a * 2, bb), c * 2)


@pytest.mark.parametrize("b_col_major", [False, True])
def test_addmm_ffn_projection_full_size(gpu, b_col_major):
    """addmm at M=4096, N=11008, K=4096 with a [11008] bias ~ N(0, 0.02), bf16, alpha = beta = 1 (harness of the
    reference's tests/test_blas_ops.py:24-60): sampled rows and columns against the oracle, under the override."""
    torch.manual_seed(11)
    M, N, K = 4096, 11008, 4096
    dtype = torch.bfloat16
    a = (torch.randn(M, K, device=gpu) / 64).to(dtype)
    b = (torch.randn(N, K, device=gpu) / 64).to(dtype).t() if b_col_major else (torch.randn(K, N, device=gpu) / 64).to(dtype)
    bias = (torch.randn(N, device=gpu) * 0.02).to(dtype)
    with flag_gems.use_gems():
        d = torch.addmm(bias, a, b)
    assert d.shape == (M, N) and d.dtype == dtype
    rows = torch.tensor([0, 1, 191, 192, 255, 256, 2047, 2048, M - 257, M - 256, M - 2, M - 1], device=gpu)
    cols = torch.tensor([0, 7, 8, 255, 256, 257, N // 2, 10751, 10752, N - 257, N - 256, N - 9, N - 8, N - 1],
                        device=gpu)
    gems_assert_close(d[rows], O.addmm(bias, a[rows], b), dtype, reduce_dim=K)
    gems_assert_close(d[:, cols], O.addmm(bias[cols], a, b[:, cols]), dtype, reduce_dim=K)
    # the bias really is added once per column: subtracting the plain product leaves it, to bf16 rounding
    with flag_gems.use_gems():
        c = torch.mm(a, b)
    delta = (d[rows].float() - c[rows].float()).cpu()
    torch.testing.assert_close(delta, bias.float().cpu().expand_as(delta), atol=2e-2, rtol=0)


def _shifted(rows, cols, dtype, dev, transposed, shift, pad):
    """A (rows, cols) operand contiguous along cols (along rows when transposed), `shift` elements into its
    buffer and with `pad` unused elements behind every line: base and row stride only element-aligned."""
    r, c = (cols, rows) if transposed else (rows, cols)
    buf = torch.randn(shift + r * (c + pad) + 8, dtype=dtype, device=dev)
    t = buf[shift:shift + r * (c + pad)].view(r, c + pad)[:, :c]
    return t.t() if transposed else t


# Operands that are contiguous along one axis but miss the alignment of the 16-byte staging modes (K or the row
# stride not a multiple of 8 elements, a base address that is only element-aligned, ragged row counts): the
# element-aligned vector modes (also what fp32 operands that are contiguous along M or N take).
@pytest.mark.parametrize("dtype", FLOAT_DTYPES)
@pytest.mark.parametrize("M,N,K", [(300, 500, 1004), (257, 129, 71), (128, 136, 64), (1, 9, 3), (513, 1001, 130)])
@pytest.mark.parametrize("b_col_major", [False, True])
@pytest.mark.parametrize("a_col_major", [False, True])
@pytest.mark.parametrize("shift,pad", [(0, 0), (3, 5), (1, 0)])
def test_mm_unaligned_operands(gpu, M, N, K, dtype, a_col_major, b_col_major, shift, pad):
    torch.manual_seed(M + N + K + shift)
    a = _shifted(M, K, dtype, gpu, a_col_major, shift, pad)
    b = _shifted(K, N, dtype, gpu, b_col_major, shift, pad)
    ref = O.mm(a, b)
    res = flag_gems.mm(a, b)
    gems_assert_close(res, ref, dtype, reduce_dim=K)
    bias = torch.randn(N, dtype=dtype, device=gpu)
    res = flag_gems.addmm(bias, a, b, alpha=0.5, beta=2.0)
    gems_assert_close(res, O.addmm(bias, a, b, alpha=0.5, beta=2.0), dtype, reduce_dim=K)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
@pytest.mark.parametrize("rows,cols,src_pad,dst_pad", [(64, 64, 0, 0), (4096, 1024, 0, 0), (1000, 130, 0, 0), (257, 511, 3, 5),
                                                       (1, 7, 0, 0), (129, 1, 8, 8), (300, 200, 8, 16)])
def test_transpose2d(gpu, rows, cols, src_pad, dst_pad, dtype):
    """fg_transpose2d through the C ABI: bit-exact, ragged tiles, padded row strides, nothing written outside dst."""
    from flaggems_amd import _C

    torch.manual_seed(rows + cols)
    src = torch.randn(rows, cols + src_pad, dtype=dtype, device=gpu)
    dst = torch.full((cols, rows + dst_pad), 7.0, dtype=dtype, device=gpu)
    rc = _C.lib().fg_transpose2d(src.data_ptr(), dst.data_ptr(), rows, cols, cols + src_pad, rows + dst_pad,
                                 src.element_size(), _C.current_stream(src.device))
    assert rc == 0, _C.last_error()
    assert torch.equal(dst[:, :rows], src[:, :cols].t())
    assert (dst[:, rows:] == 7.0).all()
