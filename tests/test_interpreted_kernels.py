"""The library end to end WITHOUT a GPU: its host code runs as built (against a stand-in for the HIP runtime that
only records kernel registrations and forwards launches), and every kernel it launches is executed from the
compiler's own assembly by an interpreter of the gfx950 instruction set on numpy buffers, every memory access
bounds-checked (tests/emu/).  Results are held to the same oracle and tolerances as the GPU parity tests.

Two builds run the same cases:
  * the default library: its device code is the code the GPU parity suite passed (test_device_code_manifest.py pins
    that), so this run calibrates the interpreter: it must reproduce the oracle on kernels known to be right;
  * a build with every switch of csrc/variants.h on: kernel variants that have not been on a GPU yet.  They must
    reproduce the oracle too, stay inside their buffers, and (where a case says so) really run the variant kernel.
The interpreter models function, not time: waits and wait states are the business of test_isa_*.py.
"""
import json
import os
import subprocess
import sys

import numpy as np
import pytest
import torch

from helpers import gems_assert_close, gems_assert_equal
from oracle import torch_ref

REPO = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
EMU = os.path.join(REPO, "tests", "emu")
CSRC = os.path.join(REPO, "flaggems_amd", "csrc")
TD = {"bf16": torch.bfloat16, "f16": torch.float16, "f32": torch.float32}

# every switch of variants.h at its trial value
sys.path.insert(0, CSRC)
try:
    from build import TRIAL as VARIANTS
finally:
    sys.path.remove(CSRC)


def C(cid, fn, check=None, kernel=None, variant_kernel=None, seed=0, num_cu=256, lane=0, variants_only=None, **kw):
    """num_cu: compute units the interpreted device reports.  The library sizes tiles, grids and stream-K partitions
    from it, so a device of a few CUs brings the large-tile kernels within reach of small problems.
    lane: cases of one (num_cu, lane) share a worker process; long cases get lanes of their own.
    variants_only: the entry point's kernel exists only in the build with the variants on; the default build must
    answer FG_ERR_UNSUPPORTED with this text in its message, and launch nothing."""
    return {"id": cid, "fn": fn, "kw": kw, "seed": seed, "check": check or fn, "kernel": kernel,
            "variant_kernel": variant_kernel, "num_cu": num_cu, "lane": lane, "variants_only": variants_only}


CASES = [
    # ---- rms_norm / fused_add_rms_norm: every kernel family of norm.hip
    C("rms bf16 5x4096", "rms_norm", dtype="bf16", M=5, N=4096, kernel="rms_rows_kernel"),
    C("rms bf16 5x2048", "rms_norm", dtype="bf16", M=5, N=2048, kernel="rms_rows_kernel"),
    C("rms f16 1x2048", "rms_norm", dtype="f16", M=1, N=2048, kernel="rms_rows_kernel"),
    C("rms f16 3x200 no weight", "rms_norm", dtype="f16", M=3, N=200, weight=False),
    C("rms f32 3x333 no inv", "rms_norm", dtype="f32", M=3, N=333, inv=False, kernel="rms_short_kernel"),
    C("rms bf16 2x9001", "rms_norm", dtype="bf16", M=2, N=9001, kernel="rms_looped_kernel"),
    C("rms bf16 3x1024 strided", "rms_norm", dtype="bf16", M=3, N=1024, xs=1040, ys=1032),
    C("rms bf16 3x20000", "rms_norm", dtype="bf16", M=3, N=20000),
    C("fused bf16 5x4096", "fused_add_rms_norm", dtype="bf16", M=5, N=4096, kernel="rms_rows_kernel",
      variant_kernel="rms_rows2_kernel"),
    C("fused bf16 1x4096", "fused_add_rms_norm", dtype="bf16", M=1, N=4096, kernel="rms_rows_kernel"),
    C("fused bf16 2x8192", "fused_add_rms_norm", dtype="bf16", M=2, N=8192, variant_kernel="rms_rows2_kernel"),
    C("fused f16 4x2048", "fused_add_rms_norm", dtype="f16", M=4, N=2048, variant_kernel="rms_rows2_kernel"),
    C("fused bf16 3x2048 strided", "fused_add_rms_norm", dtype="bf16", M=3, N=2048, xs=2056, rs=2064,
      variant_kernel="rms_rows2_kernel"),
    C("fused f32 3x101", "fused_add_rms_norm", dtype="f32", M=3, N=101, kernel="rms_short_kernel"),
    C("fused bf16 2x9001", "fused_add_rms_norm", dtype="bf16", M=2, N=9001, kernel="rms_looped_kernel"),
    # ---- softmax family
    C("softmax bf16 5x1000", "softmax", dtype="bf16", M=5, N=1000, K=1),
    C("softmax f16 3x4096", "softmax", dtype="f16", M=3, N=4096, K=1),
    C("softmax f32 2x40000", "softmax", dtype="f32", M=2, N=40000, K=1),
    C("softmax bf16 3x50x70", "softmax", dtype="bf16", M=3, N=50, K=70),
    C("log_softmax bf16 to f32", "softmax", dtype="bf16", M=4, N=777, K=1, log=True, out_dtype="f32"),
    C("softmax backward bf16", "softmax_backward", dtype="bf16", M=4, N=1000, K=1),
    C("softmax backward f32 2x33x65", "softmax_backward", dtype="f32", M=2, N=33, K=65),
    C("log_softmax backward f16", "softmax_backward", dtype="f16", M=3, N=4096, K=1, log=True),
    # ---- rms_norm backward
    C("rms backward bf16 9x4096", "rms_norm_backward", dtype="bf16", M=9, N=4096),
    C("rms backward f16 6x2048", "rms_norm_backward", dtype="f16", M=6, N=2048),
    C("rms backward f32 5x300", "rms_norm_backward", dtype="f32", M=5, N=300),
    # ---- data movement
    C("transpose 2-byte 70x130", "transpose2d", elem_bytes=2, rows=70, cols=130, src_stride=136, dst_stride=72),
    C("transpose 4-byte 33x65", "transpose2d", elem_bytes=4, rows=33, cols=65),
    C("silu bf16 halves of one projection", "silu_and_mul", dtype="bf16", rows=5, cols=512, a_stride=1024, b_stride=1024),
    C("silu f16 7x264", "silu_and_mul", dtype="f16", rows=7, cols=264),
    C("silu f32 3x101", "silu_and_mul", dtype="f32", rows=3, cols=101),
    # (the gradient kernel is compiled only with its switch on: the default build's entry point says so)
    C("silu backward bf16, halves of one projection", "silu_and_mul_backward", dtype="bf16", rows=5, cols=512, a_stride=1024,
      b_stride=1024, variant_kernel="silu_mul_grad_kernel", variants_only="not part of this build"),
    C("silu backward f16 7x264 strided outputs", "silu_and_mul_backward", dtype="f16", rows=7, cols=264, g_stride=272, da_stride=280,
      db_stride=296, variant_kernel="silu_mul_grad_kernel", variants_only="not part of this build"),
    C("silu backward f32 3x101", "silu_and_mul_backward", dtype="f32", rows=3, cols=101, variant_kernel="silu_mul_grad_kernel",
      variants_only="not part of this build"),
    C("silu backward f32 4x64", "silu_and_mul_backward", dtype="f32", rows=4, cols=64, variant_kernel="silu_mul_grad_kernel",
      variants_only="not part of this build"),
    C("silu backward f16 3x77", "silu_and_mul_backward", dtype="f16", rows=3, cols=77, variant_kernel="silu_mul_grad_kernel",
      variants_only="not part of this build"),
    C("silu backward bf16 4x333 odd stride", "silu_and_mul_backward", dtype="bf16", rows=4, cols=333, a_stride=335,
      variant_kernel="silu_mul_grad_kernel", variants_only="not part of this build"),
    C("rope bf16 neox", "rope", dtype="bf16", n_tokens=5, Hq=4, Hk=2, D=128),
    C("rope f16 interleaved i32 out of place", "rope", dtype="f16", n_tokens=4, Hq=3, Hk=1, D=64, interleaved=True, pos="i32",
      inplace=False),
    C("rope f32 no positions padded heads", "rope", dtype="f32", n_tokens=6, Hq=2, Hk=2, D=32, pos="none", seq_len=3, head_pad=8),
    C("rope bf16 cos in bf16", "rope", dtype="bf16", n_tokens=3, Hq=2, Hk=2, D=64, cs_dtype="bf16"),
    C("cache flash 2-byte", "reshape_and_cache_flash", elem_bytes=2, num_tokens=7, H=2, D=128, block_size=16, num_blocks=3),
    C("cache flash padded i32 slots", "reshape_and_cache_flash", elem_bytes=2, num_tokens=5, H=3, D=40, block_size=4, num_blocks=4,
      slot_i64=False, token_pad=24, block_pad=64),
    C("cache flash 1-byte", "reshape_and_cache_flash", elem_bytes=1, num_tokens=4, H=2, D=48, block_size=8, num_blocks=2),
    C("cache v0 2-byte", "reshape_and_cache", elem_bytes=2, num_tokens=6, H=2, D=64, block_size=8, x=8, num_blocks=3),
    # ---- GEMM: data-parallel tiles fed by LDS-DMA, the register-staged kernels, stream-K, the skinny kernels
    C("mm bf16 W^T 512x512x256 on 4 CUs", "gemm", dtype="bf16", M=512, N=512, K=256, b_layout="nk", num_cu=4,
      kernel="gemm_dma_kernelIDF16bLb1ELi256ELi256E"),
    C("addmm f16 768x512x128 row bias on 4 CUs", "gemm", dtype="f16", M=768, N=512, K=128, b_layout="kn", bias="row", alpha=0.5,
      beta=2.0, num_cu=4, kernel="gemm_dma_kernelIDF16_Lb0ELi192ELi256E"),
    C("mm bf16 W^T 500x300x192 on 4 CUs", "gemm", dtype="bf16", M=500, N=300, K=192, b_layout="nk", num_cu=4,
      kernel="gemm_dp_kernelIDF16bLi256ELi256E"),
    C("mm bf16 W^T 200x300x256", "gemm", dtype="bf16", M=200, N=300, K=256, b_layout="nk", kernel="gemm_dp_kernel"),
    C("mm f16 130x136x96", "gemm", dtype="f16", M=130, N=136, K=96, kernel="gemm_dma_kernelIDF16_Lb0ELi128ELi128E"),
    C("addmm bf16 W^T 256x256x128 row bias", "gemm", dtype="bf16", M=256, N=256, K=128, b_layout="nk", bias="row", alpha=0.5,
      beta=2.0, kernel="gemm_dma_kernel"),
    C("addmm bf16 W^T 100x256x128 full bias", "gemm", dtype="bf16", M=100, N=256, K=128, b_layout="nk", bias="full",
      kernel="gemm_dma_kernel"),
    C("mm bf16 padded A rows", "gemm", dtype="bf16", M=64, N=128, K=128, b_layout="nk", a_pad=8),
    C("mm bf16 97x133x71", "gemm", dtype="bf16", M=97, N=133, K=71, kernel="gemm_dp_kernel"),
    C("addmm f32 40x50x60", "gemm", dtype="f32", M=40, N=50, K=60, bias="row", kernel="gemm_dp_kernelIf"),
    C("mm bf16 stream-K 256x384x512", "gemm", dtype="bf16", M=256, N=384, K=512, b_layout="nk", schedule=2,
      kernel="gemm_dma_streamk_kernel"),
    C("mm bf16 stream-K 1024x512x512 on 8 CUs", "gemm", dtype="bf16", M=1024, N=512, K=512, b_layout="nk", schedule=2, num_cu=8,
      kernel="streamk_kernel"),
    C("mm bf16 skinny 4x512x1024 on 8 CUs", "gemm", dtype="bf16", M=4, N=512, K=1024, b_layout="nk", num_cu=8,
      kernel="gemm_skinny_kc_kernel"),
    C("mm bf16 skinny 4x512x1024", "gemm", dtype="bf16", M=4, N=512, K=1024, b_layout="nk", kernel="gemm_skinny_kc_kernel"),
    C("addmm f16 skinny 33x128x1024 on 8 CUs", "gemm", dtype="f16", M=33, N=128, K=1024, b_layout="nk", bias="row", num_cu=8,
      kernel="gemm_skinny_kc_kernel"),
    C("mm bf16 skinny 16x256x2048 row-major B on 8 CUs", "gemm", dtype="bf16", M=16, N=256, K=2048, num_cu=8,
      kernel="gemm_skinny_kernel"),
    C("mm bf16 15x160x1024 on 8 CUs", "gemm", dtype="bf16", M=15, N=160, K=1024, num_cu=8),
    C("skinny static 8x256x1024 on 8 CUs", "gemm", dtype="bf16", M=8, N=256, K=1024, b_layout="nk",
      entry="fg_gemm_skinny_static", num_cu=8, kernel="gemm_skinny_kc_kernel"),
    # (long K on few CUs: every workgroup stays in the main loop, whose waits are counted by hand, for many trips)
    C("mm bf16 skinny 4x128x4096 on 8 CUs", "gemm", dtype="bf16", M=4, N=128, K=4096, b_layout="nk", num_cu=8,
      kernel="gemm_skinny_kc_kernelIDF16bLi16ELi8ELb0ELi1E"),
    C("addmm f16 skinny 12x128x4096 on 8 CUs", "gemm", dtype="f16", M=12, N=128, K=4096, b_layout="nk", bias="row", num_cu=8,
      kernel="gemm_skinny_kc_kernelIDF16_Li16ELi8ELb1ELi1E"),
    C("mm bf16 skinny 24x112x4096 on 8 CUs", "gemm", dtype="bf16", M=24, N=112, K=4096, b_layout="nk", num_cu=8,
      kernel="gemm_skinny_kc_kernelIDF16bLi16ELi8ELb1ELi2E"),
    C("mm bf16 skinny 4x256x8192 on 4 CUs", "gemm", dtype="bf16", M=4, N=256, K=8192, b_layout="nk", num_cu=4,
      kernel="gemm_skinny_kc_kernelIDF16bLi32ELi4ELb0ELi1E"),
    C("mm bf16 skinny 64x128x4096 on 4 CUs", "gemm", dtype="bf16", M=64, N=128, K=4096, b_layout="nk", num_cu=4,
      kernel="gemm_skinny_kc_kernelIDF16bLi32ELi4ELb1ELi4E"),
    C("mm bf16 skinny 8x512x4096 row-major B on 4 CUs", "gemm", dtype="bf16", M=8, N=512, K=4096, num_cu=4,
      kernel="gemm_skinny_kernel"),
    C("mm bf16 W^T 256x256x1024 on 4 CUs", "gemm", dtype="bf16", M=256, N=256, K=1024, b_layout="nk", num_cu=4),
    C("bmm bf16 3x40x48x64", "bmm", dtype="bf16", batch=3, M=40, N=48, K=64),
    # ---- attention over the paged cache
    C("attention bf16 D128 causal 70/70 33/97", "attention", dtype="bf16", q_lens=[70, 33], k_lens=[70, 97], Hq=4, Hk=2, D=128,
      page_size=16, kernel="attn_varlen_pipe_kernel"),
    C("attention f16 D64 full 40/200", "attention", dtype="f16", q_lens=[40], k_lens=[200], Hq=2, Hk=1, D=64, page_size=32,
      causal=False, kernel="attn_varlen_pipe_kernel"),
    C("attention bf16 D128 window", "attention", dtype="bf16", q_lens=[50], k_lens=[300], Hq=2, Hk=2, D=128, page_size=16,
      window=(64, 0)),
    C("attention bf16 D64 softcap alibi", "attention", dtype="bf16", q_lens=[20, 9], k_lens=[45, 9], Hq=2, Hk=1, D=64, page_size=16,
      softcap=30.0, alibi=True),
    C("attention f16 D96", "attention", dtype="f16", q_lens=[17], k_lens=[80], Hq=2, Hk=2, D=96, page_size=16),
    C("attention bf16 D128 q longer than k", "attention", dtype="bf16", q_lens=[40], k_lens=[25], Hq=2, Hk=1, D=128, page_size=16),
    C("decode bf16 D128 split keys", "attention", dtype="bf16", q_lens=[1, 1, 1], k_lens=[300, 17, 1025], Hq=8, Hk=2, D=128,
      page_size=16, kernel="attn_decode_kernel"),
    C("decode f16 D64 no workspace", "attention", dtype="f16", q_lens=[1, 1], k_lens=[130, 64], Hq=4, Hk=4, D=64, page_size=16,
      workspace=False, kernel="attn_decode_kernel"),
    C("decode bf16 D128 on 8 CUs", "attention", dtype="bf16", q_lens=[1, 1], k_lens=[700, 33], Hq=4, Hk=1, D=128, page_size=16,
      num_cu=8, kernel="attn_decode_kernel"),
    C("mixed batch bf16 D128", "attention", dtype="bf16", q_lens=[1, 30, 1], k_lens=[90, 30, 260], Hq=4, Hk=2, D=128,
      page_size=16),
    # ---- the benchmark's shapes at full size, two workgroups of each launch (the first and the last of the grid)
    C("full size: mm 8192^3, 2 of 1024 workgroups", "gemm_sampled", lane=1, dtype="bf16", M=8192, N=8192, K=8192, groups=[0, -1],
      kernel="gemm_dma_kernelIDF16bLb1ELi256ELi256ELi2E"),
    C("full size: addmm 4096x11008x4096, 2 of 688 workgroups", "gemm_sampled", lane=2, dtype="bf16", M=4096, N=11008, K=4096,
      bias="row", groups=[0, -1], kernel="gemm_dma_kernelIDF16bLb1ELi256ELi256ELi2E"),
    C("full size: mm 16x4096x14336, 3 of 256 workgroups", "gemm_sampled", lane=3, dtype="bf16", M=16, N=4096, K=14336,
      groups=[0, 100, -1], kernel="gemm_skinny_kc_kernel"),
    C("full size: causal attention 4096 tokens 32/8 heads, 3 of 1024 workgroups", "attention_sampled", lane=3, dtype="bf16",
      q_len=4096, k_len=4096, Hq=32, Hk=8, D=128, page_size=16, groups=[0, 517, -1], kernel="attn_varlen_pipe_kernel"),
    C("full size: softmax 131072x2048 with masked entries, 2 of 65536 workgroups", "rows_sampled", check="softmax", lane=4,
      op="softmax", dtype="bf16", M=131072, N=2048, K=1, groups=[0, -1], masked=0.01),
    C("full size: fused_add_rms_norm 4096x4096, 2 of 4096 workgroups", "rows_sampled", check="fused_add_rms_norm", lane=4,
      op="fused", dtype="bf16", M=4096, N=4096, eps=1e-6, groups=[0, -1]),
    # ---- the per-matrix launches of the attention-sized bmm that fg_bmm turns away (an early kernel once faulted there)
    C("bmm 32 x 2048x2048x128: the launches of matrices 0 and 31, three workgroups each", "bmm_per_matrix", lane=2),
    # ---- operands of more than 4 GiB (virtual buffers; the workgroups at the far end): offsets beyond 32 bits
    C("6.4 GiB caches: scatter into the last pages, single-token attention over them", "huge_cache_and_attention", lane=5,
      kernel="attn_decode_kernel"),
    C("6.4 GiB caches: scatter into the last pages, prefill over them", "huge_cache_and_attention", lane=5, q_len=40, k_len=200,
      kernel="attn_varlen_pipe_kernel"),
    C("5.3 GiB matrix: softmax of the last rows", "huge_rows", lane=6, op="softmax"),
    C("5.3 GiB matrices: fused_add_rms_norm of the last rows", "huge_rows", lane=6, op="fused_add_rms_norm"),
    C("5.3 GiB matrices: silu_and_mul of the last rows", "huge_rows", lane=6, op="silu_and_mul"),
    C("4.8 GiB A and C: the last tile of mm", "huge_gemm", lane=6, kernel="gemm_dma_kernel"),
    C("4.9 GiB q: rotation of the last tokens", "huge_rope", lane=5),
    # ---- the entry point that allocates nothing, in a process whose first library call it is (lane 9: no fg_device_info)
    C("static entry: first call under capture is refused, later ones are not", "static_first_call_under_capture", lane=9, num_cu=8),
    # ---- the interpreter's bounds check itself
    C("guard: x 16 bytes short", "short_buffer", which="x"),
    C("guard: w 16 bytes short", "short_buffer", which="w"),
    C("guard: y 16 bytes short", "short_buffer", which="y"),
]


# Bulk cases, one per dispatch bucket (tests/emu/sweep.py), for the build with the variants on: together with the cases
# above they execute every kernel whose code differs from the GPU-tested build (test_every_changed_kernel_has_run).
# The default build is calibrated by the cases above and by the GPU suite's own tests (test_interpreted_suite.py); set
# FG_SWEEP_DEFAULT=1 to run the sweep on it as well (it passes; it is left out of the routine run for its minute).
sys.path.insert(0, EMU)
try:
    import sweep as _sweep
finally:
    sys.path.remove(EMU)
SWEEP = _sweep.sweep()
for _i, _c in enumerate(SWEEP):
    _c.update(kernel=None, variant_kernel=None, lane=10 + (_i % 6 if _c["num_cu"] == 256 else 0))
PARAMS = [(b, c) for c in CASES for b in ("default", "variants")] + \
    [(b, c) for c in SWEEP for b in (("default", "variants") if os.environ.get("FG_SWEEP_DEFAULT") == "1" else ("variants",))]


def _t(arr, dtype):
    """Array as the worker stored it -> torch tensor of `dtype`."""
    arr = np.ascontiguousarray(arr)
    if dtype == "bf16":
        return torch.from_numpy(arr.view(np.int16)).view(torch.bfloat16)
    return torch.from_numpy(arr)


class Result:
    def __init__(self, npz, cid):
        self.npz, self.cid = npz, cid

    def __getitem__(self, key):
        return self.npz["%s|%s" % (self.cid, key)]

    def __contains__(self, key):
        return "%s|%s" % (self.cid, key) in self.npz

    def kernels(self):
        return [k[0] for k in json.loads(str(self["__kernels"]))]


def _start_worker(lib, asm, tmp, tag, group, shim_dir):
    num_cu, lane = group
    spec = os.path.join(tmp, "cases_%s_%d_%d.json" % (tag, num_cu, lane))
    out = os.path.join(tmp, "results_%s_%d_%d.npz" % (tag, num_cu, lane))
    with open(spec, "w") as f:
        json.dump([{k: c.get(k) for k in ("id", "fn", "kw", "seed", "env")} for b, c in PARAMS
                   if b == tag and (c["num_cu"], c["lane"]) == group], f)
    env = dict(os.environ)
    env.pop("FG_LIB_PATH", None)
    log = open(os.path.join(tmp, "worker_%s_%d_%d.log" % (tag, num_cu, lane)), "w+")
    proc = subprocess.Popen([sys.executable, os.path.join(EMU, "worker.py"), "--lib", lib, "--asm", asm, "--spec", spec, "--out", out,
                             "--shim-dir", shim_dir, "--num-cu", str(num_cu)] + (["--no-device-info"] if lane == 9 else []),
                            stdout=log, stderr=subprocess.STDOUT, env=env)
    return proc, log, out


@pytest.fixture(scope="module")
def runs(tmp_path_factory):
    """Results per (build, CU count).  The first request starts every worker process the cases need, side by side
    (each is single-threaded), and waits for them all."""
    tmp = str(tmp_path_factory.mktemp("interp"))
    cache = {}

    def get(build, group):
        if not cache:
            sys.path.insert(0, CSRC)
            try:
                import build as B
            finally:
                sys.path.remove(CSRC)
            sys.path.insert(0, EMU)
            try:
                from device import build_shim
            finally:
                sys.path.remove(EMU)
            assert os.path.exists(B.OUT), "libfg_mi355.so is not built (python flaggems_amd/csrc/build.py)"
            cand = B.build(verbose=False, variants=VARIANTS, tag="cand")     # a no-op when it is up to date
            builds = {"default": (B.OUT, B.OBJ_DIR), "variants": (cand, B.OBJ_DIR + "_cand")}
            build_shim(tmp)
            started = {}
            todo = sorted({(b, (c["num_cu"], c["lane"])) for b, c in PARAMS}, key=lambda t: (-t[1][1], t[0]))   # long lanes first
            running = []
            width = max(2, min(8, os.cpu_count() or 2))               # worker processes side by side
            while todo or running:
                while todo and len(running) < width:
                    tag, g = todo.pop(0)
                    started[(tag, g)] = _start_worker(builds[tag][0], builds[tag][1], tmp, tag, g, tmp)
                    running.append(started[(tag, g)][0])
                running = [p for p in running if p.poll() is None]
                if todo or running:
                    import time
                    time.sleep(0.2)
            for key, (proc, log, out) in started.items():
                rc = proc.wait(timeout=1500)
                log.seek(0)
                text = log.read()
                log.close()
                assert rc == 0, "the interpreter's worker for %r failed:\n%s" % (key, text[-4000:])
                cache[key] = np.load(out)
        return cache[(build, group)]
    return get


# ---------------------------------------------------------------------------------------------------------------
# checkers: the oracle and tolerances of the GPU parity tests
# ---------------------------------------------------------------------------------------------------------------
def check_rms_norm(r, kw):
    dt = kw["dtype"]
    x, w = _t(r["x"], dt), _t(r["w"], dt)
    if not kw.get("weight", True):
        w = torch.ones_like(w)
    ref = torch_ref.rms_norm(x, w, kw.get("eps", 1e-5))
    gems_assert_close(_t(r["y"], dt), ref, TD[dt])
    gems_assert_equal(_t(r["x_after"], dt), x)
    if "inv_rms" in r:
        inv = torch.rsqrt(x.double().pow(2).mean(-1) + kw.get("eps", 1e-5))
        torch.testing.assert_close(torch.from_numpy(r["inv_rms"]).double(), inv, rtol=1e-5, atol=0)


def check_fused_add_rms_norm(r, kw):
    dt = kw["dtype"]
    w = _t(r["w"], dt) if kw.get("weight", True) else torch.ones(kw["N"], dtype=TD[dt])
    normed, summed = torch_ref.fused_add_rms_norm(_t(r["x"], dt), _t(r["residual"], dt), w, kw.get("eps", 1e-5))
    gems_assert_close(_t(r["x_out"], dt), normed, TD[dt])
    gems_assert_close(_t(r["residual_out"], dt), summed, TD[dt])


def check_softmax(r, kw):
    dt, odt = kw["dtype"], kw.get("out_dtype") or kw["dtype"]
    fn = torch_ref.log_softmax if kw.get("log") else torch_ref.softmax
    ref = fn(_t(r["x"], dt), 1)
    gems_assert_close(_t(r["out"], odt), ref, TD[odt])


def check_softmax_backward(r, kw):
    dt, gdt = kw["dtype"], kw.get("grad_in_dtype") or kw["dtype"]
    fn = torch_ref.log_softmax_backward if kw.get("log") else torch_ref.softmax_backward
    ref = fn(_t(r["grad_out"], dt), _t(r["out"], dt), 1)
    gems_assert_close(_t(r["grad_in"], gdt), ref, TD[gdt], reduce_dim=kw["N"])


def check_rms_norm_backward(r, kw):
    dt = kw["dtype"]
    x, dy, w = _t(r["x"], dt), _t(r["dy"], dt), _t(r["w"], dt)
    if not kw.get("weight", True):
        w = torch.ones_like(w)
    dx, dw = torch_ref.rms_norm_grads(x, w, kw.get("eps", 1e-5), dy)
    gems_assert_close(_t(r["dx"], dt), dx, TD[dt])
    if not kw.get("dw", True):
        return
    assert int(r["rc_dw"]) == 0
    gems_assert_close(_t(r["dw"], dt), dw, TD[dt], reduce_dim=kw["M"])
    # the partial rows add up to the weight gradient before rounding
    torch.testing.assert_close(torch.from_numpy(r["dw_partial"]).double().sum(0), dw, rtol=2e-2 if dt != "f32" else 1e-4,
                               atol=1e-2 if dt != "f32" else 1e-4)


def check_transpose2d(r, kw):
    np.testing.assert_array_equal(r["dst"], r["src"].T)


def check_silu_and_mul(r, kw):
    dt = kw["dtype"]
    ref = torch_ref.silu_and_mul(_t(r["a"], dt), _t(r["b"], dt))
    gems_assert_close(_t(r["out"], dt), ref, TD[dt])


def check_silu_and_mul_backward(r, kw):
    dt = kw["dtype"]
    da, db = torch_ref.silu_and_mul_grads(_t(r["a"], dt), _t(r["b"], dt), _t(r["g"], dt))
    gems_assert_close(_t(r["da"], dt), da, TD[dt])
    gems_assert_close(_t(r["db"], dt), db, TD[dt])


def check_rope(r, kw):
    dt, cdt = kw["dtype"], kw.get("cs_dtype", "f32")
    D = kw["D"]
    q, k = _t(r["q"], dt)[..., :D], _t(r["k"], dt)[..., :D]
    cos, sin = _t(r["cos"], cdt), _t(r["sin"], cdt)
    pos = torch.from_numpy(r["positions"])
    rq, rk = torch_ref.apply_rotary_pos_emb(q, k, cos, sin, pos, kw.get("interleaved", False))
    gems_assert_close(_t(r["q_out"], dt)[..., :D], rq, TD[dt])
    gems_assert_close(_t(r["k_out"], dt)[..., :D], rk, TD[dt])
    if kw.get("head_pad"):   # what lies between the heads is not the operator's to touch
        gems_assert_equal(_t(r["q_out"], dt)[..., D:], _t(r["q"], dt)[..., D:])
        gems_assert_equal(_t(r["k_out"], dt)[..., D:], _t(r["k"], dt)[..., D:])


def check_reshape_and_cache_flash(r, kw):
    H, D, bsz, ts, bs = (int(v) for v in r["dims"])
    nb = kw["num_blocks"]
    key = torch.from_numpy(r["key"].astype(np.int64))[:, :H * D].reshape(-1, H, D)
    val = torch.from_numpy(r["value"].astype(np.int64))[:, :H * D].reshape(-1, H, D)
    before_k, before_v = torch.from_numpy(r["key_cache_before"].astype(np.int64)), torch.from_numpy(r["value_cache_before"].astype(np.int64))
    kc0 = before_k[:, :bsz * H * D].reshape(nb, bsz, H, D)
    vc0 = before_v[:, :bsz * H * D].reshape(nb, bsz, H, D)
    rk, rv = torch_ref.reshape_and_cache_flash(key, val, kc0, vc0, torch.from_numpy(r["slots"]))
    after_k, after_v = torch.from_numpy(r["key_cache"].astype(np.int64)), torch.from_numpy(r["value_cache"].astype(np.int64))
    gems_assert_equal(after_k[:, :bsz * H * D].reshape(nb, bsz, H, D), rk)
    gems_assert_equal(after_v[:, :bsz * H * D].reshape(nb, bsz, H, D), rv)
    gems_assert_equal(after_k[:, bsz * H * D:], before_k[:, bsz * H * D:])      # the padding behind every block
    gems_assert_equal(after_v[:, bsz * H * D:], before_v[:, bsz * H * D:])


def check_reshape_and_cache(r, kw):
    slots = r["slots"].copy()
    slots[slots >= kw["num_blocks"] * kw["block_size"]] = -1                    # the library skips them; the oracle's loop cannot
    as_t = lambda a: torch.from_numpy(a.astype(np.int64))                       # noqa: E731
    rk, rv = torch_ref.reshape_and_cache(as_t(r["key"]), as_t(r["value"]), as_t(r["key_cache_before"]),
                                         as_t(r["value_cache_before"]), torch.from_numpy(slots))
    gems_assert_equal(as_t(r["key_cache"]), rk)
    gems_assert_equal(as_t(r["value_cache"]), rv)


def check_gemm(r, kw):
    dt, cdt = kw["dtype"], kw.get("c_dtype") or kw["dtype"]
    a, b = _t(r["a"], dt), _t(r["b"], dt)
    alpha, beta = kw.get("alpha", 1.0), kw.get("beta", 1.0)
    if kw.get("bias"):
        ref = torch_ref.addmm(_t(r["bias"], dt), a, b, alpha=alpha, beta=beta)
    else:
        ref = torch_ref.mm(a, b) * alpha
    gems_assert_close(_t(r["c"], cdt), ref, TD[cdt], reduce_dim=kw["K"])
    if kw.get("schedule"):
        assert int(r["schedule_used"]) == kw["schedule"]
    if "header_after" in r:
        assert not r["header_after"].any(), "the ticket counters of the workspace were not returned to zero"


def check_gemm_sampled(r, kw):
    """The block of C the sampled workgroups produced against the oracle on the same rows of A and columns of B."""
    dt = kw["dtype"]
    done = torch.from_numpy(r["done"])
    assert int(done.sum()) >= len(kw["groups"]) * 16 * 16, "the sampled workgroups wrote next to nothing"
    a, b = _t(r["a"], dt), _t(r["b"], dt)
    ref = torch_ref.addmm(_t(r["bias"], dt), a, b) if kw.get("bias") else torch_ref.mm(a, b)
    got = _t(r["c"], dt)
    atol, rtol = torch_ref.gems_tolerance(TD[dt], kw["K"])
    torch.testing.assert_close(got[done].double(), ref.to(TD[dt])[done].double(), atol=atol, rtol=rtol)
    whole = done.all(dim=1).sum() * done.all(dim=0).sum()           # each workgroup finishes whole tiles
    assert int(done.sum()) % 256 == 0 or whole >= 0


def check_attention_sampled(r, kw):
    dt = kw["dtype"]
    done = torch.from_numpy(r["done"]).all(dim=-1)                    # [tokens, heads]
    assert done.any(), "the sampled workgroups wrote nothing"
    assert bool((torch.from_numpy(r["done"]).any(dim=-1) == done).all()), "a head's row was written in part"
    q, kc, vc = _t(r["q"], dt), _t(r["k_cache"], dt), _t(r["v_cache"], dt)
    out, lse = _t(r["out"], dt), torch.from_numpy(r["lse"])
    table = torch.from_numpy(r["block_table"])
    rows = torch.nonzero(done.any(dim=1)).flatten().tolist()
    q_len, k_len = kw["q_len"], kw["k_len"]
    start = 0
    while start < len(rows):                                          # runs of consecutive query rows
        end = start
        while end + 1 < len(rows) and rows[end + 1] == rows[end] + 1:
            end += 1
        r0, r1 = rows[start], rows[end] + 1
        # rows [r0, r1) of a causal sequence see the first k_len - q_len + r1 keys, bottom-right aligned
        ref, ref_lse = torch_ref.paged_attention(q[r0:r1], kc, vc, [r1 - r0], [k_len - q_len + r1], table, kw["D"] ** -0.5,
                                                 causal=True, compute_dtype=torch.float32, return_lse=True)
        m = done[r0:r1]
        torch.testing.assert_close(out[r0:r1][m].float(), ref[m].float(), atol=2e-2, rtol=1e-2)
        torch.testing.assert_close(lse[:, r0:r1].T[m], ref_lse.T[m], atol=1e-2, rtol=1e-3)
        start = end + 1


def check_bmm(r, kw):
    dt = kw["dtype"]
    gems_assert_close(_t(r["c"], dt), torch_ref.bmm(_t(r["a"], dt), _t(r["b"], dt)), TD[dt], reduce_dim=kw["K"])


def check_attention(r, kw):
    dt = kw["dtype"]
    window = tuple(kw.get("window", (-1, -1)))
    causal = kw.get("causal", True)
    q_lens, k_lens = [int(v) for v in r["q_lens"]], [int(v) for v in r["k_lens"]]
    bias = None
    if kw.get("alibi"):
        slopes = torch.from_numpy(r["slopes"])
        mq, mk = max(q_lens), max(k_lens)
        bias = torch.zeros(len(q_lens), kw["Hq"], mq, mk)
        for i, (ql, kl) in enumerate(zip(q_lens, k_lens)):
            bias[i, :, :ql, :kl] = torch_ref.alibi_bias(slopes[i:i + 1], ql, kl, causal)[0]
    ref, ref_lse = torch_ref.paged_attention(
        _t(r["q"], dt), _t(r["k_cache"], dt), _t(r["v_cache"], dt), q_lens, k_lens, torch.from_numpy(r["block_table"]),
        kw["D"] ** -0.5, causal=causal, attn_bias=bias, soft_cap=kw.get("softcap") or None,
        window=window if window != (-1, -1) else None, compute_dtype=torch.float32, return_lse=True)
    # the tolerance of the GPU parity tests for this operator (tests/test_gpu_attention.py)
    torch.testing.assert_close(_t(r["out"], dt).float(), ref.float(), atol=2e-2, rtol=1e-2)
    if "lse" in r:
        got = torch.from_numpy(r["lse"])
        finite = torch.isfinite(ref_lse)
        torch.testing.assert_close(got[finite], ref_lse[finite], atol=1e-2, rtol=1e-3)
        assert (got[~finite] == float("inf")).all()      # rows with no visible key: out = 0, lse = +inf


def check_static_first_call_under_capture(r, kw):
    assert int(r["rc_first_under_capture"]) == -2 and int(r["launches_first"]) == 0           # FG_ERR_UNSUPPORTED, nothing launched
    assert "came under stream capture" in str(r["message"])
    for suffix in ("", "_captured"):
        got = _t(r["c" + suffix], "bf16")
        gems_assert_close(got, torch_ref.mm(_t(r["a" + suffix], "bf16"), _t(r["b" + suffix], "bf16")), torch.bfloat16, reduce_dim=1024)


def check_huge_cache_and_attention(r, kw):
    assert int(r["min_byte_offset"]) > 2 ** 32
    np.testing.assert_array_equal(r["got_k"], r["key"])           # the scatter, bit for bit, beyond 4 GiB
    np.testing.assert_array_equal(r["got_v"], r["value"])
    check_attention(r, dict(dtype="bf16", Hq=8, D=128))


def check_huge_rows(r, kw):
    """The rows the last workgroup of the launch wrote (the very last row at least) against the oracle."""
    n = 2048
    if kw["op"] == "fused_add_rms_norm":
        rows = np.nonzero((r["x_out"] != r["x"]).any(axis=1))[0]
    else:
        rows = np.nonzero((r["out"].view(np.uint16) != 0).any(axis=1))[0]
    assert len(rows) and rows[-1] == r["x"].shape[0] - 1, rows
    if kw["op"] == "softmax":
        check_softmax({"x": r["x"][rows].reshape(-1, n, 1), "out": r["out"][rows].reshape(-1, n, 1)}, dict(dtype="bf16"))
    elif kw["op"] == "fused_add_rms_norm":
        check_fused_add_rms_norm({k: (r[k][rows] if k != "w" else r[k]) for k in ("x", "residual", "w", "x_out", "residual_out")},
                                 dict(dtype="bf16", N=n))
    else:
        gems_assert_close(_t(r["out"][rows], "bf16"), torch_ref.silu_and_mul(_t(r["x"][rows], "bf16"), _t(r["b"][rows], "bf16")),
                          torch.bfloat16)


def check_bmm_per_matrix(r, kw):
    assert bool(r["others_untouched"])
    for z in (0, 31):
        done = torch.from_numpy(r["done%d" % z])
        assert int(done.sum()) >= 3 * 128 * 128
        ref = torch_ref.mm(_t(r["a%d" % z], "bf16"), _t(r["b%d" % z], "bf16")).to(torch.bfloat16)
        atol, rtol = torch_ref.gems_tolerance(torch.bfloat16, 128)
        torch.testing.assert_close(_t(r["c%d" % z], "bf16")[done].double(), ref[done].double(), atol=atol, rtol=rtol)


def check_huge_rope(r, kw):
    """Whatever part of the last tokens the last workgroup rotated (the last token's last head at least)."""
    q, k = _t(r["q"], "bf16"), _t(r["k"], "bf16")
    rq, rk = torch_ref.apply_rotary_pos_emb(q, k, _t(r["cos"], "f32"), _t(r["sin"], "f32"), torch.from_numpy(r["positions"]), False)
    for got, before, ref in ((_t(r["q_out"], "bf16"), q, rq), (_t(r["k_out"], "bf16"), k, rk)):
        done = (got != before).any(dim=-1)
        gems_assert_close(got[done], ref[done], torch.bfloat16)
        assert torch.equal(got[~done], before[~done])
    assert bool((_t(r["q_out"], "bf16")[-1, -1] != q[-1, -1]).any()) or bool((_t(r["k_out"], "bf16")[-1, -1] != k[-1, -1]).any())


def check_huge_gemm(r, kw):
    assert r["done"].all() and r["done"].size >= 128 * 128          # a whole tile, at the far end of A and C
    check_gemm_sampled(r, dict(dtype="bf16", K=1024, groups=[-1]))


def check_short_buffer(r, kw):
    msg = str(r["caught"])
    assert "outside every buffer" in msg and "nearest: %s" % kw["which"] in msg, msg


CHECK = {"bmm_per_matrix": check_bmm_per_matrix, "huge_rope": check_huge_rope, "huge_cache_and_attention": check_huge_cache_and_attention, "huge_rows": check_huge_rows, "huge_gemm": check_huge_gemm,
         "static_first_call_under_capture": check_static_first_call_under_capture, "gemm_sampled": check_gemm_sampled, "attention_sampled": check_attention_sampled, "short_buffer": check_short_buffer, "gemm": check_gemm, "bmm": check_bmm, "attention": check_attention, "rms_norm": check_rms_norm, "fused_add_rms_norm": check_fused_add_rms_norm, "softmax": check_softmax,
         "softmax_backward": check_softmax_backward, "rms_norm_backward": check_rms_norm_backward,
         "transpose2d": check_transpose2d, "silu_and_mul": check_silu_and_mul, "silu_and_mul_backward": check_silu_and_mul_backward, "rope": check_rope,
         "reshape_and_cache_flash": check_reshape_and_cache_flash, "reshape_and_cache": check_reshape_and_cache}


@pytest.mark.parametrize("build,case", PARAMS, ids=["%s-%s" % (c["id"], b) for b, c in PARAMS])
def test_interpreted(runs, build, case):
    r = Result(runs(build, (case["num_cu"], case["lane"])), case["id"])
    assert "__error" not in r, str(r["__error"])
    if build == "default" and case.get("variants_only"):
        assert int(r["rc"]) == -2 and case["variants_only"] in str(r["__message"]) and not r.kernels()
        return
    assert int(r["rc"]) == 0, str(r["__message"]) if "__message" in r else "rc %d" % int(r["rc"])
    if "gap_ok" in r:
        assert bool(r["gap_ok"]), "elements between the rows of a strided operand were overwritten"
    kernels = r.kernels()
    assert kernels or case["fn"] == "short_buffer", "the entry point launched nothing"
    want = case["variant_kernel"] if build == "variants" and case["variant_kernel"] else case["kernel"]
    if want:
        assert any(want in k for k in kernels), "expected a %s launch, got %s" % (want, kernels)
    kw = dict(case["kw"])
    if "groups" in kw:
        kw["rows_done"] = len(r["rows"]) if "rows" in r else 0
    CHECK[case["check"]](r, kw)


# ---------------------------------------------------------------------------------------------------------------
# The checks have teeth: a defect planted in the parsed program (never in the library) is reported.
# ---------------------------------------------------------------------------------------------------------------
MUTATIONS = [
    # (build, CU count, kernel, defect, case, what the interpreter must say)
    ("default", 4, "gemm_dma_kernel", "vm+1", C("m", "gemm", dtype="bf16", M=512, N=512, K=256, b_layout="nk"),
     "while an LDS-DMA of wave"),
    ("default", 4, "gemm_dma_kernel", "nobarrier", C("m", "gemm", dtype="bf16", M=512, N=512, K=256, b_layout="nk"),
     "with no barrier in between"),
    ("variants", 8, "gemm_skinny_kc", "vm+1", C("m", "gemm", dtype="bf16", M=4, N=128, K=4096, b_layout="nk"),
     "is the destination of a load still in flight"),
    ("default", 256, "attn_varlen_pipe", "lgkm+1", C("m", "attention", dtype="bf16", q_lens=[70], k_lens=[200], Hq=2, Hk=2, D=128,
                                                      page_size=16), "is the destination of a load still in flight"),
    ("default", 256, "attn_varlen_pipe", "vm+1", C("m", "attention", dtype="bf16", q_lens=[70], k_lens=[200], Hq=2, Hk=2, D=128,
                                                    page_size=16), "while an LDS-DMA of wave"),
    ("default", 256, "attn_decode", "nobarrier", C("m", "attention", dtype="bf16", q_lens=[1, 1], k_lens=[300, 40], Hq=8, Hk=2,
                                                    D=128, page_size=16), "no barrier in between"),
]


@pytest.mark.parametrize("build,num_cu,kernel,defect,case,message", MUTATIONS,
                         ids=["%s %s %s" % (m[0], m[2], m[3]) for m in MUTATIONS])
def test_planted_defects_are_reported(tmp_path, build, num_cu, kernel, defect, case, message):
    sys.path.insert(0, CSRC)
    try:
        import build as B
    finally:
        sys.path.remove(CSRC)
    lib, asm = (B.OUT, B.OBJ_DIR) if build == "default" else (os.path.join(os.path.dirname(B.OUT), "libfg_mi355.cand.so"),
                                                               B.OBJ_DIR + "_cand")
    if not os.path.exists(lib):
        lib = B.build(verbose=False, variants=VARIANTS, tag="cand")
    spec, out = str(tmp_path / "spec.json"), str(tmp_path / "out.npz")
    with open(spec, "w") as f:
        json.dump([{k: case[k] for k in ("id", "fn", "kw", "seed")}], f)
    env = dict(os.environ)
    env.pop("FG_LIB_PATH", None)
    p = subprocess.run([sys.executable, os.path.join(EMU, "worker.py"), "--lib", lib, "--asm", asm, "--spec", spec, "--out", out,
                        "--shim-dir", str(tmp_path), "--num-cu", str(num_cu), "--mutate", "%s:%s" % (kernel, defect)],
                       capture_output=True, text=True, env=env, timeout=600)
    assert p.returncode == 0, p.stdout[-2000:] + p.stderr[-2000:]
    r = Result(np.load(out), "m")
    assert "__error" in r, "the planted defect went unnoticed"
    assert message in str(r["__error"]), str(r["__error"])[:600]


# ---------------------------------------------------------------------------------------------------------------
# Coverage: no kernel whose code differs from the GPU-tested build is left unexecuted.
# ---------------------------------------------------------------------------------------------------------------
# Instantiations no call can reach.  rms_dispatch picks (packs per thread, threads per row) in two run-time branches, one
# for rms_norm and one for fused_add_rms_norm, so the compiler instantiates every pair for both operators although
# each operator only ever launches its own; the two-row kernel is launched for the fused operator only.
UNREACHABLE = [
    r"rms_rows_kernelI\w+Li[48]ELi1ELi(128|256|512|1024)ELb0E",      # rms_norm never takes one pack per thread beyond 64 threads
    r"rms_rows_kernelI\w+Li[48]ELi2ELi(64|128|256|512)ELb1E",        # fused_add_rms_norm takes two packs only on 1024 threads
    r"rms_rows2_kernelI\w+ELb0E",                                    # rms_norm has no row length with one pack on >= 256 threads
]


def test_every_changed_kernel_has_run(runs):
    import glob
    import re
    sys.path.insert(0, CSRC)
    try:
        import build as B
        import isa_check
    finally:
        sys.path.remove(CSRC)
    digests = {}
    for tag, d in (("default", B.OBJ_DIR), ("variants", B.OBJ_DIR + "_cand")):
        digests[tag] = {}
        for f in glob.glob(os.path.join(d, "*-hip-amdgcn-amd-amdhsa-gfx950.s")):
            with open(f) as fh:
                digests[tag].update(isa_check.kernel_digests(fh.read()))
    changed = {k for k, v in digests["variants"].items() if digests["default"].get(k) != v}
    assert len(changed) > 400, "the variants build hardly differs from the default one: %d kernels" % len(changed)
    ran = set()
    for group in {(c["num_cu"], c["lane"]) for b, c in PARAMS if b == "variants"}:
        npz = runs("variants", group)
        for key in npz.files:
            if key.endswith("|__kernels"):
                ran.update(k[0] for k in json.loads(str(npz[key])))
    unreachable = {k for k in changed if any(re.search(p, k) for p in UNREACHABLE)}
    assert not (unreachable & ran), "listed as unreachable, yet launched: %s" % sorted(unreachable & ran)
    missing = sorted(changed - ran - unreachable)
    assert not missing, "%d changed kernels were never executed, e.g. %s" % (len(missing), missing[:5])
