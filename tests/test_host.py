"""CPU-side tests: the drop-in boundary (registration, signatures, error behaviour) and the C ABI
loading with every symbol the header declares.  No kernel is launched here."""
import ctypes
import os
import re

import pytest
import torch

import flag_gems
import flaggems_amd
from flaggems_amd import _C

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def test_package_surface():
    assert flag_gems.device == "cuda"
    assert flag_gems.vendor_name == "amd"
    assert flag_gems.__version__
    for name in [
        "enable", "use_gems", "all_ops", "mm", "mm_out", "addmm", "addmm_out", "softmax", "rms_norm",
        "fused_add_rms_norm", "apply_rotary_pos_emb", "reshape_and_cache_flash", "silu_and_mul",
        "silu_and_mul_out", "flash_attn_varlen_func",
    ]:
        assert callable(getattr(flag_gems, name)), name
    assert flag_gems.ops.flash_attn_varlen_func is flaggems_amd.ops.flash_attn_varlen_func
    assert flag_gems.testing.assert_close and flag_gems.testing.assert_equal
    assert flag_gems.runtime.device.support_bf16 and flag_gems.runtime.device.support_fp64
    assert flag_gems.runtime.torch_device_fn is torch.cuda
    assert flag_gems.config.use_c_extension is False


def _cuda_kernel_of(op):
    table = torch._C._dispatch_dump_table(op)
    for line in table.splitlines():
        if line.startswith("CUDA:"):
            return line
    return ""


def test_use_gems_registers_and_unregisters():
    before = _cuda_kernel_of("aten::mm")
    with flag_gems.use_gems():
        assert sorted(flag_gems.all_ops()) == sorted(
            ["_flash_attention_forward", "_log_softmax", "_log_softmax_backward_data", "_softmax", "_softmax_backward_data", "addmm", "addmm.out", "bmm", "mm", "mm.out", "rms_norm"])
        inside = _cuda_kernel_of("aten::mm")
        assert "flaggems_amd" in inside
        assert "flaggems_amd" in _cuda_kernel_of("aten::rms_norm")
        assert "flaggems_amd" in _cuda_kernel_of("aten::_softmax")
    after = _cuda_kernel_of("aten::mm")
    assert after == before and "flaggems_amd" not in after


def test_unused_filters_by_function_name():
    with flag_gems.use_gems(unused=["mm", "softmax"]):
        ops = flag_gems.all_ops()
        assert "mm" not in ops and "_softmax" not in ops
        assert "mm.out" in ops and "addmm" in ops  # mm_out is a different python function
        assert "flaggems_amd" not in _cuda_kernel_of("aten::mm")


def test_enable_record_writes_log(tmp_path):
    import logging

    lib = torch.library.Library("aten", "IMPL")
    path = tmp_path / "oplist.log"
    try:
        flag_gems.enable(lib=lib, record=True, once=True, path=str(path))
        logging.getLogger("flag_gems.ops.mm").debug("GEMS MM probe")
        for h in logging.getLogger("flag_gems").handlers:
            h.flush()
        assert "GEMS MM probe" in path.read_text()
    finally:
        lib._destroy()
        lg = logging.getLogger("flag_gems")
        for h in lg.handlers[:]:
            lg.removeHandler(h)
            h.close()


def test_registration_error_is_wrapped():
    class Boom:
        def impl(self, *a):
            raise ValueError("no")

    with pytest.raises(RuntimeError) as ei:
        flaggems_amd.runtime.Register((("mm", flag_gems.mm),), lib=Boom())
    assert "An error was encountered while registering the triton operator." in str(ei.value.args)


def test_library_exports_every_declared_symbol():
    header = open(os.path.join(ROOT, "include", "fg_mi355.h")).read()
    declared = set(re.findall(r"\b(fg_[a-z0-9_]+)\s*\(", header))
    assert declared, "no declarations found"
    handle = ctypes.CDLL(_C.LIB_PATH)
    for name in declared:
        assert hasattr(handle, name), f"{name} declared in include/fg_mi355.h but not exported"
    assert declared == set(_C.exported_symbols()), "python binding and header disagree"
    assert _C.lib().fg_abi_version() == 2


_C_BINDER = r"""
#include <stddef.h>
#include <stdio.h>
#include "fg_mi355.h"
int main(void) {
  FgFlashParams p;
  int rc = fg_softmax(NULL, NULL, -1, 4, 1, FG_F32, FG_F32, NULL);
  printf("abi=%d rc=%d (%s) invalid=%d unsupported=%d\n", fg_abi_version(), rc, fg_last_error(), FG_ERR_INVALID,
         FG_ERR_UNSUPPORTED);
  printf("params=%d workspace_at=%d\n", (int)sizeof p, (int)offsetof(FgFlashParams, workspace));
  return 0;
}
"""


def test_header_is_plain_c_and_a_c_program_binds_the_library(tmp_path):
    """The boundary is a C ABI: the header compiles as strict C99 and as C++11, and a C program that includes it and
    links the library calls an entry point and reads its error message; the struct the attention entry point takes has
    the size and field offset the ctypes mirror gives it.  (No launch: the call is rejected on the host.)"""
    import shutil
    import subprocess

    gcc, gxx = shutil.which("gcc"), shutil.which("g++")
    if gcc is None or gxx is None:
        pytest.skip("no host compiler")
    inc = os.path.join(ROOT, "include")
    strict = ["-Wall", "-Wextra", "-Werror", "-pedantic", "-fsyntax-only"]
    subprocess.run([gcc, "-std=c99", "-x", "c"] + strict + [os.path.join(inc, "fg_mi355.h")], check=True)
    subprocess.run([gxx, "-std=c++11", "-x", "c++"] + strict + [os.path.join(inc, "fg_mi355.h")], check=True)
    src, exe = tmp_path / "binder.c", tmp_path / "binder"
    src.write_text(_C_BINDER)
    libdir = os.path.dirname(_C.LIB_PATH)
    subprocess.run([gcc, "-std=c99", "-Wall", "-Wextra", "-Werror", "-pedantic", "-I", inc, str(src), "-o", str(exe),
                    "-L", libdir, "-l:" + os.path.basename(_C.LIB_PATH), "-Wl,-rpath," + libdir], check=True)
    out = subprocess.run([str(exe)], check=True, capture_output=True, text=True).stdout
    assert "abi=2 rc=-1 (softmax: negative size) invalid=-1 unsupported=-2" in out, out
    assert "params=%d workspace_at=%d" % (ctypes.sizeof(_C.FgFlashParams), _C.FgFlashParams.workspace.offset) in out, out


def test_documented_cpp_binding_compiles():
    """The C++ binding that the integration notes show for the reference's native layer (an ATen function around
    fg_rms_norm) is real code: it passes the compiler's front end against this image's torch and HIP headers."""
    import shutil
    import subprocess

    gxx = shutil.which("g++")
    notes = os.path.join(ROOT, "INTEGRATION.md")
    if gxx is None or not os.path.exists(notes) or not os.path.isdir("/opt/rocm/include"):
        pytest.skip("needs g++, the integration notes and the ROCm headers")
    from torch.utils.cpp_extension import include_paths

    block = re.search(r"```cpp\n(.*?)```", open(notes).read(), re.S)
    assert block and "fg_rms_norm(" in block.group(1)
    unit = ("#include <ATen/ATen.h>\n#include <c10/core/DeviceGuard.h>\n#include <c10/hip/HIPStream.h>\n"
            "#include <torch/library.h>\n" + block.group(1))
    cmd = [gxx, "-std=c++17", "-fsyntax-only", "-D__HIP_PLATFORM_AMD__", "-DUSE_ROCM", "-x", "c++", "-"]
    for inc in include_paths() + ["/opt/rocm/include", os.path.join(ROOT, "include")]:
        cmd += ["-I", inc]
    p = subprocess.run(cmd, input=unit, capture_output=True, text=True)
    assert p.returncode == 0, p.stderr[-3000:]


def test_struct_mirror_matches_header_order():
    header = open(os.path.join(ROOT, "include", "fg_mi355.h")).read()
    body = header[header.index("typedef struct FgFlashParams {"):header.index("} FgFlashParams;")]
    body = re.sub(r"/\*.*?\*/", "", body, flags=re.S)
    body = body[body.index("{") + 1:]
    names = []
    for decl in body.split(";"):
        decl = decl.strip()
        if not decl:
            continue
        parts = decl.replace("*", " ").split(",")
        first = parts[0].split()
        names.append(first[-1])
        names.extend(p.strip() for p in parts[1:])
    assert names == [f[0] for f in _C.FgFlashParams._fields_]


def test_abi_validation_errors_without_gpu():
    lib = _C.lib()
    # invalid arguments are rejected on the host before any launch
    assert lib.fg_softmax(None, None, -1, 4, 1, _C.FG_F32, _C.FG_F32, None) == -1
    assert "negative" in _C.last_error()
    assert lib.fg_softmax(None, None, 4, 4, 1, _C.FG_F32, _C.FG_F32, None) == -1  # null pointers
    assert lib.fg_rms_norm(None, None, None, None, 4, 4, 4, 4, 1e-5, _C.FG_F32, None) == -1
    assert lib.fg_rms_norm(None, None, None, None, 0, 4, 4, 4, 1e-5, _C.FG_F32, None) == 0  # empty: nothing to do
    assert lib.fg_silu_and_mul(None, None, None, 2, 2, 2, 2, 2, 7, None) == -1
    assert lib.fg_reshape_and_cache_flash(None, None, None, None, None, 1, 4, 2, 8, 0, 16, 16, 256, 2, None) == -1
    assert "block_size" in _C.last_error()
    one = ctypes.c_void_p(256)
    rc = lib.fg_gemm(one, one, None, one, 4, 4, 4, 4, 1, 4, 1, 0, 0, 4, 1, 1.0, 0.0, _C.FG_F16, _C.FG_F32, _C.FG_F16,
                     0, None, 0, None, None)
    assert rc == -2 and "output dtype" in _C.last_error()
    rc = lib.fg_gemm(one, one, None, one, 4, 4, 0, 4, 1, 4, 1, 0, 0, 4, 1, 1.0, 0.0, _C.FG_F16, _C.FG_F16, _C.FG_F16,
                     0, None, 0, None, None)
    assert rc == -1 and "K must be positive" in _C.last_error()
    # the entry point that allocates nothing turns away what its static scratch array cannot hold, before any launch
    rc = lib.fg_gemm_skinny_static(one, one, None, one, 65, 512, 2048, 2048, 1, 1, 2048, 0, 0, 512, 1, 1.0, 0.0,
                                   _C.FG_BF16, _C.FG_BF16, _C.FG_BF16, None)
    assert rc == -2 and "exceed the maximum of 64" in _C.last_error()
    rc = lib.fg_gemm_skinny_static(one, one, None, one, 8, 512, 2048, 2048, 1, 1, 2048, 0, 0, 512, 1, 1.0, 0.0,
                                   _C.FG_F32, _C.FG_F32, _C.FG_F32, None)
    assert rc == -2 and "16-bit inputs only" in _C.last_error()
    p = _C.FgFlashParams()
    p.dtype = _C.FG_F32
    assert lib.fg_flash_attn_varlen_fwd(ctypes.byref(p), None) == -1
    assert "fp16 and bf16" in _C.last_error()
    with pytest.raises(RuntimeError):
        _C.check(-1, "probe")


def test_bmm_abi_refuses_batches_beyond_the_verified_envelope():
    """fg_bmm itself, not only the Python wrapper, keeps callers inside the batch sizes its parity cases cover: the
    refusal happens on the host, before any launch (the pointers here are never dereferenced)."""
    import importlib

    bmm_mod = importlib.import_module("flaggems_amd.ops.bmm")

    lib = _C.lib()
    one = ctypes.c_void_p(256)

    def call(batch, M, N, K):
        return lib.fg_bmm(one, one, one, batch, M, N, K, M * K, K, 1, K * N, N, 1, M * N, N, 1, _C.FG_BF16, None)

    assert call(32, 2048, 2048, 128) == -2                      # FG_ERR_UNSUPPORTED: the batch that once faulted
    assert "verified envelope" in _C.last_error()
    assert call(17, 8, 8, 8) == -2                              # more than 16 matrices
    assert call(16, 1024, 1025, 8) == -2                        # more than 2^24 output elements
    assert call(0, 2048, 2048, 128) == 0 and call(64, 0, 8, 8) == 0   # empty: nothing to do, whatever the batch
    header = open(os.path.join(os.path.dirname(os.path.dirname(os.path.abspath(__file__))), "include", "fg_mi355.h")).read()
    assert int(re.search(r"#define FG_BMM_MAX_BATCH (\d+)", header).group(1)) == bmm_mod._MAX_BATCH
    assert 1 << int(re.search(r"#define FG_BMM_MAX_OUT_ELEMS \(1LL << (\d+)\)", header).group(1)) == bmm_mod._MAX_OUT_ELEMS


def test_python_wrappers_assert_like_the_reference():
    a = torch.randn(4, 5)
    b = torch.randn(6, 7)
    with pytest.raises(AssertionError, match="incompatible dimensions"):
        from flaggems_amd.ops.mm import _prepare

        _prepare(a, b)
    with pytest.raises(AssertionError, match="Incompatible dimensions"):
        flag_gems.addmm(torch.randn(7), a, b)
    with pytest.raises(AssertionError, match="Incompatible input shape"):
        flag_gems.addmm(torch.randn(3), a, torch.randn(5, 7))
    with pytest.raises(AssertionError, match="Invalid dim"):
        flag_gems.softmax(torch.randn(3, 3), 2)
    q = torch.randn(2, 3, 4, 8)
    with pytest.raises(AssertionError, match="same last dimension"):
        flag_gems.apply_rotary_pos_emb(q, torch.randn(2, 3, 4, 16), torch.randn(8, 4), torch.randn(8, 4))
    with pytest.raises(AssertionError, match="half of q/k dim"):
        flag_gems.apply_rotary_pos_emb(q, q, torch.randn(8, 8), torch.randn(8, 8))
    with pytest.raises(AssertionError, match="4 dimensions"):
        flag_gems.apply_rotary_pos_emb(q[0], q[0], torch.randn(8, 4), torch.randn(8, 4))
    cu = torch.zeros(2, dtype=torch.int32)
    with pytest.raises(AssertionError, match="cu_seqlens_k or seqused_k must be provided"):
        flag_gems.flash_attn_varlen_func(q[0], q, q, 3, cu, 3)
    with pytest.raises(AssertionError, match="cannot be provided at the same time"):
        flag_gems.flash_attn_varlen_func(q[0], q, q, 3, cu, 3, cu_seqlens_k=cu, seqused_k=cu[:1])
    with pytest.raises(RuntimeError, match="Only FA2"):
        flag_gems.flash_attn_varlen_func(q[0], q, q, 3, cu, 3, seqused_k=cu[:1], fa_version=3)
    with pytest.raises(RuntimeError, match="num_splits"):
        flag_gems.flash_attn_varlen_func(q[0], q, q, 3, cu, 3, seqused_k=cu[:1], num_splits=2)


def test_broadcastable_and_dtype_order():
    from flaggems_amd.ops._gemm import get_higher_dtype
    from flaggems_amd.ops.addmm import broadcastable_to

    assert broadcastable_to((), (3, 4)) and broadcastable_to((4,), (3, 4)) and broadcastable_to((1, 4), (3, 4))
    assert broadcastable_to((3, 1), (3, 4)) and not broadcastable_to((3,), (3, 4)) and not broadcastable_to((2, 3, 4), (3, 4))
    assert not broadcastable_to((4,), ())
    f16, bf16, f32 = torch.float16, torch.bfloat16, torch.float32
    assert get_higher_dtype(f16, bf16) is bf16 and get_higher_dtype(bf16, f32) is f32 and get_higher_dtype(f16, f16) is f16


def test_assert_close_rule():
    from flag_gems.testing import assert_close

    ref = torch.tensor([1.0, 100.0], dtype=torch.float64)
    assert_close(torch.tensor([1.0, 101.5], dtype=torch.bfloat16), ref, torch.bfloat16)  # rtol 1.6e-2
    with pytest.raises(AssertionError):
        assert_close(torch.tensor([1.0, 103.0], dtype=torch.bfloat16), ref, torch.bfloat16)
    assert_close(torch.tensor([1.05, 100.0], dtype=torch.float32), ref, torch.float32, reduce_dim=1000)  # atol 0.1
    with pytest.raises(AssertionError):
        assert_close(torch.tensor([1.0], dtype=torch.float32), ref[:1], torch.float16)  # dtype must match


def test_missing_library_fails_loudly(monkeypatch, tmp_path):
    monkeypatch.setattr(_C, "_lib", None)
    monkeypatch.setattr(_C, "LIB_PATH", str(tmp_path / "nope.so"))
    with pytest.raises(_C.ExtensionMissing):
        _C.lib()


def test_product_never_imports_the_oracle():
    pkg = os.path.join(ROOT, "flaggems_amd")
    for base, _, files in os.walk(pkg):
        for f in files:
            if f.endswith((".py", ".hip", ".h", ".cpp")):
                text = open(os.path.join(base, f)).read()
                assert "oracle" not in text.replace("the oracle", ""), f"{f} mentions the oracle package"


def test_custom_op_namespace_schemas():
    """torch.ops.flag_gems.* carries the reference's schemas for the operators of this path
    (src/flag_gems/csrc/cstub.cpp:26-90), each with a kernel on the CUDA key."""
    from flaggems_amd import custom_ops

    want = {
        "mm", "addmm", "bmm", "softmax", "softmax_backward", "rms_norm", "fused_add_rms_norm",
        "rotary_embedding", "rotary_embedding_inplace", "reshape_and_cache_flash", "flash_attn_varlen_func",
    }
    assert set(custom_ops.op_names()) == want
    for name in want:
        op = getattr(torch.ops.flag_gems, name).default
        assert "custom_ops.py" in _cuda_kernel_of("flag_gems::" + name), name
        assert op._schema.name == "flag_gems::" + name
    s = torch.ops.flag_gems.fused_add_rms_norm.default._schema
    assert [a.name for a in s.arguments] == ["input", "residual", "weight", "epsilon"]
    assert s.arguments[0].alias_info.is_write and s.arguments[1].alias_info.is_write and len(s.returns) == 0
    s = torch.ops.flag_gems.rms_norm.default._schema
    assert [a.name for a in s.arguments] == ["input", "weight", "epsilon"]
    s = torch.ops.flag_gems.reshape_and_cache_flash.default._schema
    assert [a.name for a in s.arguments] == [
        "key", "value", "key_cache", "value_cache", "slot_mapping", "kv_cache_dtype", "k_scale", "v_scale"]
    assert s.arguments[2].alias_info.is_write and s.arguments[3].alias_info.is_write and len(s.returns) == 0
    s = torch.ops.flag_gems.flash_attn_varlen_func.default._schema
    assert [a.name for a in s.arguments] == [
        "q", "k", "v", "max_seqlen_q", "cu_seqlens_q", "max_seqlen_k", "cu_seqlens_k", "seqused_k", "q_v", "dropout_p",
        "softmax_scale", "causal", "window_size", "softcap", "alibi_slopes", "deterministic", "return_attn_probs",
        "block_table", "return_softmax_lse", "out", "scheduler_metadata", "q_descale", "k_descale", "v_descale",
        "fa_version"]
    assert len(s.returns) == 2
    s = torch.ops.flag_gems.addmm.default._schema
    assert [(a.name, a.kwarg_only) for a in s.arguments] == [
        ("self", False), ("mat1", False), ("mat2", False), ("beta", True), ("alpha", True)]
    s = torch.ops.flag_gems.rotary_embedding_inplace.default._schema
    assert s.arguments[0].alias_info.is_write and s.arguments[1].alias_info.is_write and len(s.returns) == 0
    assert len(torch.ops.flag_gems.rotary_embedding.default._schema.returns) == 2
    # a CPU tensor finds no kernel: the namespace is served on the CUDA key only, as in the reference
    with pytest.raises((NotImplementedError, RuntimeError)):
        torch.ops.flag_gems.mm(torch.ones(2, 2), torch.ones(2, 2))


def test_gemm_workspace_made_under_capture_is_cleared_on_first_eager_use(monkeypatch):
    """Bookkeeping of the cached stream-K scratch buffer (flaggems_amd/ops/_gemm.py), with a stand-in library that
    reports capture ids: a buffer first made while its stream is being captured has had its clear only recorded, so
    the first eager use clears the header itself; later eager uses do not touch it; a new capture records a clear."""
    from flaggems_amd.ops import _gemm

    state = {"capture": 7}

    class Lib:
        def fg_stream_capture_id(self, stream, out):
            out._obj.value = state["capture"]
            return 0

        def fg_gemm_workspace_layout(self, dev, total, header):
            total._obj.value, header._obj.value = 4096, 256
            return 0

    monkeypatch.setattr(_C, "lib", lambda: Lib())
    monkeypatch.setattr(_gemm, "_workspaces", {})
    monkeypatch.setattr(_gemm, "_layouts", {})
    dev = torch.device("cpu")
    buf = _gemm._workspace(dev, 123)                  # made "under capture 7"
    entry = _gemm._workspaces[(dev.index, 123)]
    assert entry[1] == 7 and entry[3] is False
    buf.fill_(0xFF)                                   # the recorded clear never ran
    assert _gemm._workspace(dev, 123) is buf and (buf[:256] == 0xFF).all()   # same capture: nothing new recorded
    state["capture"] = 0
    assert _gemm._workspace(dev, 123) is buf
    assert (buf[:256] == 0).all() and (buf[256:] == 0xFF).all() and entry[3] is True
    buf[:256].fill_(5)                                # kernels own the header between eager calls
    assert _gemm._workspace(dev, 123) is buf and (buf[:256] == 5).all()
    state["capture"] = 9                              # a new capture on the stream records its own clear
    _gemm._workspace(dev, 123)
    assert (buf[:256] == 0).all() and entry[1] == 9
    state["capture"] = 0
    buf[:256].fill_(5)
    _gemm._workspace(dev, 123)                        # back to eager: already cleared once for real, left alone
    assert (buf[:256] == 5).all()
    buf2 = _gemm._workspace(dev, 456)                 # a buffer made eagerly is cleared on the spot
    assert (buf2[:256] == 0).all() and _gemm._workspaces[(dev.index, 456)][3] is True
