"""The GPU parity tests on the interpreter: with FG_INTERPRETED=1 in the environment, tests/conftest.py calls
install() before anything imports torch.  From then on the `gpu` fixture hands out the CPU device, the Python
wrappers run unchanged on CPU tensors, the library's host code runs against the HIP stand-in and every kernel is
interpreted; a tensor's storage becomes a bounds-checked buffer of the interpreted device the moment a wrapper asks
for its data_ptr().  Test infrastructure: nothing outside tests/ uses this.
"""
import os
import sys
import tempfile

HERE = os.path.dirname(os.path.abspath(__file__))
REPO = os.path.dirname(os.path.dirname(HERE))
DEVICE = None


def install():
    global DEVICE
    if DEVICE is not None:
        return DEVICE
    assert "torch" not in sys.modules, "the interpreter's HIP stand-in must be bound before torch maps the real runtime"
    sys.path.insert(0, HERE)
    try:
        from device import Device, build_shim
    finally:
        sys.path.remove(HERE)
    lib = os.environ.get("FG_LIB_PATH") or os.path.join(REPO, "flaggems_amd", "libfg_mi355.so")
    asm = os.environ.get("FG_ASM_DIR") or os.path.join(REPO, "flaggems_amd", "csrc", "build")
    dev = Device(lib, asm, build_shim(os.environ.get("FG_SHIM_DIR") or tempfile.gettempdir()))
    dev.shim.shim_set_num_cu(int(os.environ.get("FG_INTERPRETED_CUS", "256")))

    import torch
    from flaggems_amd import _C, runtime

    real_data_ptr = torch.Tensor.data_ptr

    def data_ptr(t):
        p = real_data_ptr(t)
        st = t.untyped_storage()
        if st.nbytes():
            dev.mem.map_external(st.data_ptr(), st.nbytes(), "tensor storage of %d bytes" % st.nbytes())
        dev.keep.append(t)
        return p

    dev.keep = []
    dev.total_launches = 0
    torch.Tensor.data_ptr = data_ptr
    torch.Tensor.is_cuda = property(lambda t: True)
    _C.current_stream = lambda device: 0
    _C.device_guard = lambda device: _C._NO_GUARD
    runtime.device.dispatch_key = "CPU"          # the ATen overrides of flag_gems.enable() then catch CPU tensors
    handle = _C.lib()                                # the library mapped above (same file, same mapping), with signatures
    for name in ("fg_gemm_workspace_bytes", "fg_gemm_workspace_layout"):
        def with_device_zero(*args, _fn=getattr(handle, name)):      # a CPU tensor's device has no index
            return _fn(*[0 if a is None else a for a in args])
        setattr(handle, name, with_device_zero)
    # hipMalloc hands out 256-byte aligned memory, which the stream-K workspace relies on; the CPU allocator promises 64
    from flaggems_amd.ops import _gemm

    class _AlignedTorch:
        def __getattr__(self, name):
            return getattr(torch, name)

        @staticmethod
        def empty(n, dtype=None, device=None):
            raw = torch.empty(n + 256, dtype=dtype, device=device)
            skip = (-real_data_ptr(raw)) % 256
            return raw[skip:skip + n]

    _gemm.torch = _AlignedTorch()
    torch.cuda.synchronize = lambda *a, **k: None
    torch.cuda.current_device = lambda: 0
    DEVICE = dev
    return dev


def between_tests():
    """Forget the tensors of the test that just ended; report what the interpreter refused, if anything."""
    dev = DEVICE
    err, dev.error = dev.error, None
    dev.keep.clear()
    dev.mem.drop_externals()
    dev.total_launches += len(dev.launches)
    dev.launches.clear()
    return err
