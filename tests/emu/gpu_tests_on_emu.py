"""Runs `-m gpu` test functions of tests/ on the CPU: the library is the emulated build (libmoe_gg_emu.so: the device
sources compiled for the host, tests/emu) and every torch "cuda" tensor is a CPU tensor, so the GPU tests' own code -
their inputs, the Python entry functions of applied-ai_amd, the ctypes calls, the comparisons against the oracle -
executes end to end without a GPU. It checks the tests and the host layer, at the sizes the emulation can carry; what
the emulation says about the kernels themselves is tests/test_emu_kernels.py's job. Test infrastructure only.

    python tests/emu/gpu_tests_on_emu.py <pytest node ids and options ...>

The process stands in for a GPU box: torch.cuda.is_available() is true here, so it runs nothing but the tests named.
"""
import contextlib
import functools
import os
import sys
import types

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(os.path.dirname(HERE))
for p in (ROOT, HERE):
    if p not in sys.path:
        sys.path.insert(0, p)

import pytest  # noqa: E402
import torch  # noqa: E402

import harness as H  # noqa: E402


def _is_cuda(d):
    return (isinstance(d, str) and d.startswith("cuda")) or (isinstance(d, torch.device) and d.type == "cuda")


def _fix(args, kwargs):
    args = tuple("cpu" if _is_cuda(a) else a for a in args)
    if _is_cuda(kwargs.get("device")):
        kwargs = dict(kwargs, device="cpu")
    return args, kwargs


def _aligned(t, real_empty):
    """`t` in storage that starts at a 256-byte boundary, as device allocations do (the C ABI checks alignment)."""
    if not isinstance(t, torch.Tensor) or t.numel() == 0 or not t.is_contiguous() or t.data_ptr() % 256 == 0:
        return t
    nbytes = t.numel() * t.element_size()
    raw = real_empty(nbytes + 256, dtype=torch.uint8)
    off = (-raw.data_ptr()) % 256
    out = raw[off:off + nbytes].view(t.dtype).view(t.shape)
    out.copy_(t)
    return out


def _wrap(fn, real_empty=None):
    @functools.wraps(fn)
    def inner(*args, **kwargs):
        args, kwargs = _fix(args, kwargs)
        out = fn(*args, **kwargs)
        return _aligned(out, real_empty) if real_empty is not None else out
    return inner


def install():
    import applied_ai_amd
    from applied_ai_amd import _lib, moe, ops, quant, routing

    emu = H.lib()
    _lib._lib = emu
    _lib.lib = lambda: emu
    cpu = torch.device("cpu")
    for mod in (ops, moe, quant, routing):
        if hasattr(mod, "_require_cuda"):
            mod._require_cuda = lambda *t: cpu
        if hasattr(mod, "_stream_ptr"):
            mod._stream_ptr = lambda dev: 0
    # factories that take a device
    real_empty = torch.empty
    for name in ("randn", "rand", "randint", "empty", "zeros", "ones", "full", "tensor", "arange", "empty_like", "zeros_like",
                 "ones_like", "full_like", "randn_like", "as_tensor", "eye", "linspace"):
        setattr(torch, name, _wrap(getattr(torch, name), real_empty))
    real_generator = torch.Generator
    torch.Generator = lambda device="cpu": real_generator("cpu")
    real_device = torch.device
    # tensor methods
    torch.Tensor.cuda = lambda self, *a, **k: _aligned(self.contiguous(), real_empty)
    torch.Tensor.to = _wrap(torch.Tensor.to)
    for name in ("new_empty", "new_zeros", "new_full", "new_ones", "new_tensor"):
        setattr(torch.Tensor, name, _wrap(getattr(torch.Tensor, name), real_empty))
    # the cuda namespace
    cus = int(os.environ.get("EMU_CUS", "8"))
    c = torch.cuda
    c.is_available = lambda: True
    c.synchronize = lambda *a, **k: None
    c.set_device = lambda *a, **k: None
    c.empty_cache = lambda: None
    c.current_stream = lambda *a, **k: types.SimpleNamespace(cuda_stream=0)
    c.device = lambda *a, **k: contextlib.nullcontext()
    c.get_device_properties = lambda *a, **k: types.SimpleNamespace(multi_processor_count=cus, total_memory=1 << 34, name="emulated")
    c.mem_get_info = lambda *a, **k: (1 << 33, 1 << 34)
    c.memory_allocated = lambda *a, **k: 0
    c.device_count = lambda: 1

    class Event:  # host-clock stand-in for torch.cuda.Event (the emulated launches are synchronous)
        def __init__(self, enable_timing=True):
            self.t = 0.0

        def record(self, *a):
            import time
            self.t = time.perf_counter()

        def elapsed_time(self, other):
            return (other.t - self.t) * 1e3 + 1e-3

    c.Event = Event
    return applied_ai_amd, real_device


def main(argv):
    install()
    return pytest.main(["-p", "no:cacheprovider", "-m", "gpu", "-x", "-q"] + argv)


if __name__ == "__main__":
    sys.exit(main(sys.argv[1:]))
