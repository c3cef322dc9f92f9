"""TEST INFRASTRUCTURE: lets the Python host layer (libmolgrid_amd.gridding, torch_bindings, bench.py)
run on a machine without a GPU, against the emulated kernels of tests/emu.

`activate()` swaps the C library of the package for tests/emu/libmolgrid_emu.so and makes torch look
as if it had one ROCm device: tensors created "on the device" are CPU tensors of a subclass that
answers is_cuda = True (their data pointers are host pointers, which is what the emulated library
takes), streams and events are stand-ins (an event's time is the host clock), graph capture is
refused.  Nothing in the product knows about this; it exists so that the argument plumbing of the
host layer -- which workspace goes to which call, which overload takes which path -- is exercised
before the first run on real hardware."""
import contextlib
import ctypes
import os
import sys
import time

import torch

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, HERE)


class _Device(object):
    type = "cuda"
    index = 0

    def __str__(self):
        return "cuda:0"


class DevTensor(torch.Tensor):
    """A CPU tensor that says it lives on cuda:0."""

    @staticmethod
    def __new__(cls, t):
        return torch.Tensor._make_subclass(cls, t.detach() if t.requires_grad else t, t.requires_grad)

    is_cuda = property(lambda self: True)
    device = property(lambda self: _Device())

    def cuda(self, *a, **k):
        return self

    def cpu(self):
        return torch.Tensor._make_subclass(torch.Tensor, self.detach())

    def numpy(self):
        return self.cpu().numpy()

    def record_stream(self, stream):
        return None


def on_device(t):
    return t if isinstance(t, DevTensor) else DevTensor(t)


class FakeStream(object):
    cuda_stream = 0

    def __init__(self, *a, **k):
        pass

    def wait_event(self, e):
        pass

    def wait_stream(self, s):
        pass

    def synchronize(self):
        pass


class FakeEvent(object):
    def __init__(self, enable_timing=False, **k):
        self.t = None

    def record(self, stream=None):
        self.t = time.perf_counter()

    def elapsed_time(self, other):
        return (other.t - self.t) * 1e3

    def synchronize(self):
        pass

    def wait(self, stream=None):
        pass


class _NoGraph(object):
    def __init__(self, *a, **k):
        raise RuntimeError("the fake device captures no graphs")


def _is_cuda_device(d):
    return d is not None and (isinstance(d, _Device) or str(d).startswith("cuda"))


def _aligned(t, alignment=512):
    """A copy-free stand-in for the device allocator's alignment: byte buffers (the workspaces of
    the host layer) start at a multiple of 512 bytes, as torch's device allocations do."""
    if t.dtype != torch.uint8 or t.dim() != 1 or t.data_ptr() % alignment == 0:
        return t
    big = torch.empty(t.numel() + alignment, dtype=torch.uint8)
    shift = (-big.data_ptr()) % alignment
    return big[shift:shift + t.numel()]


def _factory(fn):
    def wrapped(*a, **k):
        d = k.get("device")
        if _is_cuda_device(d):
            k["device"] = "cpu"
            return on_device(_aligned(fn(*a, **k)))
        return fn(*a, **k)
    return wrapped


_active = False


def activate():
    """Patches torch and the package for the rest of the process."""
    global _active
    if _active:
        return
    _active = True
    import emu_capi                                   # builds and loads the emulated library
    lib = emu_capi.lib
    lib.emu_check_allocations.argtypes = [ctypes.c_int]
    lib.emu_check_allocations(0)                      # torch's memory is not the emulator's
    from libmolgrid_amd import _capi, gridding
    _capi.lib = lib
    gridding._lib = lib
    import libmolgrid_amd
    libmolgrid_amd._lib = lib
    gridding._device = lambda: _Device()
    gridding._stream = lambda: 0

    torch.cuda.is_available = lambda: True
    torch.cuda.device_count = lambda: 1
    torch.cuda.set_device = lambda d: None
    torch.cuda.current_device = lambda: 0
    torch.cuda.synchronize = lambda *a, **k: None
    torch.cuda.current_stream = lambda *a, **k: FakeStream()
    torch.cuda.Stream = FakeStream
    torch.cuda.Event = FakeEvent
    torch.cuda.stream = lambda s: contextlib.nullcontext()
    torch.cuda.CUDAGraph = _NoGraph
    torch.cuda.graph = _NoGraph
    real_generator = torch.Generator

    class HostGenerator(real_generator):              # a generator "on the device" is a host one
        def __new__(cls, device=None):
            return real_generator.__new__(cls)

    torch.Generator = HostGenerator
    for name in ("empty", "zeros", "ones", "full", "randn", "rand", "randint", "arange", "tensor", "linspace"):
        setattr(torch, name, _factory(getattr(torch, name)))
    real_as_tensor = torch.as_tensor
    torch.as_tensor = real_as_tensor
    # (a copy, as a transfer to a device is)
    torch.Tensor.cuda = lambda self, *a, **k: self if isinstance(self, DevTensor) else on_device(self.clone())
    real_to = torch.Tensor.to

    def to(self, *a, **k):
        dev = k.get("device", a[0] if a and not isinstance(a[0], torch.dtype) else None)
        if _is_cuda_device(dev):
            if "device" in k:
                k["device"] = "cpu"
            a = tuple("cpu" if x is dev else x for x in a)
            moved = real_to(self, *a, **k)
            return moved if isinstance(self, DevTensor) and moved is self else on_device(
                moved.clone() if moved.data_ptr() == self.data_ptr() else moved)
        return real_to(self, *a, **k)
    torch.Tensor.to = to
    torch.Tensor.record_stream = lambda self, s: None
