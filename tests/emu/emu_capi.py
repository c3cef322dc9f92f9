"""TEST INFRASTRUCTURE: loads tests/emu/libmolgrid_emu.so (the library's kernels compiled for the
host against the HIP emulation) with the prototypes of the real C ABI, and hands out arrays whose
memory ends at an inaccessible page, so that a kernel that runs past an array faults."""
import ctypes
import os
import sys

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(os.path.dirname(HERE))
sys.path.insert(0, ROOT)
sys.path.insert(0, HERE)

import build_emu  # noqa: E402
from libmolgrid_amd import _capi  # noqa: E402  (prototypes only)

lib = _capi.declare(ctypes.CDLL(build_emu.build()))
lib.emu_alloc.restype = ctypes.c_void_p
lib.emu_alloc.argtypes = [ctypes.c_size_t]
lib.emu_alloc_tight.restype = ctypes.c_void_p
lib.emu_alloc_tight.argtypes = [ctypes.c_size_t]
lib.emu_free.argtypes = [ctypes.c_void_p]

mg_gridmaker = _capi.mg_gridmaker
f3, f4 = _capi.f3, _capi.f4
_keep = []


# Number of 4-byte elements by which arrays of 4-byte elements start past a 16-byte boundary (0..3):
# callers hand the library views into larger tensors, whose first element sits anywhere.
MISALIGN = 0


def array(shape, dtype=np.float32, fill=None, tight=True):
    """Uninitialised (0xCB bytes) array in guarded memory."""
    shape = tuple(int(d) for d in np.atleast_1d(shape))
    item = np.dtype(dtype).itemsize
    n = int(np.prod(shape)) * item
    # (a tight block ends within 15 bytes of the guard page: shifting the array's start by
    # 4 * MISALIGN bytes keeps that, as the size is rounded up to 16 bytes first)
    shift = 4 * MISALIGN if (tight and item == 4) else 0
    total = max(n, 1) + (16 if shift else 0)
    if shift:
        total = (total + 15) & ~15
    p = (lib.emu_alloc_tight if tight else lib.emu_alloc)(total)
    buf = (ctypes.c_char * total).from_address(p)
    start = ((total - n - shift) // 16) * 16 + shift if shift else 0      # as far back as it goes
    a = np.frombuffer(buf, dtype=dtype, count=int(np.prod(shape)), offset=start).reshape(shape)
    _keep.append(buf)
    if fill is not None:
        a[...] = fill
    return a


def release_all():
    """Gives back every array handed out so far (their numpy views must not be used afterwards):
    for runs of many cases in one process."""
    for buf in _keep:
        lib.emu_free(ctypes.addressof(buf))
    del _keep[:]


def put(x, dtype=np.float32):
    """Copy of x in guarded memory."""
    x = np.ascontiguousarray(x, dtype=dtype)
    a = array(x.shape, dtype)
    a[...] = x
    return a


def ptr(a):
    return None if a is None or a.size == 0 else a.ctypes.data


def gridmaker(resolution, dimension, binary=False, radii_type_indexed=False, radius_scale=1.0,
              gaussian_radius_multiple=1.0):
    g = mg_gridmaker()
    code = lib.mg_gridmaker_init(ctypes.byref(g), resolution, dimension, int(binary),
                                 int(radii_type_indexed), radius_scale, gaussian_radius_multiple)
    assert code == 0
    return g
