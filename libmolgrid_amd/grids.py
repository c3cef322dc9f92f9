"""Grid views and managed grids with the names and behaviour of the reference's Python module
(python/bindings_grids.cpp, include/libmolgrid/grid.h, include/libmolgrid/managed_grid.h):

  Grid{N}f / Grid{N}d            non-owning view of host memory (a numpy array, a CPU tensor, ...)
  Grid{N}fCUDA / Grid{N}dCUDA    non-owning view of device memory (a ROCm tensor)
  MGrid{N}f / MGrid{N}d          owning buffer that lives on the host or on the device and
                                 migrates as a whole when the other side is asked for

for N = 1 .. 8.  The memory is held as torch tensors; a view never copies.  Every class can be
passed wherever this package takes an array (GridMaker, Transform, GridInterpolater).
"""
import numpy as np
import torch

MAX_GRID_DIM = 8

_DTYPES = {"f": (torch.float32, np.float32, "float32"), "d": (torch.float64, np.float64, "float64")}


def _flat_copy(dst, src):
    """Copy min(size) elements in flat (row-major) order; returns the count (grid.h copyTo)."""
    n = min(dst.numel(), src.numel())
    if n:
        dst.reshape(-1)[:n].copy_(src.reshape(-1)[:n])
    return n


def _tensor_of(x, want_cuda=None):
    """torch tensor sharing the memory of a grid, managed grid, tensor or numpy array."""
    if isinstance(x, ManagedGridBase):
        if want_cuda is None:
            return x._current()
        return x.gpu()._t if want_cuda else x.cpu()._t
    if isinstance(x, GridBase):
        return x._t
    if isinstance(x, torch.Tensor):
        return x
    if isinstance(x, np.ndarray):
        return torch.from_numpy(x)
    raise TypeError("cannot view %r as a grid" % type(x).__name__)


class GridBase(object):
    """Common behaviour of the non-owning views; subclasses fix N, the element type and the side."""
    N = 0
    _code = "f"
    _cuda = False

    def __init__(self, src):
        tdtype, ndtype, _ = _DTYPES[self._code]
        if isinstance(src, ManagedGridBase):
            src = src.gpu() if self._cuda else src.cpu()
        if isinstance(src, GridBase):
            t = src._t
        elif isinstance(src, torch.Tensor):
            t = src.detach()
        elif isinstance(src, np.ndarray):
            if self._cuda:
                raise ValueError("a numpy array is host memory: use the Grid class without CUDA")
            if src.dtype != ndtype:
                raise ValueError("array has type %s, the grid wants %s" % (src.dtype, ndtype.__name__))
            if not src.flags.c_contiguous:
                raise ValueError("array is not C-contiguous")
            t = torch.from_numpy(src)
        else:
            raise TypeError("cannot make a grid from %r" % type(src).__name__)
        # python/bindings_grids.cpp:91-137
        if t.dtype != tdtype:
            raise ValueError("tensor has type %s, the grid wants %s" % (t.dtype, tdtype))
        if t.dim() != self.N:
            raise ValueError("expected %d dimensions, got %d" % (self.N, t.dim()))
        if not t.is_contiguous():
            raise ValueError("tensor is not contiguous")
        if t.is_cuda != self._cuda:
            raise ValueError("tensor is on the %s, the grid type is for the %s"
                             % ("device" if t.is_cuda else "host", "device" if self._cuda else "host"))
        if t.is_cuda and t.device.index != torch.cuda.current_device():
            raise ValueError("tensor is on device %d but the current device is %d"
                             % (t.device.index, torch.cuda.current_device()))
        self._t = t

    # -- shape ----------------------------------------------------------------
    @property
    def shape(self):
        return tuple(self._t.shape)

    def size(self):
        return int(self._t.numel())

    def dimension(self, i):
        return int(self._t.shape[i])

    def __len__(self):
        return int(self._t.shape[0])

    def data(self):
        return self._t.data_ptr()

    def type(self):
        return _DTYPES[self._code][2]

    # -- elements ---------------------------------------------------------------
    def _sub(self, t):
        return _grid_class(self.N - 1, self._code, self._cuda)(t)

    def __getitem__(self, idx):
        if isinstance(idx, tuple):
            if len(idx) != self.N:
                raise IndexError("%d indices for a %d-dimensional grid" % (len(idx), self.N))
            return self._t[idx].item()
        if idx < 0 or idx >= self._t.shape[0]:
            raise IndexError("Invalid access. Indices must be less than dimension.")
        if self.N == 1:
            return self._t[idx].item()
        return self._sub(self._t[idx])

    def __setitem__(self, idx, val):
        if isinstance(idx, tuple):
            if len(idx) != self.N:
                raise IndexError("%d indices for a %d-dimensional grid" % (len(idx), self.N))
        elif self.N != 1:
            raise TypeError("assigning to a slice is not supported: index every dimension")
        self._t[idx] = val

    # -- bulk -------------------------------------------------------------------
    def copyTo(self, dest):
        return _flat_copy(_tensor_of(dest), self._t)

    def copyFrom(self, src):
        return _flat_copy(self._t, _tensor_of(src))

    def fill_zero(self):
        self._t.zero_()

    def tonumpy(self):
        """A numpy copy (python/__init__.py:12-17)."""
        return self._t.detach().cpu().numpy().copy()

    def __array__(self, dtype=None, copy=None):
        a = self.tonumpy()
        return a if dtype is None else a.astype(dtype)

    def __repr__(self):
        return "%s%s" % (type(self).__name__, self.shape)


class _Storage(object):
    """The one buffer behind a managed grid and all of its sub-grids."""

    def __init__(self, host):
        self.host = host        # flat CPU tensor, always allocated
        self.dev = None         # flat device tensor, allocated on first use
        self.on_gpu = False     # which side holds the current values

    def to_gpu(self):
        if not self.on_gpu:
            if self.dev is None:
                self.dev = self.host.to(torch.device("cuda", torch.cuda.current_device()))
            else:
                self.dev.copy_(self.host)
            self.on_gpu = True

    def to_cpu(self):
        if self.on_gpu:
            self.host.copy_(self.dev)
            self.on_gpu = False


class ManagedGridBase(object):
    """Owning grid; ``cpu()`` / ``gpu()`` return views after migrating the WHOLE buffer to that
    side (include/libmolgrid/managed_grid.h:373-404).  Sub-grids share the buffer."""
    N = 0
    _code = "f"

    def __init__(self, *dims, **kw):
        storage = kw.pop("_storage", None)
        if storage is None:
            if len(dims) != self.N:
                raise TypeError("%s takes %d dimensions" % (type(self).__name__, self.N))
            n = 1
            for d in dims:
                n *= int(d)
            storage = _Storage(torch.zeros(n, dtype=_DTYPES[self._code][0]))
            offset = 0
        else:
            offset = kw.pop("_offset")
        self._s = storage
        self._offset = offset
        self._shape = tuple(int(d) for d in dims)
        self._n = 1
        for d in self._shape:
            self._n *= d

    def _view(self, flat):
        return flat[self._offset:self._offset + self._n].view(self._shape)

    def _current(self):
        return self._view(self._s.dev if self._s.on_gpu else self._s.host)

    # -- sides --------------------------------------------------------------------
    def cpu(self):
        self._s.to_cpu()
        return _grid_class(self.N, self._code, False)(self._view(self._s.host))

    def gpu(self):
        self._s.to_gpu()
        return _grid_class(self.N, self._code, True)(self._view(self._s.dev))

    def tocpu(self):
        self._s.to_cpu()

    def togpu(self):
        self._s.to_gpu()

    def ongpu(self):
        return self._s.on_gpu

    def oncpu(self):
        return not self._s.on_gpu

    # -- shape ----------------------------------------------------------------------
    @property
    def shape(self):
        return self._shape

    def size(self):
        return self._n

    def dimension(self, i):
        return self._shape[i]

    def __len__(self):
        return self._shape[0]

    def type(self):
        return _DTYPES[self._code][2]

    # -- elements (host side, like ManagedGrid::operator()) ----------------------------
    def __getitem__(self, idx):
        if isinstance(idx, tuple):
            return self.cpu()[idx]
        if idx < 0 or idx >= self._shape[0]:
            raise IndexError("Invalid access. Indices must be less than dimension.")
        if self.N == 1:
            return self.cpu()[idx]
        step = self._n // self._shape[0]
        return _mgrid_class(self.N - 1, self._code)(*self._shape[1:], _storage=self._s,
                                                   _offset=self._offset + idx * step)

    def __setitem__(self, idx, val):
        self.cpu()[idx] = val

    # -- bulk ---------------------------------------------------------------------------
    def copyTo(self, dest):
        return _flat_copy(_tensor_of(dest), self._current())

    def copyFrom(self, src):
        return _flat_copy(self._current(), _tensor_of(src))

    def fill_zero(self):
        self._current().zero_()

    def clone(self):
        """A managed grid of its own with the same values, on the same side."""
        c = _mgrid_class(self.N, self._code)(*self._shape)
        c._s.host.copy_(self._current().reshape(-1))
        if self._s.on_gpu:
            c._s.to_gpu()
        return c

    def tonumpy(self):
        return self._current().detach().cpu().numpy().copy()

    def __array__(self, dtype=None, copy=None):
        a = self.tonumpy()
        return a if dtype is None else a.astype(dtype)

    def __repr__(self):
        return "%s%s" % (type(self).__name__, self._shape)


_GRID_CLASSES = {}
_MGRID_CLASSES = {}


def _grid_class(n, code, cuda):
    return _GRID_CLASSES[(n, code, cuda)]


def _mgrid_class(n, code):
    return _MGRID_CLASSES[(n, code)]


def tonumpy(g):
    """python/__init__.py:12-17"""
    return g.tonumpy()


__all__ = ["tonumpy", "MAX_GRID_DIM"]
for _n in range(1, MAX_GRID_DIM + 1):
    for _code in ("f", "d"):
        for _cuda in (False, True):
            _name = "Grid%d%s%s" % (_n, _code, "CUDA" if _cuda else "")
            _cls = type(_name, (GridBase,), {"N": _n, "_code": _code, "_cuda": _cuda,
                                             "__doc__": "%d-dimensional %s view of %s memory"
                                             % (_n, _DTYPES[_code][2], "device" if _cuda else "host")})
            _GRID_CLASSES[(_n, _code, _cuda)] = _cls
            globals()[_name] = _cls
            __all__.append(_name)
        _name = "MGrid%d%s" % (_n, _code)
        _cls = type(_name, (ManagedGridBase,), {"N": _n, "_code": _code,
                                                "__doc__": "%d-dimensional managed %s grid"
                                                % (_n, _DTYPES[_code][2])})
        _MGRID_CLASSES[(_n, _code)] = _cls
        globals()[_name] = _cls
        __all__.append(_name)
