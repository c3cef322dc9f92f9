"""Host-side mirror of libmolgrid's gridding classes on top of the HIP C ABI.

``GridMaker``, ``GridInterpolater``, ``Transform``, ``Quaternion``, ``float3`` and
``CoordinateSet`` keep the names, argument order and error behaviour of the
reference's Python module (python/bindings.in.cpp:286-309, 455-520, 816-943)
for the gridding path.  Every numeric call validates its arguments as the
reference does (std::out_of_range -> IndexError, std::invalid_argument ->
ValueError) and then makes exactly one call into ``libmolgrid_hip.so``.

Arrays may be ROCm torch tensors (used in place, on torch's current stream) or
host arrays (numpy / CPU tensors): host arrays are staged through device memory
and the kernels still do the work -- there is no CPU implementation here.
"""
import functools
import math

import numpy as np
import torch

from . import _capi
from . import grids as _grids

_lib = _capi.lib


# --------------------------------------------------------------------------- #
# small value types
# --------------------------------------------------------------------------- #
class float3(object):
    """x, y, z triple; any 3-sequence converts (bindings.in.cpp:286-309)."""
    __slots__ = ("x", "y", "z")

    def __init__(self, x=0.0, y=0.0, z=0.0):
        self.x, self.y, self.z = float(x), float(y), float(z)

    def __iter__(self):
        return iter((self.x, self.y, self.z))

    def __len__(self):
        return 3

    def __getitem__(self, i):
        return (self.x, self.y, self.z)[i]

    def __eq__(self, o):
        return tuple(self) == tuple(o)

    def __repr__(self):
        return "float3(%g, %g, %g)" % (self.x, self.y, self.z)


def _to_float3(v):
    if isinstance(v, float3):
        return v
    v = _unwrap(v)
    if isinstance(v, torch.Tensor):
        v = v.detach().cpu().tolist()
    v = tuple(v)
    if len(v) != 3:
        raise ValueError("expected a sequence of 3 floats")
    return float3(*v)


_f32 = np.float32


class Quaternion(object):
    """Single-precision quaternion (a + bi + cj + dk), not assumed normalised.

    Arithmetic is done in float32 in the association order of
    include/libmolgrid/quaternion.h:82-166 so that host-side results are the
    same floats the device kernels produce.
    """
    __slots__ = ("a", "b", "c", "d")

    def __init__(self, a=1.0, b=0.0, c=0.0, d=0.0):
        self.a, self.b, self.c, self.d = _f32(a), _f32(b), _f32(c), _f32(d)

    def R_component_1(self):
        return float(self.a)

    def R_component_2(self):
        return float(self.b)

    def R_component_3(self):
        return float(self.c)

    def R_component_4(self):
        return float(self.d)

    def real(self):
        return float(self.a)

    def as_tuple(self):
        return (float(self.a), float(self.b), float(self.c), float(self.d))

    def __eq__(self, o):
        return isinstance(o, Quaternion) and self.as_tuple() == o.as_tuple()

    def __repr__(self):
        return "Quaternion(%g, %g, %g, %g)" % self.as_tuple()

    def __mul__(self, r):
        if not isinstance(r, Quaternion):
            r = _f32(r)
            return Quaternion(self.a * r, self.b * r, self.c * r, self.d * r)
        a, b, c, d = self.a, self.b, self.c, self.d
        return Quaternion(+a * r.a - b * r.b - c * r.c - d * r.d,
                          +a * r.b + b * r.a + c * r.d - d * r.c,
                          +a * r.c - b * r.d + c * r.a + d * r.b,
                          +a * r.d + b * r.c - c * r.b + d * r.a)

    def __truediv__(self, r):
        if not isinstance(r, Quaternion):
            r = _f32(r)
            return Quaternion(self.a / r, self.b / r, self.c / r, self.d / r)
        a, b, c, d = self.a, self.b, self.c, self.d
        den = r.a * r.a + r.b * r.b + r.c * r.c + r.d * r.d
        return Quaternion((+a * r.a + b * r.b + c * r.c + d * r.d) / den,
                          (-a * r.b + b * r.a - c * r.d + d * r.c) / den,
                          (-a * r.c + b * r.d + c * r.a - d * r.b) / den,
                          (-a * r.d - b * r.c + c * r.b + d * r.a) / den)

    def conj(self):
        return Quaternion(self.a, -self.b, -self.c, -self.d)

    def norm(self):
        """Cayley norm: the square of the Euclidean length."""
        return float(self.a * self.a + self.b * self.b + self.c * self.c + self.d * self.d)

    def inverse(self):
        n = self.a * self.a + self.b * self.b + self.c * self.c + self.d * self.d
        return Quaternion(self.a / n, -self.b / n, -self.c / n, -self.d / n)

    def rotate(self, x, y, z):
        p = self * Quaternion(0, x, y, z) * (self.conj() / _f32(self.norm()))
        return float3(p.b, p.c, p.d)

    def transform(self, x, y, z, center, translate):
        center, translate = _to_float3(center), _to_float3(translate)
        pt = self.rotate(_f32(x) - _f32(center.x), _f32(y) - _f32(center.y),
                         _f32(z) - _f32(center.z))
        return float3(_f32(pt.x) + _f32(center.x) + _f32(translate.x),
                      _f32(pt.y) + _f32(center.y) + _f32(translate.y),
                      _f32(pt.z) + _f32(center.z) + _f32(translate.z))


# random source for Transform's random constructor (the reference keeps one
# global engine, src/libmolgrid.cpp:11; set_random_seed reseeds it)
_rng = np.random.default_rng()


def set_random_seed(seed):
    global _rng
    _rng = np.random.default_rng(int(seed))


# --------------------------------------------------------------------------- #
# array staging
# --------------------------------------------------------------------------- #
def _device():
    if not torch.cuda.is_available():
        raise RuntimeError("libmolgrid_amd needs a ROCm device: the gridding kernels have no "
                           "CPU fallback")
    return torch.device("cuda", torch.cuda.current_device())


def _stream():
    return torch.cuda.current_stream().cuda_stream


def _unwrap(x):
    """Grid views and managed grids (grids.py) stand for their tensor; a managed grid for the side
    its values currently live on (python/bindings_grids.cpp:140-165)."""
    if isinstance(x, (_grids.GridBase, _grids.ManagedGridBase)):
        return _grids._tensor_of(x)
    return x


def _accepts_grids(fn):
    """Lets a public entry point take Grid / MGrid objects wherever it takes an array."""
    @functools.wraps(fn)
    def wrapper(*args, **kw):
        return fn(*[_unwrap(a) for a in args], **{k: _unwrap(v) for k, v in kw.items()})
    return wrapper


class _Arg(object):
    """A user array made visible to the device.

    ROCm tensors are used in place after the checks of
    python/bindings_grids.cpp:91-137 (contiguous, on the current device).  Host
    arrays are copied to the device when the pointer is first asked for (after
    all shape checks have passed) and, for outputs, back.

    The kernels read and write float32.  Where the reference has a
    ``Grid<double, ...>`` overload (``wide=True``: output grids, upstream
    gradients and gradients, transformed coordinates;
    python/bindings_grids.cpp:108-116) a float64 array is staged through a
    float32 copy on the device: narrowed before the call, widened after it.
    """

    def __init__(self, x, name, ndim, out=False, wide=False):
        x = _unwrap(x)
        self.name = name
        self.out = out
        self.host = None
        self.t = None
        self.wide_dev = None        # the caller's float64 device tensor, if that is what came
        if isinstance(x, torch.Tensor) and x.is_cuda:
            if x.dtype != torch.float32 and not (wide and x.dtype == torch.float64):
                raise ValueError("%s: only float32 device tensors are supported" % name)
            if not x.is_contiguous():
                raise ValueError("%s: tensor is not contiguous" % name)
            if x.device.index != torch.cuda.current_device():
                raise ValueError("%s: tensor is on device %d but the current device is %d"
                                 % (name, x.device.index, torch.cuda.current_device()))
            if x.dtype == torch.float64:
                self.wide_dev = x
            else:
                self.t = x
            self.shape = tuple(x.shape)
        else:
            if isinstance(x, torch.Tensor):
                if x.dtype != torch.float32 and not (wide and x.dtype == torch.float64):
                    raise ValueError("%s: only float32 tensors are supported" % name)
                if not x.is_contiguous():
                    raise ValueError("%s: tensor is not contiguous" % name)
                self.host = x.detach()
            elif out:
                ok = (np.float32, np.float64) if wide else (np.float32,)
                if not (isinstance(x, np.ndarray) and x.dtype in ok
                        and x.flags.c_contiguous and x.flags.writeable):
                    raise ValueError("%s: output must be a writable C-contiguous float32 "
                                     "array" % name)
                self.host = torch.from_numpy(x)
            else:
                self.host = torch.from_numpy(np.ascontiguousarray(x, dtype=np.float32))
            self.shape = tuple(self.host.shape)
        if len(self.shape) != ndim:
            raise ValueError("%s: expected %d dimensions, got %d" % (name, ndim, len(self.shape)))

    @property
    def ptr(self):
        if self.t is None:
            if self.out:
                self.t = torch.empty(self.shape, dtype=torch.float32, device=_device())
            elif self.wide_dev is not None:
                self.t = torch.empty(self.shape, dtype=torch.float32, device=_device())
                if self.t.numel():
                    _capi.check(_lib.mg_narrow(self.wide_dev.data_ptr(), self.t.data_ptr(),
                                               self.t.numel(), _stream()), self.name)
            else:
                self.t = self.host.to(device=_device(), dtype=torch.float32)
        return self.t.data_ptr() if self.t.numel() else None

    def finish(self):
        if not self.out or self.t is None:
            return
        if self.wide_dev is not None:
            if self.t.numel():
                _capi.check(_lib.mg_widen(self.t.data_ptr(), self.wide_dev.data_ptr(),
                                          self.t.numel(), _stream()), self.name)
        elif self.host is not None:
            self.host.copy_(self.t)          # widens on the way when the host array is float64


def _same_memory(a, b):
    a, b = _unwrap(a), _unwrap(b)
    try:
        pa = a.data_ptr() if isinstance(a, torch.Tensor) else a.ctypes.data
        pb = b.data_ptr() if isinstance(b, torch.Tensor) else b.ctypes.data
    except AttributeError:
        return False
    return pa == pb and pa != 0


def _is_host(x):
    x = _unwrap(x)
    return not (isinstance(x, torch.Tensor) and x.is_cuda)


def _small_device(values, width):
    """B x width float32 parameter rows on the device (None -> None)."""
    values = _unwrap(values)
    if values is None:
        return None
    if isinstance(values, torch.Tensor) and values.is_cuda:
        t = values
        if t.dtype != torch.float32 or not t.is_contiguous():
            raise ValueError("per-example parameters must be contiguous float32")
    else:
        t = torch.as_tensor(np.ascontiguousarray(values, dtype=np.float32)).to(_device())
    if t.dim() != 2 or t.shape[1] != width:
        raise ValueError("per-example parameters must have shape (B, %d)" % width)
    return t


class AtomBatch(object):
    """Atom offsets of a ragged batch, kept on the host and on the device.

    Build it once per batch layout and pass it wherever ``offsets`` is taken:
    the calls then need no host/device copy of the offsets.
    """

    def __init__(self, offsets):
        if isinstance(offsets, torch.Tensor):
            offsets = offsets.detach().cpu().numpy()
        host = np.ascontiguousarray(offsets, dtype=np.int64)
        if host.ndim != 1 or host.size < 1:
            raise ValueError("atom offsets must be a 1-D array of length batch+1")
        if host[0] < 0 or np.any(np.diff(host) < 0):
            raise ValueError("atom offsets must be non-decreasing")
        if host[-1] >= 2 ** 31:
            raise ValueError("too many atoms for 32-bit offsets")
        self.host = host
        self.nbatch = host.size - 1
        self.largest = max(int(np.max(np.diff(host))) if host.size > 1 else 0, 1)
        self.total = int(host[-1])
        self._dev = None
        self.scratch = {}            # device workspaces that calls on this layout keep

    @property
    def dev(self):
        if self._dev is None:
            self._dev = torch.as_tensor(self.host.astype(np.int32)).to(_device())
        return self._dev


class SortedBatch(object):
    """What ``GridMaker.sort_batch`` leaves for ``GridMaker.splat_batch``: the device workspace
    with the sorted atom records and their tables, and the sizes it was made for."""

    def __init__(self, workspace, nbytes, nbatch, largest, ntypes):
        self.workspace, self.nbytes = workspace, nbytes
        self.nbatch, self.largest, self.ntypes = nbatch, largest, ntypes


def _offsets_arg(offsets):
    """(device int32 tensor, nbatch, largest example, total atoms) for a ragged batch."""
    b = offsets if isinstance(offsets, AtomBatch) else AtomBatch(offsets)
    return b.dev, b.nbatch, b.largest, b.total


_Z3 = (0.0, 0.0, 0.0)
_IDQ = (1.0, 0.0, 0.0, 0.0)


def _ptr(t):
    return t.data_ptr() if t is not None and t.numel() else None


# --------------------------------------------------------------------------- #
# Transform
# --------------------------------------------------------------------------- #
def _qmul(p, q):
    """Hamilton product of (arrays of) float32 quaternion components, every product and sum
    rounded to float32 in the order of include/libmolgrid/quaternion.h:82-91."""
    a, b, c, d = p
    ar, br, cr, dr = q
    return (+a * ar - b * br - c * cr - d * dr,
            +a * br + b * ar + c * dr - d * cr,
            +a * cr - b * dr + c * ar + d * br,
            +a * dr + b * cr - c * br + d * ar)


def _qrotate(q, x, y, z):
    """q * (0, x, y, z) * (conj(q) / norm(q)) on float32 arrays (quaternion.h:145-149)."""
    a, b, c, d = q
    n = a * a + b * b + c * c + d * d
    cj = (a / n, -b / n, -c / n, -d / n)
    r = _qmul(_qmul(q, (np.zeros_like(x), x, y, z)), cj)
    return r[1], r[2], r[3]


def _host_transform(tr, inverse, src, dst, dotranslate):
    """Transform.forward / backward for host arrays, on the host (src/transform.cpp:57-108):
    numpy float32 arithmetic, one rounding per operation, in the reference's order -- the same
    floats the device kernel stores.  float64 arrays are narrowed where the reference narrows
    them (at the call of Quaternion::transform / rotate, which take floats)."""
    def view(x, out):
        x = _unwrap(x)
        if isinstance(x, torch.Tensor):
            if x.dtype not in (torch.float32, torch.float64):
                raise ValueError("only float32 and float64 tensors are supported")
            if not x.is_contiguous():
                raise ValueError("tensor is not contiguous")
            return x.detach().numpy()
        if out:
            if not (isinstance(x, np.ndarray) and x.dtype in (np.float32, np.float64)
                    and x.flags.c_contiguous and x.flags.writeable):
                raise ValueError("out: output must be a writable C-contiguous float32 array")
            return x
        x = np.asarray(x)
        return x if x.dtype == np.float64 else np.ascontiguousarray(x, dtype=np.float32)

    a_in, a_out = view(src, False), view(dst, True)
    if a_in.ndim != 2 or a_out.ndim != 2:
        raise ValueError("expected 2 dimensions")
    # transform.h:131-146 (checkGrids)
    if a_in.shape[0] != a_out.shape[0]:
        raise ValueError("Different dimensions and input and output coordinates grids.")
    if a_in.shape[1] != 3:
        raise ValueError("Input coordinates wrong dimension.")
    if a_out.shape[1] != 3:
        raise ValueError("Output coordinates are wrong dimension.")
    q = tuple(_f32(v) for v in tr.Q.as_tuple())
    c = [_f32(v) for v in tr.center]
    t = [_f32(v) if dotranslate else _f32(0.0) for v in tr.translate]
    with np.errstate(all="ignore"):
        if not inverse:
            x, y, z = (a_in[:, k].astype(np.float32) - c[k] for k in range(3))
            r = _qrotate(q, x, y, z)
            res = [r[k] + c[k] + t[k] for k in range(3)]
        else:
            n = q[0] * q[0] + q[1] * q[1] + q[2] * q[2] + q[3] * q[3]
            qinv = (q[0] / n, -q[1] / n, -q[2] / n, -q[3] / n)
            un = [-t[k] - c[k] for k in range(3)]
            # the sum is formed in the array's own type, then narrowed (transform.cpp:97-99)
            x, y, z = ((a_in[:, k] + un[k]).astype(np.float32) for k in range(3))
            r = _qrotate(qinv, x, y, z)
            res = [r[k] + c[k] for k in range(3)]
    for k in range(3):
        a_out[:, k] = res[k]


class Transform(object):
    """Rigid transform: rotate about ``center`` by ``Q``, then translate.

    Constructors (include/libmolgrid/transform.h:33-55):
      Transform()                                   identity
      Transform(Q, center=(0,0,0), translate=(0,0,0))
      Transform(center, random_translate=0.0, random_rotate=False)
    The random constructor draws the translation first (three U(-1,1) values
    scaled by ``random_translate``) and then a uniform rotation from three unit
    samples (src/transform.cpp:13-33).
    """

    def __init__(self, *args, **kw):
        self.Q = Quaternion()
        self.center = float3()
        self.translate = float3()
        if not args and not kw:
            return
        first = args[0] if args else kw.get("Q", kw.get("center"))
        if isinstance(first, Quaternion):
            names = ("Q", "center", "translate")
            vals = dict(zip(names, args))
            vals.update(kw)
            self.Q = vals["Q"]
            self.center = _to_float3(vals.get("center", _Z3))
            self.translate = _to_float3(vals.get("translate", _Z3))
        else:
            names = ("center", "random_translate", "random_rotate")
            vals = dict(zip(names, args))
            vals.update(kw)
            self.center = _to_float3(vals["center"])
            rt = float(vals.get("random_translate", 0.0))
            r = _rng.uniform(-1.0, 1.0, 3)
            self.translate = float3(_f32(r[0] * rt), _f32(r[1] * rt), _f32(r[2] * rt))
            if vals.get("random_rotate", False):
                u1, u2, u3 = _rng.uniform(0.0, 1.0, 3)
                sq1, sqr = math.sqrt(1 - u1), math.sqrt(u1)
                self.Q = Quaternion(sq1 * math.sin(2 * math.pi * u2),
                                    sq1 * math.cos(2 * math.pi * u2),
                                    sqr * math.sin(2 * math.pi * u3),
                                    sqr * math.cos(2 * math.pi * u3))

    def get_quaternion(self):
        return self.Q

    def get_rotation_center(self):
        return self.center

    def get_translation(self):
        return self.translate

    def set_quaternion(self, q):
        self.Q = q

    def set_rotation_center(self, c):
        self.center = _to_float3(c)

    def set_translation(self, t):
        self.translate = _to_float3(t)

    def is_identity(self):
        return self.Q == Quaternion() and tuple(self.translate) == _Z3

    def _apply(self, fn, what, src, dst, dotranslate):
        if isinstance(src, CoordinateSet):
            if not isinstance(dst, CoordinateSet):
                raise ValueError("output must be a CoordinateSet as well")
            if src.coords.shape[0] != dst.coords.shape[0]:
                raise ValueError("Incompatible coordinateset sizes")
            src, dst = src.coords, dst.coords
        if _is_host(src) and _is_host(dst):
            # the reference's Grid<Dtype, 2, false> overloads (src/transform.cpp:57-108) run on
            # the host; so do these, with the same float arithmetic as the kernel
            _host_transform(self, fn is _lib.mg_transform_backward, src, dst, dotranslate)
            return
        same = dst is src
        a_in = _Arg(src, "in", 2, wide=True)
        a_out = a_in if same and a_in.t is not None else _Arg(dst, "out", 2, out=True, wide=True)
        # transform.h:131-146 (checkGrids)
        if a_in.shape[0] != a_out.shape[0]:
            raise ValueError("Different dimensions and input and output coordinates grids.")
        if a_in.shape[1] != 3:
            raise ValueError("Input coordinates wrong dimension.")
        if a_out.shape[1] != 3:
            raise ValueError("Output coordinates are wrong dimension.")
        n = a_in.shape[0]
        code = fn(1, None, n, None, _capi.f4(self.Q.as_tuple()), None, _capi.f3(self.center),
                  None, _capi.f3(self.translate), int(bool(dotranslate)), a_in.ptr, a_out.ptr,
                  _stream())
        _capi.check(code, what)
        a_out.finish()

    @_accepts_grids
    def forward(self, src, dst, dotranslate=True):
        """dst = Q.rotate(src - center) + center (+ translate).  In place is fine."""
        self._apply(_lib.mg_transform_forward, "Transform.forward", src, dst, dotranslate)

    @_accepts_grids
    def backward(self, src, dst, dotranslate=True):
        """Inverse: un-translate, then rotate by the inverse about center."""
        self._apply(_lib.mg_transform_backward, "Transform.backward", src, dst, dotranslate)


@_accepts_grids
def transform_batch(offsets, quats, centers, translations, src, dst, dotranslate=True,
                    inverse=False):
    """Apply one rigid transform per example to a packed (ragged) batch of atoms.

    offsets: batch+1 atom offsets; quats (B,4), centers (B,3), translations (B,3).
    """
    off, nbatch, largest, total = _offsets_arg(offsets)
    q, c, t = _small_device(quats, 4), _small_device(centers, 3), _small_device(translations, 3)
    a_in = _Arg(src, "in", 2, wide=True)
    a_out = a_in if dst is src and a_in.t is not None else _Arg(dst, "out", 2, out=True, wide=True)
    if a_in.shape != a_out.shape or a_in.shape[1] != 3 or a_in.shape[0] < total:
        raise ValueError("coordinate arrays must both be (n, 3) with n >= offsets[-1]")
    for name, v in (("quats", q), ("centers", c), ("translations", t)):
        if v is not None and v.shape[0] != nbatch:
            raise ValueError("Mismatched batch sizes: %s has %d rows vs %d"
                             % (name, v.shape[0], nbatch))
    fn = _lib.mg_transform_backward if inverse else _lib.mg_transform_forward
    code = fn(nbatch, _ptr(off), largest, _ptr(q), _capi.f4(_IDQ), _ptr(c), _capi.f3(_Z3),
              _ptr(t), _capi.f3(_Z3), int(bool(dotranslate)), a_in.ptr, a_out.ptr, _stream())
    _capi.check(code, "transform_batch")
    a_out.finish()


# --------------------------------------------------------------------------- #
# CoordinateSet (array constructors only)
# --------------------------------------------------------------------------- #
def _managed(x, ndim, cols=None):
    """Managed float32 grid holding a copy of x (array, tensor or grid), on the side x is on."""
    x = _unwrap(x)
    if isinstance(x, torch.Tensor):
        t = x.detach()
    else:
        t = torch.from_numpy(np.ascontiguousarray(np.asarray(x, dtype=np.float32)))
    if t.dim() != ndim:
        raise ValueError("expected a %d-dimensional array, got %d dimensions" % (ndim, t.dim()))
    if cols is not None and t.dim() == 2 and t.shape[1] != cols and t.shape[0] > 0:
        raise ValueError("expected %d columns, got %d" % (cols, t.shape[1]))
    m = _grids._mgrid_class(ndim, "f")(*[int(d) for d in t.shape])
    if t.is_cuda:
        m.togpu()
    m.copyFrom(t.to(torch.float32).contiguous())
    return m


def _resized_copy(src, *shape):
    """Managed grid of the given shape holding the leading elements of src (flat order), on the
    side src is on (ManagedGrid::resized, include/libmolgrid/managed_grid.h)."""
    m = _grids._mgrid_class(len(shape), "f")(*shape)
    if src.ongpu():
        m.togpu()
    m.copyFrom(src)
    return m


class CoordinateSet(object):
    """Atoms of one molecule: ``coords`` (N,3), ``type_index`` (N, integers stored as floats) or
    ``type_vector`` (N,T), ``radii`` (N, or T once the radii are indexed by type), all managed
    grids that the set owns (include/libmolgrid/coordinateset.h:33-120).

      CoordinateSet()                                   empty
      CoordinateSet(coords, type_index, radii, max_type)
      CoordinateSet(coords, type_vector, radii)
      CoordinateSet(rec, lig, unique_index_types=True)  rec followed by lig

    Building one from a molecule file needs a chemistry toolkit and is outside the gridding path.
    """

    @_accepts_grids
    def __init__(self, *args, **kw):
        self.coords = _grids.MGrid2f(0, 3)
        self.type_index = _grids.MGrid1f(0)
        self.type_vector = _grids.MGrid2f(0, 0)
        self.radii = _grids.MGrid1f(0)
        self.max_type = 0
        self.src = None
        if not args and not kw:
            return
        if isinstance(args[0], CoordinateSet):
            names = ("rec", "lig", "unique_index_types")
            vals = dict(zip(names, args))
            vals.update(kw)
            self.mergeInto(vals["rec"], vals["lig"], vals.get("unique_index_types", True))
            return
        names = ("coords", "types", "radii", "max_type")
        vals = dict(zip(names, args))
        vals.update(kw)
        coords, types, radii = vals["coords"], vals["types"], vals["radii"]
        max_type = vals.get("max_type")
        tdim = len(tuple(types.shape))
        if tdim not in (1, 2):
            raise ValueError("types must be 1-D (indices) or 2-D (vectors)")
        n = tuple(coords.shape)[0]
        if tuple(types.shape)[0] != n:
            raise ValueError("Types and coordinates are of different sizes")
        self.coords = _managed(coords, 2, 3)
        self.radii = _managed(radii, 1)
        if tdim == 1:
            # src/coordinateset.cpp:124-128
            if max_type is None:
                raise ValueError("max_type is required with index types")
            if self.radii.size() != n:
                raise ValueError("Radii and coordinates are of different sizes")
            self.type_index = _managed(types, 1)
            self.max_type = int(max_type)
        else:
            # src/coordinateset.cpp:161-166
            self.type_vector = _managed(types, 2)
            self.max_type = int(tuple(types.shape)[1])

    # -- typing ---------------------------------------------------------------------------
    def has_indexed_types(self):
        return self.type_index.size() > 0 or self.coords.size() == 0

    def has_vector_types(self):
        return self.type_vector.size() > 0 or self.coords.size() == 0

    def make_vector_types(self, include_dummy_type=False, type_radii=()):
        """One-hot vectors from the index types, in place; with ``type_radii`` the radii become
        indexed by type (src/coordinateset.cpp:187-213)."""
        type_radii = [float(r) for r in type_radii]
        if type_radii and len(type_radii) != self.max_type:
            raise ValueError("Type radii size %d does not equal max type %d"
                             % (len(type_radii), self.max_type))
        if include_dummy_type:
            self.max_type += 1
        idx = self.type_index.tonumpy()
        n = idx.shape[0]
        vec = np.zeros((n, self.max_type), np.float32)
        t = idx.astype(np.int64)
        ok = (idx >= 0) & (t < self.max_type)
        vec[np.nonzero(ok)[0], t[ok]] = 1.0
        on_gpu = self.coords.ongpu()
        self.type_vector = _grids.MGrid2f(n, self.max_type)
        self.type_vector.copyFrom(vec)
        if on_gpu:
            self.type_vector.togpu()
        if type_radii:
            r = np.zeros(self.max_type, np.float32)
            r[:len(type_radii)] = type_radii
            self.radii = _grids.MGrid1f(self.max_type)
            self.radii.copyFrom(r)

    def num_types(self):
        return self.max_type

    def set_num_types(self, maxt):
        self.max_type = int(maxt)

    def sum_types(self, out, zerofirst=True):
        """out[t] (+)= number of atoms of type t, or the column sums of the type vectors
        (src/coordinateset.cpp:340-365)."""
        o = _unwrap(out)
        if tuple(o.shape) != (self.max_type,):
            raise ValueError("Type sum output dimension does not match number of types: %d vs %d"
                             % (tuple(o.shape)[0], self.max_type))
        if not (self.has_vector_types() and self.type_vector.size() > 0):
            t = np.round(self.type_index.tonumpy()).astype(np.int64)
            t = t[t >= 0]
            if t.size and t.max() >= self.max_type:
                raise IndexError("Somehow an index type is too large (internal error).")
            sums = np.bincount(t, minlength=self.max_type).astype(np.float32)
        else:
            sums = self.type_vector.tonumpy().sum(axis=0, dtype=np.float32)
        if isinstance(o, torch.Tensor):
            add = torch.from_numpy(sums).to(o.device, o.dtype)
            if zerofirst:
                o.copy_(add)
            else:
                o.add_(add)
        elif zerofirst:
            o[...] = sums
        else:
            o += sums

    # -- size, centre ---------------------------------------------------------------------
    def size(self):
        return self.coords.dimension(0)

    def __len__(self):
        return self.size()

    def center(self):
        """Mean coordinate, summed in float in atom order (src/coordinateset.cpp:214-229)."""
        n = self.size()
        if n == 0:
            return float3()
        c = self.coords.tonumpy()
        s = np.cumsum(c, axis=0, dtype=np.float32)[-1]
        return float3(*(s / np.float32(n)))

    # -- copies ---------------------------------------------------------------------------
    def clone(self):
        c = CoordinateSet()
        c.coords, c.type_index = self.coords.clone(), self.type_index.clone()
        c.type_vector, c.radii = self.type_vector.clone(), self.radii.clone()
        c.max_type, c.src = self.max_type, self.src
        return c

    def togpu(self, copy=True):
        for g in (self.coords, self.type_index, self.type_vector, self.radii):
            g.togpu()

    def tocpu(self, copy=True):
        for g in (self.coords, self.type_index, self.type_vector, self.radii):
            g.tocpu()

    def copyInto(self, other):
        c = other.clone()
        self.coords, self.type_index, self.type_vector = c.coords, c.type_index, c.type_vector
        self.radii, self.max_type, self.src = c.radii, c.max_type, c.src

    def copyTo(self, coords, types, radii):
        """Copy into the caller's arrays, truncating what does not fit and leaving what is beyond
        untouched; type vectors go row by row when the widths differ.  Returns the number of
        coordinates copied (src/coordinateset.cpp:300-337)."""
        c, t, r = _unwrap(coords), _unwrap(types), _unwrap(radii)
        if tuple(c.shape)[1] != 3:
            raise ValueError("Coordinates have wrong secondary dimension in copyTo")
        copied = self.coords.copyTo(c)
        self.radii.copyTo(r)
        if len(tuple(t.shape)) == 1:
            self.type_index.copyTo(t)
        elif self.type_vector.size() > 0 and tuple(t.shape)[1] != self.type_vector.dimension(1):
            src = _grids._tensor_of(self.type_vector)
            dst = t if isinstance(t, torch.Tensor) else torch.from_numpy(t)
            rows = min(dst.shape[0], src.shape[0])
            cols = min(dst.shape[1], src.shape[1])
            dst[:rows, :cols].copy_(src[:rows, :cols])
        else:
            self.type_vector.copyTo(t)
        return copied // 3

    def mergeInto(self, rec, lig, unique_index_types=True):
        """This set becomes rec followed by lig; with unique_index_types the index types of lig
        are shifted past those of rec (src/coordinateset.cpp:258-298)."""
        if rec.type_vector.dimension(1) != lig.type_vector.dimension(1):
            raise ValueError("Type vectors are incompatible sizes")
        if (rec.has_vector_types() != lig.has_vector_types()) and \
                (rec.has_indexed_types() != lig.has_indexed_types()):
            raise ValueError("Incompatible types when combining coodinate sets")
        if rec.has_indexed_types():
            max_type = rec.max_type + lig.max_type if unique_index_types \
                else max(rec.max_type, lig.max_type)
        else:
            if rec.max_type != lig.max_type:
                raise ValueError("Type vectors are incompatible sizes, weirdly")
            max_type = self.max_type
        on_gpu = rec.coords.ongpu()

        def joined(a, b, ndim, cols=None):
            x, y = a.tonumpy(), b.tonumpy()
            if ndim == 2:
                x = x.reshape(x.shape[0], cols)
                y = y.reshape(y.shape[0], cols)
            m = _managed(np.concatenate([x, y]), ndim)
            if on_gpu:
                m.togpu()
            return m

        nr = rec.type_index.size()
        coords = joined(rec.coords, lig.coords, 2, 3)
        tindex = np.concatenate([rec.type_index.tonumpy(), lig.type_index.tonumpy()])
        if unique_index_types:
            tindex[nr:] += np.float32(rec.max_type)
        tvec = joined(rec.type_vector, lig.type_vector, 2, rec.type_vector.dimension(1))
        radii = joined(rec.radii, lig.radii, 1)
        self.coords, self.type_vector, self.radii = coords, tvec, radii
        self.type_index = _managed(tindex, 1)
        if on_gpu:
            self.type_index.togpu()
        self.max_type = max_type

    def __eq__(self, other):
        if not isinstance(other, CoordinateSet):
            return NotImplemented
        return (self.max_type == other.max_type and
                all(np.array_equal(a.tonumpy(), b.tonumpy()) for a, b in (
                    (self.coords, other.coords), (self.type_index, other.type_index),
                    (self.type_vector, other.type_vector), (self.radii, other.radii))))

    __hash__ = None


class Example(object):
    """The coordinate sets (receptor, ligand, ...) and labels of one training example
    (include/libmolgrid/example.h:29-110)."""

    def __init__(self):
        self.coord_sets = []
        self.labels = []
        self.group = -1
        self.seqcont = False

    @property
    def sets(self):
        return self.coord_sets

    def num_coordinates(self):
        return sum(c.size() for c in self.coord_sets)

    def num_types(self, unique_index_type=True):
        if unique_index_type:
            return sum(c.max_type for c in self.coord_sets)
        return max([c.max_type for c in self.coord_sets] + [0])

    def has_vector_types(self, start=0):
        return all(c.has_vector_types() for c in self.coord_sets[start:] if c.size() > 0)

    def has_index_types(self, start=0):
        return all(c.has_indexed_types() for c in self.coord_sets[start:] if c.size() > 0)

    def togpu(self):
        for c in self.coord_sets:
            c.togpu()

    def tocpu(self):
        for c in self.coord_sets:
            c.tocpu()

    def _merged_arrays(self, start, unique_index_types, vector):
        """coords, types, radii of the sets from `start` on as numpy arrays
        (src/example.cpp:69-100 and 138-195)."""
        sets = self.coord_sets[start:]
        if not vector:
            coords, types, radii, toffset = [], [], [], 0
            for cs in sets:
                if cs.size() == 0:
                    continue
                if not cs.has_indexed_types():
                    raise RuntimeError("Coordinate sets do not have compatible index types for merge.")
                coords.append(cs.coords.tonumpy())
                types.append(cs.type_index.tonumpy() + np.float32(toffset))
                radii.append(cs.radii.tonumpy())
                if unique_index_types:
                    toffset += cs.max_type
            if not coords:
                return (np.zeros((0, 3), np.float32), np.zeros(0, np.float32),
                        np.zeros(0, np.float32))
            return np.concatenate(coords), np.concatenate(types), np.concatenate(radii)
        maxt = 0
        for i, cs in enumerate(sets):
            maxt = maxt + cs.max_type if unique_index_types else max(maxt, cs.max_type)
            if cs.size() == 0:
                continue
            if not cs.has_vector_types():
                raise RuntimeError("Coordinate sets do not have compatible vector types for merge.")
            if cs.max_type != cs.type_vector.dimension(1):
                raise RuntimeError("Coordinate set %d does not have consistent max_type/vector "
                                   "type sizes" % (start + i))
        coords, types, radii, offset = [], [], [], 0
        for cs in sets:
            n = cs.size()
            tv = cs.type_vector.tonumpy()
            tv = tv.reshape(n, tv.shape[1] if tv.ndim == 2 else 0)
            if offset + tv.shape[1] > maxt and n > 0:
                raise RuntimeError("Incompatible vector sizes in merge_coordinates")
            block = np.zeros((n, maxt), np.float32)
            block[:, offset:offset + tv.shape[1]] = tv
            coords.append(cs.coords.tonumpy().reshape(n, 3))
            types.append(block)
            radii.append(cs.radii.tonumpy())
            if unique_index_types:
                offset += cs.max_type
        if not coords:
            return (np.zeros((0, 3), np.float32), np.zeros((0, maxt), np.float32),
                    np.zeros(0, np.float32))
        return np.concatenate(coords), np.concatenate(types), np.concatenate(radii)

    def merge_coordinates(self, *args, **kw):
        """merge_coordinates(start=0, unique_index_types=True) -> CoordinateSet
        merge_coordinates(coord, types, radius, start=0, unique_index_types=True)   fills arrays
        (src/example.cpp:40-67, 102-136 and 197-228)."""
        if args and not isinstance(args[0], (int, bool)):
            names = ("coord", "types", "radius", "start", "unique_index_types")
            vals = dict(zip(names, args))
            vals.update(kw)
            c, t, r = _unwrap(vals["coord"]), _unwrap(vals["types"]), _unwrap(vals["radius"])
            vector = len(tuple(t.shape)) == 2
            coords, types, radii = self._merged_arrays(vals.get("start", 0),
                                                       vals.get("unique_index_types", True), vector)
            if vector and types.shape[0] == 0:
                return
            if tuple(c.shape)[0] != coords.shape[0]:
                raise ValueError("Coordinates do not have correct dimension: %d != %d"
                                 % (tuple(c.shape)[0], coords.shape[0]))
            if tuple(c.shape)[1] != 3:
                raise ValueError("Coordinates do not have correct second dimension (3): %d"
                                 % tuple(c.shape)[1])
            if tuple(t.shape) != types.shape:
                raise ValueError("Types do not have correct dimension: %r != %r"
                                 % (tuple(t.shape), types.shape))
            if tuple(r.shape)[0] != radii.shape[0]:
                raise ValueError("Radii do not have correct dimension: %d != %d"
                                 % (tuple(r.shape)[0], radii.shape[0]))
            for dst, src in ((c, coords), (t, types), (r, radii)):
                if isinstance(dst, torch.Tensor):
                    dst.copy_(torch.from_numpy(src))
                else:
                    dst[...] = src
            return
        names = ("start", "unique_index_types")
        vals = dict(zip(names, args))
        vals.update(kw)
        start, unique = int(vals.get("start", 0)), bool(vals.get("unique_index_types", True))
        has_vec, has_ind = self.has_vector_types(), self.has_index_types()
        if not has_ind and not has_vec:
            raise ValueError("Inconsistent typing schemes in merge_coordinates")
        if len(self.coord_sets) <= start:
            return CoordinateSet()
        if len(self.coord_sets) == start + 1:
            return self.coord_sets[start].clone()
        if not has_vec:
            coords, types, radii = self._merged_arrays(start, unique, False)
            return CoordinateSet(coords, types, radii, self.num_types(unique))
        coords, types, radii = self._merged_arrays(start, unique, True)
        return CoordinateSet(coords, types, radii)

    def sum_types(self, out, unique_types=True):
        """src/example.cpp:345-368"""
        o = _unwrap(out)
        nt = self.num_types(unique_types)
        if tuple(o.shape) != (nt,):
            raise ValueError("Size of sum output doesn't match number of types in example: %d vs %d"
                             % (tuple(o.shape)[0], nt))
        if not unique_types:
            o[...] = 0
            for cs in self.coord_sets:
                if cs.num_types() == nt:
                    cs.sum_types(o, False)
                else:
                    part = np.zeros(cs.num_types(), np.float32)
                    cs.sum_types(part)
                    if isinstance(o, torch.Tensor):
                        o[:part.shape[0]] += torch.from_numpy(part).to(o.device)
                    else:
                        o[:part.shape[0]] += part
            return
        offset = 0
        for cs in self.coord_sets:
            n = cs.num_types()
            if n == 0:
                continue
            cs.sum_types(o[offset:offset + n])
            offset += n


class ExampleVec(list):
    """A batch of examples, as ExampleProvider.next_batch returns it (python/bindings.in.cpp)."""

    def extract_labels(self, out):
        """out[i, :] = labels of example i (src/example.cpp:254-272)."""
        o = _unwrap(out)
        if tuple(o.shape)[0] != len(self):
            raise IndexError("Grid dimension does not match number of examples: %d vs %d"
                             % (tuple(o.shape)[0], len(self)))
        if not self:
            return
        nlabels = len(self[0].labels)
        if tuple(o.shape)[1] != nlabels:
            raise IndexError("Grid dimension does not match number of labels: %d vs %d"
                             % (nlabels, tuple(o.shape)[1]))
        if any(len(ex.labels) != nlabels for ex in self):
            raise RuntimeError("Non-uniform number of labels")
        vals = np.asarray([ex.labels for ex in self], np.float32).reshape(len(self), nlabels)
        if isinstance(o, torch.Tensor):
            o.copy_(torch.from_numpy(vals))
        else:
            o[...] = vals

    def sum_types(self, out, unique_types=True):
        """out[i, :] = type sums of example i (python/bindings.in.cpp:384-393)."""
        o = _unwrap(out)
        if tuple(o.shape)[0] != len(self):
            raise ValueError("Size of example vector does not match sum grid: %d vs %d"
                             % (len(self), tuple(o.shape)[0]))
        for i, ex in enumerate(self):
            ex.sum_types(o[i], unique_types)

    def extract_label(self, labelpos, out):
        """out[i] = label `labelpos` of example i (src/example.cpp:278-299)."""
        o = _unwrap(out)
        if tuple(o.shape)[0] != len(self):
            raise IndexError("Grid dimension does not match number of examples")
        if not self:
            return
        if labelpos >= len(self[0].labels):
            raise IndexError("labelpos invalid: %d >= %d" % (labelpos, len(self[0].labels)))
        if any(labelpos >= len(ex.labels) for ex in self):
            raise IndexError("labelpos invalid (nonuniform labels)")
        vals = np.asarray([ex.labels[labelpos] for ex in self], np.float32)
        if isinstance(o, torch.Tensor):
            o.copy_(torch.from_numpy(vals))
        else:
            o[...] = vals


# --------------------------------------------------------------------------- #
# GridMaker
# --------------------------------------------------------------------------- #
class GridMaker(object):
    """Atoms -> density grid and grid gradient -> atom gradients.

    Same constructor arguments and defaults as the reference's Python class
    (python/bindings.in.cpp:816-817).
    """

    def __init__(self, resolution=0.5, dimension=23.5, binary=False, radius_type_indexed=False,
                 radius_scale=1.0, gaussian_radius_multiple=1.0):
        self._radius_scale = float(radius_scale)
        self._grm_arg = float(gaussian_radius_multiple)
        self._p = _capi.mg_gridmaker()
        self._init(resolution, dimension, binary, radius_type_indexed)

    def _init(self, resolution, dimension, binary, rti):
        _capi.check(_lib.mg_gridmaker_init(self._p, resolution, dimension, int(bool(binary)),
                                           int(bool(rti)), self._radius_scale, self._grm_arg),
                    "GridMaker")

    # -- accessors (grid_maker.h:88-116) ------------------------------------
    def get_resolution(self):
        return float(self._p.resolution)

    def set_resolution(self, res):
        self._init(res, self._p.dimension, self._p.binary, self._p.radii_type_indexed)

    def get_dimension(self):
        return float(self._p.dimension)

    def set_dimension(self, d):
        self._init(self._p.resolution, d, self._p.binary, self._p.radii_type_indexed)

    def get_binary(self):
        return bool(self._p.binary)

    def set_binary(self, b):
        self._p.binary = int(bool(b))

    def get_radii_type_indexed(self):
        return bool(self._p.radii_type_indexed)

    def set_radii_type_indexed(self, b):
        self._p.radii_type_indexed = int(bool(b))

    def get_radiusmultiple(self):
        return float(_f32(self._p.radius_scale) * _f32(self._p.final_radius_multiple))

    def get_first_dim(self):
        return int(self._p.dim)

    def spatial_grid_dimensions(self):
        d = int(self._p.dim)
        return (d, d, d)

    def grid_dimensions(self, ntypes):
        d = int(self._p.dim)
        return (int(ntypes), d, d, d)

    def get_grid_origin(self, center):
        c = _to_float3(center)
        half = _f32(float(self._p.dimension) / 2.0)
        return float3(_f32(c.x) - half, _f32(c.y) - half, _f32(c.z) - half)

    # -- argument checks ----------------------------------------------------
    def _check_grid(self, shape, what="Output"):
        dim = int(self._p.dim)
        for ax in (1, 2, 3):
            if shape[ax] != dim:
                raise IndexError("%s grid dimension incorrect: %d vs %d" % (what, dim, shape[ax]))

    def _check_index_args(self, n, types, radii, out_shape):
        # src/grid_maker.cpp:39-54
        self._check_grid(out_shape)
        if types.shape[0] != n:
            raise IndexError("type_index does not match number of atoms: %d vs %d"
                             % (types.shape[0], n))
        if radii.shape[0] != n:
            raise IndexError("radii does not match number of atoms: %d vs %d"
                             % (radii.shape[0], n))

    def _check_vector_args(self, n, types, radii, out_shape):
        # src/grid_maker.cpp:66-89
        self._check_grid(out_shape)
        T = types.shape[1]
        if types.shape[0] != n:
            raise IndexError("type_vector does not match number of atoms: %d vs %d"
                             % (types.shape[0], n))
        if T != out_shape[0]:
            raise IndexError("number of types in type_vector does not match number of output "
                             "channels: %d vs %d" % (T, out_shape[0]))
        want = T if self._p.radii_type_indexed else n
        if radii.shape[0] != want:
            raise IndexError("radii does not match number of %s: %d vs %d"
                             % ("types" if self._p.radii_type_indexed else "atoms",
                                radii.shape[0], want))

    @staticmethod
    def _check_host_types(types_user, ntypes):
        """The CPU overload throws for an index >= ntypes (src/grid_maker.cpp:172); the
        check is made for host arrays, where it costs no device synchronisation."""
        if _is_host(types_user):
            t = np.asarray(types_user.detach().numpy() if isinstance(types_user, torch.Tensor)
                           else types_user)
            if t.size and np.floor(t).max() >= ntypes:
                raise IndexError("Type index %d larger than allowed %d"
                                 % (int(np.floor(t).max()), ntypes))

    def _forward_index_call(self, batch=None, vector=False):
        """mg_forward_index_ws (mg_forward_vector_ws) with a workspace from torch's allocator
        (which is stream aware); a ragged batch layout (AtomBatch) keeps its workspace for the
        next call."""
        size_of = _lib.mg_forward_vector_workspace_size if vector else \
            _lib.mg_forward_index_workspace_size
        entry = _lib.mg_forward_vector_ws if vector else _lib.mg_forward_index_ws
        name = "forward_vector_ws" if vector else "forward_index_ws"

        def call(p, B, off, n, cen, chost, coords, types, radii, T, out, stream):
            need = int(size_of(p, B, n, T))
            ws = None
            if need:
                # one workspace per device AND stream: calls on two streams may overlap
                key = (name, torch.cuda.current_device(), stream)
                ws = batch.scratch.get(key) if batch is not None else None
                if ws is None or ws.numel() < need:
                    ws = torch.empty(need, dtype=torch.uint8, device=_device())
                    if batch is not None:
                        batch.scratch[key] = ws
            return entry(p, B, off, n, cen, chost, coords, types, radii, T, out,
                         ws.data_ptr() if ws is not None else None, need, stream)
        return call

    # -- forward ------------------------------------------------------------
    @_accepts_grids
    def forward(self, *args, **kw):
        """forward(center, coordinate_set, grid)
        forward(center, coords, types, radii, grid)          one example
        forward(centers, coords, types, radii, grid)         padded batch (B leading)
        forward(example, transform, grid)                    grid centred at the rotation centre
        forward(example, grid, random_translation=0, random_rotation=False, center=None)
        forward(examples, grid5, random_translation=0, random_rotation=False)
        ``types`` is 1-D per example for index types, 2-D for type vectors."""
        if args and isinstance(args[0], Example):
            if len(args) >= 3 and isinstance(args[1], Transform):
                if kw or len(args) != 3:
                    raise TypeError("forward(example, transform, grid) expected")
                return self._forward_example(args[0], args[1], args[2])
            names = ("grid", "random_translation", "random_rotation", "center")
            vals = dict(zip(names, args[1:]))
            vals.update(kw)
            t = Transform(self._example_center(args[0], vals.get("center")),
                          vals.get("random_translation", 0.0), vals.get("random_rotation", False))
            return self._forward_example(args[0], t, vals["grid"])
        if args and isinstance(args[0], (list, tuple)) and \
                (len(args[0]) == 0 or isinstance(args[0][0], Example)):
            names = ("grid", "random_translation", "random_rotation")
            vals = dict(zip(names, args[1:]))
            vals.update(kw)
            return self._forward_examples(args[0], vals["grid"],
                                          vals.get("random_translation", 0.0),
                                          vals.get("random_rotation", False))
        if kw:
            raise TypeError("forward takes positional arguments only")
        if len(args) == 3:
            center, cs, grid = args
            if not isinstance(cs, CoordinateSet):
                raise TypeError("forward(center, CoordinateSet, grid) expected")
            types = cs.type_vector if cs.has_vector_types() and cs.size() > 0 else cs.type_index
            return self.forward(center, cs.coords, types, cs.radii, grid)
        if len(args) != 5:
            raise TypeError("forward expects 3 or 5 arguments")
        center, coords, types, radii, grid = args
        if len(tuple(coords.shape)) == 3:
            return self._forward_padded(center, coords, types, radii, grid)
        c = _to_float3(center)
        a_coords = _Arg(coords, "coords", 2)
        tdim = len(tuple(types.shape))
        a_types = _Arg(types, "types", tdim)
        a_radii = _Arg(radii, "radii", 1)
        a_out = _Arg(grid, "grid", 4, out=True, wide=True)
        n = a_coords.shape[0]
        if tdim == 1:
            self._check_index_args(n, a_types, a_radii, a_out.shape)
            if self._p.radii_type_indexed:
                raise ValueError("Type indexed radii not supported with index types.")
            self._check_host_types(types, a_out.shape[0])
            fn = self._forward_index_call()
        else:
            self._check_vector_args(n, a_types, a_radii, a_out.shape)
            fn = self._forward_index_call(vector=True)
        code = fn(self._p, 1, None, n, None, _capi.f3(c), a_coords.ptr, a_types.ptr, a_radii.ptr,
                  a_out.shape[0], a_out.ptr, _stream())
        _capi.check(code, "GridMaker.forward")
        a_out.finish()

    @staticmethod
    def _example_center(ex, center):
        """Centre of the last coordinate set, unless every set is empty or one is given
        (src/grid_maker.cpp:120-133)."""
        if center is not None:
            c = _to_float3(center)
            if not math.isinf(c.x):
                return c
        c = float3()
        for cs in reversed(ex.coord_sets):
            c = float3()
            if cs.size():
                c = ex.coord_sets[-1].center()
                break
        return c

    def _forward_example(self, ex, transform, grid):
        # src/grid_maker.cpp:108-115: merge (a copy), transform the copy, grid about the centre
        c = ex.merge_coordinates()
        g = _unwrap(grid)
        if c.max_type != tuple(g.shape)[0]:
            raise IndexError("Incorrect number of channels in output grid: %d vs %d"
                             % (c.max_type, tuple(g.shape)[0]))
        if not _is_host(g):
            c.togpu()
        transform.forward(c, c)
        self.forward(transform.get_rotation_center(), c, grid)

    def _forward_examples(self, examples, grid, random_translation, random_rotation):
        """include/libmolgrid/grid_maker.h:194-201.  The transforms are drawn example by example,
        as the reference's loop does; index-typed examples are then packed and gridded with one
        transform launch and one forward launch for the whole batch."""
        g = _unwrap(grid)
        if len(examples) != tuple(g.shape)[0]:
            raise IndexError("output grid dimension does not match size of example vector")
        transforms = [Transform(self._example_center(ex, None), random_translation,
                                random_rotation) for ex in examples]
        merged = [ex.merge_coordinates() for ex in examples]
        packable = len(examples) > 1 and len(tuple(g.shape)) == 5 and all(
            m.size() > 0 and m.type_index.size() > 0 and m.max_type == tuple(g.shape)[1]
            for m in merged) and not self._p.radii_type_indexed
        if not packable:
            for i, (ex, t) in enumerate(zip(examples, transforms)):
                self._forward_example(ex, t, g[i])
            return
        offsets = np.zeros(len(merged) + 1, np.int64)
        offsets[1:] = np.cumsum([m.size() for m in merged])
        coords = np.concatenate([m.coords.tonumpy() for m in merged])
        types = np.concatenate([m.type_index.tonumpy() for m in merged])
        radii = np.concatenate([m.radii.tonumpy() for m in merged])
        quats = np.asarray([t.get_quaternion().as_tuple() for t in transforms], np.float32)
        centers = np.asarray([tuple(t.get_rotation_center()) for t in transforms], np.float32)
        shifts = np.asarray([tuple(t.get_translation()) for t in transforms], np.float32)
        batch = AtomBatch(offsets)
        dev_coords = torch.from_numpy(coords).to(_device())
        transform_batch(batch, quats, centers, shifts, dev_coords, dev_coords)
        self.forward_batch(batch, centers, dev_coords, torch.from_numpy(types).to(_device()),
                           torch.from_numpy(radii).to(_device()), grid)

    def _forward_padded(self, centers, coords, types, radii, grid):
        # include/libmolgrid/grid_maker.h:265-301; one centre for all examples is accepted too
        one_center = not hasattr(centers, "shape") or len(tuple(centers.shape)) == 1
        chost = _capi.f3(_to_float3(centers)) if one_center else _capi.f3(_Z3)
        a_coords = _Arg(coords, "coords", 3)
        a_centers = _Shape((a_coords.shape[0], 3)) if one_center else _Arg(centers, "centers", 2)
        tdim = len(tuple(types.shape))
        if tdim not in (2, 3):
            raise ValueError("Unsupported types dimension")
        a_types = _Arg(types, "types", tdim)
        a_radii = _Arg(radii, "radii", 2)
        a_out = _Arg(grid, "grid", 5, out=True, wide=True)
        B = a_centers.shape[0]
        for a in (a_coords, a_types, a_radii, a_out):
            if a.shape[0] != B:
                raise ValueError("Mismatched batch sizes: %d vs %d" % (a.shape[0], B))
        n = a_coords.shape[1]
        if tdim == 2:
            self._check_index_args(n, _Shape(a_types.shape[1:]), _Shape(a_radii.shape[1:]),
                                   a_out.shape[1:])
            if self._p.radii_type_indexed:
                raise ValueError("Type indexed radii not supported with index types.")
            self._check_host_types(types, a_out.shape[1])
            fn = self._forward_index_call()
        else:
            self._check_vector_args(n, _Shape(a_types.shape[1:]), _Shape(a_radii.shape[1:]),
                                    a_out.shape[1:])
            fn = self._forward_index_call(vector=True)
        code = fn(self._p, B, None, n, None if one_center else a_centers.ptr, chost, a_coords.ptr,
                  a_types.ptr, a_radii.ptr, a_out.shape[1], a_out.ptr, _stream())
        _capi.check(code, "GridMaker.forward")
        a_out.finish()

    @_accepts_grids
    def forward_batch(self, offsets, centers, coords, types, radii, grid):
        """Ragged batch in one launch: example b owns atoms offsets[b]:offsets[b+1] of the
        packed arrays; centers (B,3); grid (B,T,D,D,D).  With type-indexed radii,
        ``radii`` is (B,T)."""
        off, B, largest, total = _offsets_arg(offsets)
        cen = _small_device(centers, 3)
        a_coords = _Arg(coords, "coords", 2)
        tdim = len(tuple(types.shape))
        a_types = _Arg(types, "types", tdim)
        rti = bool(self._p.radii_type_indexed)
        a_radii = _Arg(radii, "radii", 2 if rti else 1)
        a_out = _Arg(grid, "grid", 5, out=True, wide=True)
        if cen.shape[0] != B or a_out.shape[0] != B:
            raise ValueError("Mismatched batch sizes: %d vs %d" % (a_out.shape[0], B))
        if a_coords.shape[0] < total or a_types.shape[0] < total:
            raise IndexError("atom arrays are shorter than offsets[-1]")
        self._check_grid(a_out.shape[1:])
        T = a_out.shape[1]
        if tdim == 1:
            if rti:
                raise ValueError("Type indexed radii not supported with index types.")
            if a_radii.shape[0] < total:
                raise IndexError("radii does not match number of atoms")
            self._check_host_types(types, T)
            fn = self._forward_index_call(offsets if isinstance(offsets, AtomBatch) else None)
        else:
            if a_types.shape[1] != T:
                raise IndexError("number of types in type_vector does not match number of "
                                 "output channels: %d vs %d" % (a_types.shape[1], T))
            if rti and a_radii.shape != (B, T):
                raise IndexError("radii does not match number of types")
            if not rti and a_radii.shape[0] < total:
                raise IndexError("radii does not match number of atoms")
            fn = self._forward_index_call(offsets if isinstance(offsets, AtomBatch) else None,
                                          vector=True)
        code = fn(self._p, B, _ptr(off), largest, _ptr(cen), _capi.f3(_Z3), a_coords.ptr,
                  a_types.ptr, a_radii.ptr, T, a_out.ptr, _stream())
        _capi.check(code, "GridMaker.forward_batch")
        a_out.finish()

    @_accepts_grids
    def sort_batch(self, offsets, centers, coords, types, radii, ntypes):
        """First half of ``forward_batch`` for index types: sorts the atoms of a ragged batch
        into a device workspace and returns it as a ``SortedBatch``; ``splat_batch`` turns it
        into grids.  The two halves may be enqueued on different streams (the caller orders the
        splat after the sort, e.g. with an event), which takes the sort launch off the critical
        path when other work -- the backward pass -- can run beside it.  The grids are those of
        ``forward_batch`` bit for bit."""
        off, B, largest, total = _offsets_arg(offsets)
        cen = _small_device(centers, 3)
        a_coords, a_types, a_radii = _Arg(coords, "coords", 2), _Arg(types, "types", 1), \
            _Arg(radii, "radii", 1)
        if self._p.radii_type_indexed:
            raise ValueError("Type indexed radii not supported with index types.")
        if cen.shape[0] != B:
            raise ValueError("Mismatched batch sizes: %d vs %d" % (cen.shape[0], B))
        if a_coords.shape[0] < total or a_types.shape[0] < total or a_radii.shape[0] < total:
            raise IndexError("atom arrays are shorter than offsets[-1]")
        T = int(ntypes)
        self._check_host_types(types, T)
        need = int(_lib.mg_forward_index_workspace_size(self._p, B, largest, T))
        ws = torch.empty(max(need, 1), dtype=torch.uint8, device=_device())
        code = _lib.mg_forward_index_sort(self._p, B, _ptr(off), largest, _ptr(cen), _capi.f3(_Z3),
                                          a_coords.ptr, a_types.ptr, a_radii.ptr, T,
                                          ws.data_ptr(), need, _stream())
        _capi.check(code, "GridMaker.sort_batch")
        return SortedBatch(ws, need, B, largest, T)

    @_accepts_grids
    def splat_batch(self, sorted_batch, grid):
        """Second half of ``forward_batch``: the grids (B,T,D,D,D) of a ``SortedBatch``."""
        a_out = _Arg(grid, "grid", 5, out=True, wide=True)
        sb = sorted_batch
        if a_out.shape[0] != sb.nbatch or a_out.shape[1] != sb.ntypes:
            raise ValueError("grid is %s but the atoms were sorted for %d examples and %d types"
                             % (a_out.shape, sb.nbatch, sb.ntypes))
        self._check_grid(a_out.shape[1:])
        # the workspace may have been allocated under another stream: tell the allocator that
        # this stream uses it too
        sb.workspace.record_stream(torch.cuda.current_stream())
        code = _lib.mg_forward_index_splat(self._p, sb.nbatch, sb.largest, sb.ntypes, a_out.ptr,
                                           sb.workspace.data_ptr(), sb.nbytes, _stream())
        _capi.check(code, "GridMaker.splat_batch")
        a_out.finish()

    # -- backward -----------------------------------------------------------
    @_accepts_grids
    def backward(self, *args):
        """backward(center, coordinate_set, diff, atom_gradients[, type_gradients])
        backward(center, coords, type_index, radii, diff, atom_gradients)
        backward(center, coords, type_vectors, radii, diff, atom_gradients, type_gradients)"""
        if len(args) in (4, 5) and isinstance(args[1], CoordinateSet):
            center, cs, diff = args[:3]
            if len(args) == 5:
                if not cs.has_vector_types():
                    raise ValueError("Vector types missing from coordinate set")
                return self.backward(center, cs.coords, cs.type_vector, cs.radii, diff, args[3],
                                     args[4])
            if not cs.has_indexed_types():
                raise ValueError("Index types missing from coordinate set")
            return self.backward(center, cs.coords, cs.type_index, cs.radii, diff, args[3])
        if len(args) not in (6, 7):
            raise TypeError("backward expects 4 to 7 arguments")
        center, coords, types, radii, diff, agrad = args[:6]
        if len(tuple(coords.shape)) == 3:
            return self._backward_padded(*args)
        c = _to_float3(center)
        a_coords = _Arg(coords, "coords", 2)
        tdim = len(tuple(types.shape))
        a_types = _Arg(types, "types", tdim)
        a_radii = _Arg(radii, "radii", 1)
        a_diff = _Arg(diff, "diff", 4, wide=True)
        a_ag = _Arg(agrad, "atom_gradients", 2, out=True, wide=True)
        n = a_coords.shape[0]
        dim = int(self._p.dim)
        if tdim == 1:
            if len(args) != 6:
                raise TypeError("index types take no type_gradients argument")
            # src/grid_maker.cpp:442-452
            if self._p.radii_type_indexed:
                raise ValueError("Type indexed radii not supported with index types.")
            if n != a_types.shape[0]:
                raise ValueError("Type dimension doesn't equal number of coordinates.")
            if n != a_ag.shape[0]:
                raise ValueError("Gradient dimension doesn't equal number of coordinates")
            if n != a_radii.shape[0]:
                raise ValueError("Radii dimension doesn't equal number of coordinates")
            if a_coords.shape[1] != 3 or a_ag.shape[1] != 3:
                raise ValueError("Need x,y,z,r for coord_radius")
            for ax in (1, 2, 3):
                if a_diff.shape[ax] != dim:
                    raise ValueError("diff does not have correct dimension %d: %d vs %d"
                                     % (ax, a_diff.shape[ax], dim))
            if _is_host(types):
                t = np.asarray(a_types.host.numpy())
                if t.size and np.round(t).max() >= a_diff.shape[0]:
                    raise ValueError("Incorrect channel size for diff: %d vs %d"
                                     % (int(np.round(t).max()), a_diff.shape[0]))
            code = _lib.mg_backward_index(self._p, 1, None, n, None, _capi.f3(c), a_coords.ptr,
                                          a_types.ptr, a_radii.ptr, a_diff.shape[0], a_diff.ptr,
                                          a_ag.ptr, _stream())
            _capi.check(code, "GridMaker.backward")
            a_ag.finish()
            return
        if len(args) != 7:
            raise TypeError("vector types need a type_gradients argument")
        a_tg = _Arg(args[6], "type_gradients", 2, out=True, wide=True)
        T = a_types.shape[1]
        # src/grid_maker.cpp:487-498
        if n != a_types.shape[0]:
            raise ValueError("Type dimension doesn't equal number of coordinates.")
        if T != a_diff.shape[0]:
            raise ValueError("Channels in diff doesn't equal number of types")
        if n != a_ag.shape[0]:
            raise ValueError("Atom gradient dimension doesn't equal number of coordinates")
        if n != a_tg.shape[0]:
            raise ValueError("Type gradient dimension doesn't equal number of coordinates")
        if a_tg.shape[1] != T:
            raise ValueError("Type gradient dimension has wrong number of types")
        if a_coords.shape[1] != 3 or a_ag.shape[1] != 3:
            raise ValueError("Need x,y,z,r for coord_radius")
        if self._p.radii_type_indexed:
            if T != a_radii.shape[0]:
                raise ValueError("Radii dimension doesn't equal number of types")
        elif n != a_radii.shape[0]:
            raise ValueError("Radii dimension doesn't equal number of coordinates")
        for ax in (1, 2, 3):
            if a_diff.shape[ax] != dim:
                raise ValueError("diff does not have correct dimension %d: %d vs %d"
                                 % (ax, a_diff.shape[ax], dim))
        code = _lib.mg_backward_vector(self._p, 1, None, n, None, _capi.f3(c), a_coords.ptr,
                                       a_types.ptr, a_radii.ptr, T, a_diff.ptr, a_ag.ptr,
                                       a_tg.ptr, _stream())
        _capi.check(code, "GridMaker.backward")
        a_ag.finish()
        a_tg.finish()

    @_accepts_grids
    def backward_relevance(self, *args):
        """backward_relevance(center, coordinate_set, density, diff, relevance)
        backward_relevance(center, coords, type_index, radii, density, diff, relevance)

        include/libmolgrid/grid_maker.h:558-618; values of src/grid_maker.cpp:392-432, 680-704."""
        if len(args) == 5 and isinstance(args[1], CoordinateSet):
            center, cs, density, diff, relevance = args
            if not cs.has_indexed_types():
                raise ValueError("Index types missing from coordinate set in backward relevance")
            return self.backward_relevance(center, cs.coords, cs.type_index, cs.radii, density,
                                           diff, relevance)
        if len(args) != 7:
            raise TypeError("backward_relevance expects 5 or 7 arguments")
        center, coords, types, radii, density, diff, relevance = args
        c = _to_float3(center)
        a_coords = _Arg(coords, "coords", 2)
        a_types = _Arg(types, "type_index", 1)
        a_radii = _Arg(radii, "radii", 1)
        a_dens = _Arg(density, "density", 4, wide=True)
        a_diff = _Arg(diff, "diff", 4, wide=True)
        a_rel = _Arg(relevance, "relevance", 1, out=True, wide=True)
        n = a_coords.shape[0]
        # src/grid_maker.cu:975-978
        if n != a_types.shape[0]:
            raise ValueError("Type dimension doesn't equal number of coordinates.")
        if n != a_rel.shape[0]:
            raise ValueError("Relevance dimension doesn't equal number of coordinates")
        if n != a_radii.shape[0]:
            raise ValueError("Radii dimension doesn't equal number of coordinates")
        if a_coords.shape[1] != 3:
            raise ValueError("Coordinates and radius wrong secondary dimension")
        dim = int(self._p.dim)
        if a_dens.shape != a_diff.shape or tuple(a_diff.shape[1:]) != (dim, dim, dim):
            raise ValueError("density and diff must both be (ntypes, %d, %d, %d)" % (dim, dim, dim))
        code = _lib.mg_backward_relevance(self._p, 1, None, n, None, _capi.f3(c), a_coords.ptr,
                                          a_types.ptr, a_radii.ptr, a_diff.shape[0], a_dens.ptr,
                                          a_diff.ptr, a_rel.ptr, _stream())
        _capi.check(code, "GridMaker.backward_relevance")
        a_rel.finish()

    @_accepts_grids
    def backward_gradients(self, *args):
        """backward_gradients(center, coords, type_vectors, radii, diff, atom_gradients,
                              type_gradients, diffdiff, atom_diffdiff, type_diffdiff)
        backward_gradients(center, coordinate_set, diff, atom_gradients, type_gradients,
                           diffdiff, atom_diffdiff, type_diffdiff)

        Gradients of the backward pass (include/libmolgrid/grid_maker.h:447-545, values of
        src/grid_maker.cpp:529-661): given gradients with respect to the atom and type gradients,
        fills the gradient with respect to diff, to the coordinates and to the types (zero)."""
        if len(args) == 8 and isinstance(args[1], CoordinateSet):
            cs = args[1]
            if not cs.has_vector_types():
                raise ValueError("Vector types missing from coordinate set")
            return self.backward_gradients(args[0], cs.coords, cs.type_vector, cs.radii, *args[2:])
        if len(args) != 10:
            raise TypeError("backward_gradients expects 8 or 10 arguments")
        center, coords, types, radii, diff, agrad, tgrad, diffdiff, add, tdd = args
        c = _to_float3(center)
        a_coords = _Arg(coords, "coords", 2)
        a_types = _Arg(types, "type_vectors", 2)
        a_radii = _Arg(radii, "radii", 1)
        a_diff = _Arg(diff, "diff", 4, wide=True)
        a_ag = _Arg(agrad, "atom_gradients", 2)
        a_tg = _Arg(tgrad, "type_gradients", 2)
        a_dd = _Arg(diffdiff, "diffdiff", 4, out=True)
        a_add = _Arg(add, "atom_diffdiff", 2, out=True)
        a_tdd = _Arg(tdd, "type_diffdiff", 2, out=True)
        n, T = a_coords.shape[0], a_types.shape[1]
        dim = int(self._p.dim)
        # src/grid_maker.cpp:541-559
        if n != a_types.shape[0]:
            raise ValueError("Type dimension doesn't equal number of coordinates.")
        if T != a_diff.shape[0]:
            raise ValueError("Channels in diff doesn't equal number of types")
        if n != a_ag.shape[0]:
            raise ValueError("Atom gradient dimension doesn't equal number of coordinates")
        if n != a_tg.shape[0]:
            raise ValueError("Type gradient dimension doesn't equal number of coordinates")
        if n != a_add.shape[0]:
            raise ValueError("Atom gradient gradients dimension doesn't equal number of coordinates")
        if n != a_tdd.shape[0]:
            raise ValueError("Type gradient gradients dimension doesn't equal number of coordinates")
        if a_tg.shape[1] != T or a_tdd.shape[1] != T:
            raise ValueError("Type gradient dimension has wrong number of types")
        if a_coords.shape[1] != 3 or a_ag.shape[1] != 3 or a_add.shape[1] != 3:
            raise ValueError("Need x,y,z,r for coord_radius")
        if self._p.radii_type_indexed:
            if T != a_radii.shape[0]:
                raise ValueError("Radii dimension doesn't equal number of types")
        elif n != a_radii.shape[0]:
            raise ValueError("Radii dimension doesn't equal number of coordinates")
        if self._p.binary:
            raise ValueError("Binary densities not supported")
        if tuple(a_diff.shape[1:]) != (dim, dim, dim) or a_dd.shape != a_diff.shape:
            raise ValueError("diff and diffdiff must both be (ntypes, %d, %d, %d)" % (dim, dim, dim))
        code = _lib.mg_backward_gradients(self._p, 1, None, n, None, _capi.f3(c), a_coords.ptr,
                                          a_types.ptr, a_radii.ptr, T, a_diff.ptr, a_ag.ptr,
                                          a_tg.ptr, a_dd.ptr, a_add.ptr, a_tdd.ptr, _stream())
        _capi.check(code, "GridMaker.backward_gradients")
        a_dd.finish()
        a_add.finish()
        a_tdd.finish()

    def _backward_padded(self, centers, coords, types, radii, diff, agrad, tgrad=None):
        """Padded batch (B leading): coords (B,N,3), types (B,N) or (B,N,T), radii (B,N),
        diff (B,T,D,D,D) -> gradients shaped like coords / types.  One launch for the batch.
        ``centers`` is (B,3) or one centre for every example."""
        a_coords = _Arg(coords, "coords", 3)
        tdim = len(tuple(types.shape))
        if tdim not in (2, 3):
            raise ValueError("Unsupported types dimension")
        a_types = _Arg(types, "types", tdim)
        a_radii = _Arg(radii, "radii", 2)
        a_diff = _Arg(diff, "diff", 5, wide=True)
        a_ag = _Arg(agrad, "atom_gradients", 3, out=True, wide=True)
        B, n = a_coords.shape[0], a_coords.shape[1]
        for a in (a_types, a_radii, a_diff, a_ag):
            if a.shape[0] != B:
                raise ValueError("Mismatched batch sizes: %d vs %d" % (a.shape[0], B))
        if a_ag.shape != a_coords.shape or a_coords.shape[2] != 3:
            raise ValueError("Gradient dimension doesn't equal number of coordinates")
        if a_types.shape[1] != n:
            raise ValueError("Type dimension doesn't equal number of coordinates.")
        dim = int(self._p.dim)
        for ax in (2, 3, 4):
            if a_diff.shape[ax] != dim:
                raise ValueError("diff does not have correct dimension %d: %d vs %d"
                                 % (ax - 1, a_diff.shape[ax], dim))
        T = a_diff.shape[1]
        one_center = not hasattr(centers, "shape") or len(tuple(centers.shape)) == 1
        cen = None if one_center else _small_device(centers, 3)
        chost = _capi.f3(_to_float3(centers)) if one_center else _capi.f3(_Z3)
        if cen is not None and cen.shape[0] != B:
            raise ValueError("Mismatched batch sizes: %d vs %d" % (cen.shape[0], B))
        rti = bool(self._p.radii_type_indexed)
        if tdim == 2:
            if rti:
                raise ValueError("Type indexed radii not supported with index types.")
            if a_radii.shape[1] != n:
                raise ValueError("Radii dimension doesn't equal number of coordinates")
            code = _lib.mg_backward_index(self._p, B, None, n, _ptr(cen), chost, a_coords.ptr,
                                          a_types.ptr, a_radii.ptr, T, a_diff.ptr, a_ag.ptr,
                                          _stream())
            _capi.check(code, "GridMaker.backward")
            a_ag.finish()
            return
        if tgrad is None:
            raise TypeError("vector types need a type_gradients argument")
        a_tg = _Arg(tgrad, "type_gradients", 3, out=True, wide=True)
        if a_types.shape[2] != T:
            raise ValueError("Channels in diff doesn't equal number of types")
        if a_tg.shape != a_types.shape:
            raise ValueError("Type gradient dimension has wrong number of types")
        if a_radii.shape[1] != (T if rti else n):
            raise ValueError("Radii dimension doesn't equal number of %s"
                             % ("types" if rti else "coordinates"))
        code = _lib.mg_backward_vector(self._p, B, None, n, _ptr(cen), chost, a_coords.ptr,
                                       a_types.ptr, a_radii.ptr, T, a_diff.ptr, a_ag.ptr,
                                       a_tg.ptr, _stream())
        _capi.check(code, "GridMaker.backward")
        a_ag.finish()
        a_tg.finish()

    @_accepts_grids
    def backward_batch(self, offsets, centers, coords, types, radii, diff, atom_gradients,
                       type_gradients=None, unrotate=None):
        """Ragged batch in one launch; diff is (B,T,D,D,D); gradients are packed like the
        atom arrays.  ``unrotate=(quats, rotation_centers)`` (index types) also applies
        ``Transform.backward(gradients, dotranslate=False)`` per example in the same launch."""
        off, B, largest, total = _offsets_arg(offsets)
        cen = _small_device(centers, 3)
        a_coords = _Arg(coords, "coords", 2)
        tdim = len(tuple(types.shape))
        a_types = _Arg(types, "types", tdim)
        rti = bool(self._p.radii_type_indexed)
        a_radii = _Arg(radii, "radii", 2 if rti else 1)
        a_diff = _Arg(diff, "diff", 5, wide=True)
        a_ag = _Arg(atom_gradients, "atom_gradients", 2, out=True, wide=True)
        if cen.shape[0] != B or a_diff.shape[0] != B:
            raise ValueError("Mismatched batch sizes: %d vs %d" % (a_diff.shape[0], B))
        if a_ag.shape != a_coords.shape or a_coords.shape[1] != 3:
            raise ValueError("Gradient dimension doesn't equal number of coordinates")
        if a_coords.shape[0] < total or a_types.shape[0] < total:
            raise ValueError("atom arrays are shorter than offsets[-1]")
        dim = int(self._p.dim)
        for ax in (2, 3, 4):
            if a_diff.shape[ax] != dim:
                raise ValueError("diff does not have correct dimension %d: %d vs %d"
                                 % (ax - 1, a_diff.shape[ax], dim))
        T = a_diff.shape[1]
        if tdim == 1:
            if rti:
                raise ValueError("Type indexed radii not supported with index types.")
            if unrotate is not None:
                q, rc = _small_device(unrotate[0], 4), _small_device(unrotate[1], 3)
                if q.shape[0] != B or rc.shape[0] != B:
                    raise ValueError("Mismatched batch sizes: the quaternions and rotation "
                                     "centres need %d rows" % B)
                code = _lib.mg_backward_index_unrotated(
                    self._p, B, _ptr(off), largest, _ptr(cen), _capi.f3(_Z3), a_coords.ptr,
                    a_types.ptr, a_radii.ptr, T, a_diff.ptr, _ptr(q), _capi.f4(_IDQ), _ptr(rc),
                    _capi.f3(_Z3), a_ag.ptr, _stream())
            else:
                code = _lib.mg_backward_index(self._p, B, _ptr(off), largest, _ptr(cen),
                                              _capi.f3(_Z3), a_coords.ptr, a_types.ptr,
                                              a_radii.ptr, T, a_diff.ptr, a_ag.ptr, _stream())
            _capi.check(code, "GridMaker.backward_batch")
            a_ag.finish()
            return
        if unrotate is not None:
            raise ValueError("unrotate is for index types")
        if type_gradients is None:
            raise TypeError("vector types need a type_gradients argument")
        a_tg = _Arg(type_gradients, "type_gradients", 2, out=True, wide=True)
        if a_types.shape[1] != T or a_tg.shape != a_types.shape:
            raise ValueError("Type gradient dimension has wrong number of types")
        if rti and a_radii.shape != (B, T):
            raise ValueError("Radii dimension doesn't equal number of types")
        code = _lib.mg_backward_vector(self._p, B, _ptr(off), largest, _ptr(cen), _capi.f3(_Z3),
                                       a_coords.ptr, a_types.ptr, a_radii.ptr, T, a_diff.ptr,
                                       a_ag.ptr, a_tg.ptr, _stream())
        _capi.check(code, "GridMaker.backward_batch")
        a_ag.finish()
        a_tg.finish()


class _Shape(object):
    """Carries only a ``shape`` for the shared argument checks."""

    def __init__(self, shape):
        self.shape = tuple(shape)


# --------------------------------------------------------------------------- #
# GridInterpolater
# --------------------------------------------------------------------------- #
class GridInterpolater(object):
    """Trilinear resampling of a 4-D grid through the inverse of a Transform
    (python/bindings.in.cpp:920-943, include/libmolgrid/grid_interpolater.h)."""

    def __init__(self, in_resolution=0.5, in_dimension=23.5, out_resolution=0.5,
                 out_dimension=23.5):
        self.in_resolution = float(in_resolution)
        self.in_dimension = float(in_dimension)
        self.out_resolution = float(out_resolution)
        self.out_dimension = float(out_dimension)

    @staticmethod
    def _points(dimension, resolution):
        return int(np.round(_f32(dimension) / _f32(resolution)) + 1)

    @property
    def in_dim(self):
        return self._points(self.in_dimension, self.in_resolution)

    @property
    def out_dim(self):
        return self._points(self.out_dimension, self.out_resolution)

    def get_in_resolution(self):
        return self.in_resolution

    def get_out_resolution(self):
        return self.out_resolution

    def get_in_dimension(self):
        return self.in_dimension

    def get_out_dimension(self):
        return self.out_dimension

    def set_in_resolution(self, r):
        self.in_resolution = float(r)

    def set_out_resolution(self, r):
        self.out_resolution = float(r)

    def set_in_dimension(self, d):
        self.in_dimension = float(d)

    def set_out_dimension(self, d):
        self.out_dimension = float(d)

    def _check(self, in_shape, out_shape, same):
        # src/grid_interpolater.cpp:55-76
        if same:
            raise ValueError("Input and output grid can not be the same in GridInterpolator.")
        if in_shape[0] != out_shape[0]:
            raise ValueError("Different channel dimensions for input and output  grids.")
        if tuple(in_shape[1:]) != (self.in_dim,) * 3:
            raise ValueError("Input grid wrong dimension. Should be %d along all axes but is "
                             "%d,%d,%d" % ((self.in_dim,) + tuple(in_shape[1:])))
        if tuple(out_shape[1:]) != (self.out_dim,) * 3:
            raise ValueError("Output grid wrong dimension. Should be %d along all axes but is "
                             "%d,%d,%d" % ((self.out_dim,) + tuple(out_shape[1:])))

    @_accepts_grids
    def forward(self, *args, **kw):
        """forward(in, transform, out)
        forward(in_center, in, transform, out_center, out)
        forward(in, out, random_translation=0, random_rotation=False)"""
        if len(args) == 5:
            in_center, src, transform, out_center, dst = args
        elif len(args) >= 2 and not isinstance(args[1], Transform):
            src, dst = args[:2]
            rt = args[2] if len(args) > 2 else kw.get("random_translation", 0.0)
            rr = args[3] if len(args) > 3 else kw.get("random_rotation", False)
            transform = Transform(_Z3, rt, rr)
            in_center = out_center = transform.get_rotation_center()
        elif len(args) == 3:
            src, transform, dst = args
            in_center = out_center = transform.get_rotation_center()
        else:
            raise TypeError("unsupported GridInterpolater.forward arguments")
        a_in = _Arg(src, "in", 4)
        a_out = _Arg(dst, "out", 4, out=True)
        same = (src is dst) or _same_memory(src, dst)
        self._check(a_in.shape, a_out.shape, same)
        code = _lib.mg_interpolate(
            self.in_resolution, self.in_dimension, self.out_resolution, self.out_dimension, 1,
            a_in.shape[0], None, _capi.f3(_to_float3(in_center)), a_in.ptr, None,
            _capi.f4(transform.get_quaternion().as_tuple()), None,
            _capi.f3(transform.get_rotation_center()), None,
            _capi.f3(transform.get_translation()), None, _capi.f3(_to_float3(out_center)),
            a_out.ptr, _stream())
        _capi.check(code, "GridInterpolater.forward")
        a_out.finish()

    @_accepts_grids
    def forward_batch(self, src, quats, rot_centers, translations, dst, in_centers=None,
                      out_centers=None):
        """One launch for a batch: src (B,K,Din,Din,Din) -> dst (B,K,Dout,Dout,Dout) with one
        transform per example.  Grid centres default to the rotation centres."""
        a_in = _Arg(src, "in", 5)
        a_out = _Arg(dst, "out", 5, out=True)
        B = a_in.shape[0]
        if a_out.shape[0] != B:
            raise ValueError("Mismatched batch sizes: %d vs %d" % (a_out.shape[0], B))
        same = (src is dst) or _same_memory(src, dst)
        self._check(a_in.shape[1:], a_out.shape[1:], same)
        q, c, t = (_small_device(quats, 4), _small_device(rot_centers, 3),
                   _small_device(translations, 3))
        ic = _small_device(in_centers, 3) if in_centers is not None else c
        oc = _small_device(out_centers, 3) if out_centers is not None else c
        for v in (q, c, t, ic, oc):
            if v.shape[0] != B:
                raise ValueError("Mismatched batch sizes: %d vs %d" % (v.shape[0], B))
        code = _lib.mg_interpolate(
            self.in_resolution, self.in_dimension, self.out_resolution, self.out_dimension, B,
            a_in.shape[1], _ptr(ic), _capi.f3(_Z3), a_in.ptr, _ptr(q), _capi.f4(_IDQ), _ptr(c),
            _capi.f3(_Z3), _ptr(t), _capi.f3(_Z3), _ptr(oc), _capi.f3(_Z3), a_out.ptr, _stream())
        _capi.check(code, "GridInterpolater.forward_batch")
        a_out.finish()
