"""numpy front end of the CPU oracle (``liboracle.so``) -- TEST INFRASTRUCTURE ONLY.

Only the test-suite, the smoke check and the benchmark's ``cpu_baseline`` leg may
import this module; the shipped package never does.  Each function forwards to
the C restatement in ``gridding_oracle.c`` (which cites the reference lines it
follows) and returns freshly allocated numpy arrays.
"""
import ctypes
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "liboracle.so")

_f32p = ctypes.POINTER(ctypes.c_float)
_f64p = ctypes.POINTER(ctypes.c_double)
_i64p = ctypes.POINTER(ctypes.c_int64)


class GridMakerParams(ctypes.Structure):
    _fields_ = [
        ("resolution", ctypes.c_float),
        ("dimension", ctypes.c_float),
        ("radius_scale", ctypes.c_float),
        ("gaussian_radius_multiple", ctypes.c_float),
        ("final_radius_multiple", ctypes.c_float),
        ("A", ctypes.c_float),
        ("B", ctypes.c_float),
        ("C", ctypes.c_float),
        ("D", ctypes.c_float),
        ("E", ctypes.c_float),
        ("binary", ctypes.c_int),
        ("radii_type_indexed", ctypes.c_int),
        ("dim", ctypes.c_uint),
    ]


def build(force=False):
    """Compile liboracle.so with the Makefile beside this file."""
    if force or not os.path.exists(_LIB_PATH):
        subprocess.check_call(["make", "-C", _HERE, "-B" if force else "-s", "liboracle.so"])
    return _LIB_PATH


_lib = None


def lib():
    global _lib
    if _lib is None:
        build()
        _lib = ctypes.CDLL(_LIB_PATH)
        _lib.orc_calc_point.restype = ctypes.c_float
        _lib.orc_calc_point.argtypes = [ctypes.POINTER(GridMakerParams)] + [ctypes.c_float] * 7
        _lib.orc_max_threads.restype = ctypes.c_int
    return _lib


def max_threads():
    return int(lib().orc_max_threads())


class OracleError(Exception):
    """Raised where the reference would throw (status code in ``args[0]``)."""


def _f32(a):
    return np.ascontiguousarray(a, dtype=np.float32)


def _p(a):
    return a.ctypes.data_as(_f32p)


def _check(status):
    if status:
        raise OracleError(status)


class GridMaker:
    """Mirror of the reference constructor arguments (grid_maker.h:70-74)."""

    def __init__(self, resolution=0.5, dimension=23.5, binary=False, radius_type_indexed=False,
                 radius_scale=1.0, gaussian_radius_multiple=1.0):
        self.p = GridMakerParams()
        lib().orc_gridmaker_init(ctypes.byref(self.p), ctypes.c_float(resolution),
                                 ctypes.c_float(dimension), int(bool(binary)),
                                 int(bool(radius_type_indexed)), ctypes.c_float(radius_scale),
                                 ctypes.c_float(gaussian_radius_multiple))

    @property
    def dim(self):
        return int(self.p.dim)

    def grid_shape(self, ntypes):
        d = self.dim
        return (int(ntypes), d, d, d)

    def calc_point(self, atom, radius, point):
        return float(lib().orc_calc_point(ctypes.byref(self.p), *[ctypes.c_float(v) for v in atom],
                                          ctypes.c_float(radius),
                                          *[ctypes.c_float(v) for v in point]))

    def bounds_1d(self, origin, coord, densityrad):
        lo, hi = ctypes.c_uint(), ctypes.c_uint()
        lib().orc_bounds_1d(ctypes.byref(self.p), ctypes.c_float(origin), ctypes.c_float(coord),
                            ctypes.c_float(densityrad), ctypes.byref(lo), ctypes.byref(hi))
        return lo.value, hi.value

    # -- single example -----------------------------------------------------
    def forward(self, center, coords, types, radii, ntypes=None):
        """types 1-D -> index types, 2-D -> type vectors."""
        coords, types, radii = _f32(coords), _f32(types), _f32(radii)
        c = _f32(center)
        n = coords.shape[0]
        if types.ndim == 1:
            assert ntypes is not None
            out = np.empty(self.grid_shape(ntypes), np.float32)
            _check(lib().orc_forward_index(ctypes.byref(self.p), _p(c), ctypes.c_int64(n),
                                           _p(coords), _p(types), _p(radii),
                                           ctypes.c_int64(ntypes), _p(out)))
        else:
            ntypes = types.shape[1]
            out = np.empty(self.grid_shape(ntypes), np.float32)
            _check(lib().orc_forward_vector(ctypes.byref(self.p), _p(c), ctypes.c_int64(n),
                                            _p(coords), _p(types), _p(radii),
                                            ctypes.c_int64(ntypes), _p(out)))
        return out

    def backward(self, center, coords, types, radii, diff, f64=False):
        coords, types, radii, diff = _f32(coords), _f32(types), _f32(radii), _f32(diff)
        c = _f32(center)
        n = coords.shape[0]
        ntypes = diff.shape[0]
        dt = np.float64 if f64 else np.float32
        gp = (lambda a: a.ctypes.data_as(_f64p)) if f64 else _p
        agrad = np.empty((n, 3), dt)
        if types.ndim == 1:
            fn = lib().orc_backward_index_f64 if f64 else lib().orc_backward_index
            _check(fn(ctypes.byref(self.p), _p(c), ctypes.c_int64(n), _p(coords), _p(types),
                      _p(radii), ctypes.c_int64(ntypes), _p(diff), gp(agrad)))
            return agrad
        tgrad = np.empty((n, ntypes), dt)
        fn = lib().orc_backward_vector_f64 if f64 else lib().orc_backward_vector
        _check(fn(ctypes.byref(self.p), _p(c), ctypes.c_int64(n), _p(coords), _p(types),
                  _p(radii), ctypes.c_int64(ntypes), _p(diff), gp(agrad), gp(tgrad)))
        return agrad, tgrad

    def backward_relevance(self, center, coords, types, radii, density, diff):
        c = _f32(center)
        coords, types, radii, density, diff = (_f32(coords), _f32(types), _f32(radii),
                                               _f32(density), _f32(diff))
        n = coords.shape[0]
        rel = np.empty(n, np.float32)
        _check(lib().orc_backward_relevance(
            ctypes.byref(self.p), _p(c), ctypes.c_int64(n), _p(coords), _p(types), _p(radii),
            ctypes.c_int64(diff.shape[0]), _p(density), _p(diff), _p(rel)))
        return rel

    def backward_gradients(self, center, coords, types, radii, diff, atom_gradients,
                           type_gradients):
        """-> (diffdiff, atom_diffdiff, type_diffdiff)"""
        c = _f32(center)
        coords, types, radii, diff = _f32(coords), _f32(types), _f32(radii), _f32(diff)
        ag, tg = _f32(atom_gradients), _f32(type_gradients)
        n, ntypes = coords.shape[0], diff.shape[0]
        dd = np.empty(diff.shape, np.float32)
        add = np.empty((n, 3), np.float32)
        tdd = np.empty((n, ntypes), np.float32)
        _check(lib().orc_backward_gradients(
            ctypes.byref(self.p), _p(c), ctypes.c_int64(n), _p(coords), _p(types), _p(radii),
            ctypes.c_int64(ntypes), _p(diff), _p(ag), _p(tg), _p(dd), _p(add), _p(tdd)))
        return dd, add, tdd

    # -- packed batch -------------------------------------------------------
    def forward_batch(self, offsets, centers, coords, types, radii, ntypes, nthreads=1):
        off = np.ascontiguousarray(offsets, dtype=np.int64)
        B = len(off) - 1
        centers, coords, types, radii = _f32(centers), _f32(coords), _f32(types), _f32(radii)
        out = np.empty((B,) + self.grid_shape(ntypes), np.float32)
        fn = lib().orc_forward_index_batch if types.ndim == 1 else lib().orc_forward_vector_batch
        _check(fn(ctypes.byref(self.p), B, off.ctypes.data_as(_i64p), _p(centers), _p(coords),
                  _p(types), _p(radii), ctypes.c_int64(ntypes), _p(out), int(nthreads)))
        return out

    def backward_batch(self, offsets, centers, coords, types, radii, diff, nthreads=1):
        off = np.ascontiguousarray(offsets, dtype=np.int64)
        B = len(off) - 1
        centers, coords, types, radii, diff = (_f32(centers), _f32(coords), _f32(types),
                                               _f32(radii), _f32(diff))
        ntypes = diff.shape[1]
        n = coords.shape[0]
        agrad = np.empty((n, 3), np.float32)
        if types.ndim == 1:
            _check(lib().orc_backward_index_batch(
                ctypes.byref(self.p), B, off.ctypes.data_as(_i64p), _p(centers), _p(coords),
                _p(types), _p(radii), ctypes.c_int64(ntypes), _p(diff), _p(agrad), int(nthreads)))
            return agrad
        tgrad = np.empty((n, ntypes), np.float32)
        _check(lib().orc_backward_vector_batch(
            ctypes.byref(self.p), B, off.ctypes.data_as(_i64p), _p(centers), _p(coords),
            _p(types), _p(radii), ctypes.c_int64(ntypes), _p(diff), _p(agrad), _p(tgrad),
            int(nthreads)))
        return agrad, tgrad


def quat_mul(p, q):
    p, q = _f32(p), _f32(q)
    out = np.empty(4, np.float32)
    lib().orc_quat_mul(_p(p), _p(q), _p(out))
    return out


def quat_inverse(q):
    q = _f32(q)
    out = np.empty(4, np.float32)
    lib().orc_quat_inverse(_p(q), _p(out))
    return out


def quat_rotate(q, pt):
    q = _f32(q)
    out = np.empty(3, np.float32)
    lib().orc_quat_rotate(_p(q), ctypes.c_float(pt[0]), ctypes.c_float(pt[1]),
                          ctypes.c_float(pt[2]), _p(out))
    return out


def transform_forward(q, center, translate, coords, dotranslate=True):
    q, center, translate, coords = _f32(q), _f32(center), _f32(translate), _f32(coords)
    out = np.empty_like(coords)
    lib().orc_transform_forward(_p(q), _p(center), _p(translate), int(bool(dotranslate)),
                                ctypes.c_int64(coords.shape[0]), _p(coords), _p(out))
    return out


def transform_backward(q, center, translate, coords, dotranslate=True):
    q, center, translate, coords = _f32(q), _f32(center), _f32(translate), _f32(coords)
    out = np.empty_like(coords)
    lib().orc_transform_backward(_p(q), _p(center), _p(translate), int(bool(dotranslate)),
                                 ctypes.c_int64(coords.shape[0]), _p(coords), _p(out))
    return out


def transform_forward_batch(offsets, quats, centers, translations, coords, dotranslate=True,
                            nthreads=1):
    off = np.ascontiguousarray(offsets, dtype=np.int64)
    quats, centers, translations, coords = (_f32(quats), _f32(centers), _f32(translations),
                                            _f32(coords))
    out = np.empty_like(coords)
    lib().orc_transform_forward_batch(len(off) - 1, off.ctypes.data_as(_i64p), _p(quats),
                                      _p(centers), _p(translations), int(bool(dotranslate)),
                                      _p(coords), _p(out), int(nthreads))
    return out


def transform_backward_batch(offsets, quats, centers, translations, coords, dotranslate=True,
                             nthreads=1):
    off = np.ascontiguousarray(offsets, dtype=np.int64)
    quats, centers, translations, coords = (_f32(quats), _f32(centers), _f32(translations),
                                            _f32(coords))
    out = np.empty_like(coords)
    lib().orc_transform_backward_batch(len(off) - 1, off.ctypes.data_as(_i64p), _p(quats),
                                       _p(centers), _p(translations), int(bool(dotranslate)),
                                       _p(coords), _p(out), int(nthreads))
    return out


def _npoints(dimension, resolution):
    return int(np.float32(np.round(np.float32(dimension) / np.float32(resolution))) + 1)


def interpolate(in_res, in_dimension, out_res, out_dimension, in_center, grid, q, rot_center,
                translate, out_center):
    grid = _f32(grid)
    K = grid.shape[0]
    od = _npoints(out_dimension, out_res)
    out = np.empty((K, od, od, od), np.float32)
    a = [_f32(v) for v in (in_center, q, rot_center, translate, out_center)]
    _check(lib().orc_interpolate(ctypes.c_float(in_res), ctypes.c_float(in_dimension),
                                 ctypes.c_float(out_res), ctypes.c_float(out_dimension),
                                 _p(a[0]), _p(grid), ctypes.c_int64(K), _p(a[1]), _p(a[2]),
                                 _p(a[3]), _p(a[4]), _p(out)))
    return out


def interpolate_batch(in_res, in_dimension, out_res, out_dimension, in_centers, grids, quats,
                      rot_centers, translations, out_centers, nthreads=1):
    grids = _f32(grids)
    B, K = grids.shape[:2]
    od = _npoints(out_dimension, out_res)
    out = np.empty((B, K, od, od, od), np.float32)
    a = [_f32(v) for v in (in_centers, quats, rot_centers, translations, out_centers)]
    _check(lib().orc_interpolate_batch(
        ctypes.c_float(in_res), ctypes.c_float(in_dimension), ctypes.c_float(out_res),
        ctypes.c_float(out_dimension), B, ctypes.c_int64(K), _p(a[0]), _p(grids), _p(a[1]),
        _p(a[2]), _p(a[3]), _p(a[4]), _p(out), int(nthreads)))
    return out
