"""ctypes binding of the C ABI declared in ``include/molgrid_hip.h``.

The shared library must already be built (``python libmolgrid_amd/build.py``);
importing this module fails loudly when it is missing -- there is no fallback.
"""
import ctypes
import os

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "libmolgrid_hip.so")

MG_OK = 0
MG_ERR_INVALID_ARGUMENT = -1
MG_ERR_OUT_OF_RANGE = -2
MG_ERR_UNSUPPORTED = -3
MG_ERR_NULL_POINTER = -4
MG_STATIC_SCRATCH_BYTES = 16 << 20

EXPORTED_SYMBOLS = (
    "mg_version", "mg_error_string", "mg_trace_ranges", "mg_gridmaker_init", "mg_transform_forward",
    "mg_transform_backward", "mg_forward_index", "mg_forward_index_ws",
    "mg_forward_index_workspace_size", "mg_forward_index_static", "mg_forward_index_paged",
    "mg_forward_index_core_skip",
    "mg_forward_index_sort", "mg_forward_index_splat", "mg_forward_vector_ws",
    "mg_forward_vector_workspace_size", "mg_forward_vector", "mg_backward_index",
    "mg_backward_index_unrotated",
    "mg_backward_vector", "mg_backward_relevance", "mg_backward_gradients", "mg_interpolate", "mg_interpolate_force_gather",
    "mg_narrow", "mg_widen",
)


class mg_gridmaker(ctypes.Structure):
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
        ("binary", ctypes.c_int32),
        ("radii_type_indexed", ctypes.c_int32),
        ("dim", ctypes.c_uint32),
    ]


_vp = ctypes.c_void_p
_f3 = ctypes.c_float * 3
_f4 = ctypes.c_float * 4
_i = ctypes.c_int
_f = ctypes.c_float


def _load():
    if not os.path.exists(LIB_PATH):
        raise ImportError(
            "%s is missing: build it with `python libmolgrid_amd/build.py` "
            "(the gridding kernels have no CPU fallback)" % LIB_PATH)
    return declare(ctypes.CDLL(LIB_PATH))


def declare(lib):
    """Argument and result types of every entry point of include/molgrid_hip.h on a loaded library."""
    gm = ctypes.POINTER(mg_gridmaker)
    lib.mg_version.restype = _i
    lib.mg_error_string.restype = ctypes.c_char_p
    lib.mg_error_string.argtypes = [_i]
    lib.mg_gridmaker_init.argtypes = [gm, _f, _f, _i, _i, _f, _f]
    tr = [_i, _vp, _i, _vp, _f4, _vp, _f3, _vp, _f3, _i, _vp, _vp, _vp]
    lib.mg_transform_forward.argtypes = tr
    lib.mg_transform_backward.argtypes = tr
    fwd = [gm, _i, _vp, _i, _vp, _f3, _vp, _vp, _vp, _i, _vp, _vp]
    lib.mg_forward_index.argtypes = fwd
    lib.mg_forward_index_static.argtypes = fwd
    lib.mg_forward_index_ws.argtypes = fwd[:-1] + [_vp, ctypes.c_size_t, _vp]
    lib.mg_forward_index_sort.argtypes = fwd[:-2] + [_vp, ctypes.c_size_t, _vp]
    lib.mg_forward_index_splat.argtypes = [gm, _i, _i, _i, _vp, _vp, ctypes.c_size_t, _vp]
    lib.mg_forward_index_workspace_size.argtypes = [gm, _i, _i, _i]
    lib.mg_forward_index_workspace_size.restype = ctypes.c_size_t
    lib.mg_forward_vector.argtypes = fwd
    lib.mg_forward_vector_ws.argtypes = fwd[:-1] + [_vp, ctypes.c_size_t, _vp]
    lib.mg_forward_vector_workspace_size.argtypes = [gm, _i, _i, _i]
    lib.mg_forward_vector_workspace_size.restype = ctypes.c_size_t
    lib.mg_backward_index.argtypes = [gm, _i, _vp, _i, _vp, _f3, _vp, _vp, _vp, _i, _vp, _vp, _vp]
    lib.mg_backward_index_unrotated.argtypes = [gm, _i, _vp, _i, _vp, _f3, _vp, _vp, _vp, _i, _vp,
                                                _vp, _f4, _vp, _f3, _vp, _vp]
    lib.mg_backward_vector.argtypes = [gm, _i, _vp, _i, _vp, _f3, _vp, _vp, _vp, _i, _vp, _vp,
                                       _vp, _vp]
    lib.mg_backward_relevance.argtypes = [gm, _i, _vp, _i, _vp, _f3, _vp, _vp, _vp, _i, _vp, _vp,
                                          _vp, _vp]
    lib.mg_backward_gradients.argtypes = [gm, _i, _vp, _i, _vp, _f3, _vp, _vp, _vp, _i, _vp, _vp,
                                          _vp, _vp, _vp, _vp, _vp]
    lib.mg_interpolate.argtypes = [_f, _f, _f, _f, _i, _i, _vp, _f3, _vp, _vp, _f4, _vp, _f3,
                                   _vp, _f3, _vp, _f3, _vp, _vp]
    lib.mg_narrow.argtypes = [_vp, _vp, ctypes.c_size_t, _vp]
    lib.mg_widen.argtypes = [_vp, _vp, ctypes.c_size_t, _vp]
    lib.mg_interpolate_force_gather.argtypes = [_i]
    lib.mg_forward_index_paged.argtypes = [_i]
    lib.mg_forward_index_core_skip.argtypes = [_i]
    lib.mg_trace_ranges.argtypes = [_i]
    for name in EXPORTED_SYMBOLS:
        fn = getattr(lib, name)
        if name not in ("mg_error_string", "mg_forward_index_workspace_size",
                        "mg_forward_vector_workspace_size"):
            fn.restype = _i
    return lib


lib = _load()


def error_string(code):
    return lib.mg_error_string(int(code)).decode()


def check(code, what):
    """Map a return code to the exception type the reference throws."""
    if code == MG_OK:
        return
    msg = "%s: %s" % (what, error_string(code))
    if code == MG_ERR_OUT_OF_RANGE:
        raise IndexError(msg)       # std::out_of_range
    if code in (MG_ERR_INVALID_ARGUMENT, MG_ERR_NULL_POINTER, MG_ERR_UNSUPPORTED):
        raise ValueError(msg)       # std::invalid_argument
    raise RuntimeError(msg)         # hipError_t, like LMG_CUDA_CHECK's runtime_error


def f3(v):
    return _f3(float(v[0]), float(v[1]), float(v[2]))


def f4(v):
    return _f4(float(v[0]), float(v[1]), float(v[2]), float(v[3]))
