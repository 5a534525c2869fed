"""ctypes binding of include/dpnp_amd.h (libdpnp_amd.so).

The library is the product's only compute path: if it is missing, importing this
module raises; there is no CPU or PyTorch fallback.
"""
import ctypes
import os

# Where device memory and the stream come from: the library's own pool and stream (dpx_mem_* and
# dpx_stream_*, "native") unless DPNP_AMD_MEMORY=torch asks for PyTorch's caching allocator and current
# stream (for processes that mix this package's calls with torch work on the same data).
# PyTorch ships its own HIP runtime (libamdhip64.so.7).  It must be in the process before
# libdpnp_amd.so is loaded so that both bind to the SAME runtime instance: device memory
# allocated by torch is then valid in this library's launches, and the stream handles match.
# Loading in the other order leaves two runtimes in the process and the second one finds no device.
# A process that uses torch for something else beside this package (on the native provider) imports
# torch first for the same reason.
MEMORY = os.environ.get("DPNP_AMD_MEMORY", "").lower() or "native"
if MEMORY not in ("torch", "native"):
    raise ImportError("DPNP_AMD_MEMORY must be 'torch' or 'native', not %r" % MEMORY)
torch = None
if MEMORY == "torch":
    import torch  # noqa: F401,E402

MAX_ND = 12
NOALLOC_SCRATCH_BYTES = 2 << 20  # DPX_NOALLOC_SCRATCH_BYTES

(BOOL, INT8, UINT8, INT16, UINT16, INT32, UINT32, INT64, UINT64, HALF, FLOAT,
 DOUBLE, CFLOAT, CDOUBLE) = range(14)

C_CONTIGUOUS, F_CONTIGUOUS, WRITABLE = 1, 2, 4

(OK, ERR_BAD_DTYPE, ERR_SHAPE_MISMATCH, ERR_RANK_MISMATCH, ERR_NOT_WRITABLE,
 ERR_OVERLAP, ERR_NOT_AMPLE, ERR_NOT_IMPLEMENTED, ERR_HIP, ERR_BAD_ARGUMENT) = range(10)

UNARY_OPS = [
    "abs", "negative", "positive", "square", "sqrt", "exp", "log", "erf", "sin",
    "cos", "tan", "tanh", "exp2", "expm1", "log2", "log10", "log1p", "rsqrt",
    "cbrt", "reciprocal", "floor", "ceil", "trunc", "sign", "isnan", "isinf",
    "isfinite", "logical_not", "bitwise_invert", "signbit", "asin", "acos", "atan", "sinh",
    "cosh", "asinh", "acosh", "atanh", "round", "conj", "real", "imag", "proj", "angle",
    "fabs", "degrees", "radians", "sinc", "spacing", "bitwise_count", "erfc", "erfcx", "erfinv",
    "erfcinv", "i0",
]
BINARY_OPS = [
    "add", "subtract", "multiply", "divide", "bitwise_and", "bitwise_or",
    "bitwise_xor", "equal", "not_equal", "less", "less_equal", "greater",
    "greater_equal", "maximum", "minimum", "logical_and", "logical_or",
    "logical_xor", "pow", "floor_divide", "remainder", "atan2", "hypot",
    "copysign", "bitwise_left_shift", "bitwise_right_shift", "logaddexp", "nextafter",
    "fmax", "fmin", "fmod", "logaddexp2", "heaviside", "gcd", "lcm",
]
REDUCE_OPS = ["sum", "prod", "max", "min", "sumsqdev", "logsumexp", "hypot",
              "nansum", "nanprod", "nanmax", "nanmin", "nancount", "nansumsqdev",
              "any", "all", "count_nonzero", "nanmean", "nanvar", "sqdev_onepass"]
SEARCH_OPS = ["argmax", "argmin", "nanargmax", "nanargmin", "nanargmax_marked", "nanargmin_marked"]
UNARY_ID = {n: i for i, n in enumerate(UNARY_OPS)}
BINARY_ID = {n: i for i, n in enumerate(BINARY_OPS)}
REDUCE_ID = {n: i for i, n in enumerate(REDUCE_OPS)}
SEARCH_ID = {n: i for i, n in enumerate(SEARCH_OPS)}

PATH_NAMES = {
    0: "noop", 1: "ew_contig", 2: "ew_rows", 3: "ew_rows2", 4: "ew_tile",
    10: "red_rows", 11: "red_rows_split", 12: "red_cols", 13: "red_cols_split",
    14: "red_generic", 15: "red_small", 16: "red_flat", 17: "red_short_rows",
}


class ArrayView(ctypes.Structure):
    _fields_ = [
        ("data", ctypes.c_void_p),
        ("nd", ctypes.c_int32),
        ("dtype", ctypes.c_int32),
        ("flags", ctypes.c_int32),
        ("reserved", ctypes.c_int32),
        ("shape", ctypes.c_int64 * MAX_ND),
        ("strides", ctypes.c_int64 * MAX_ND),
    ]


class Plan(ctypes.Structure):
    _fields_ = [
        ("path", ctypes.c_int32),
        ("nd", ctypes.c_int32),
        ("red_nd", ctypes.c_int32),
        ("vec", ctypes.c_int32),
        ("shape", ctypes.c_int64 * MAX_ND),
        ("strides", (ctypes.c_int64 * MAX_ND) * 4),
        ("offsets", ctypes.c_int64 * 4),
        ("grid", ctypes.c_int64 * 3),
        ("block", ctypes.c_int32),
        ("splits", ctypes.c_int32),
        ("scratch_bytes", ctypes.c_int64),
    ]


_VP = ctypes.POINTER(ArrayView)
_PP = ctypes.POINTER(Plan)
_i = ctypes.c_int
_i64 = ctypes.c_int64
_d = ctypes.c_double
_vp = ctypes.c_void_p

# every symbol include/dpnp_amd.h declares: name -> (restype, argtypes)
SIGNATURES = {
    "dpx_abi_version": (_i, []),
    "dpx_last_error": (ctypes.c_char_p, []),
    "dpx_dtype_itemsize": (_i, [_i]),
    "dpx_release_scratch": (_i, []),
    "dpx_unary_result_type": (_i, [_i, _i]),
    "dpx_binary_result_type": (_i, [_i, _i, _i]),
    "dpx_binary_inplace_supported": (_i, [_i, _i, _i]),
    "dpx_binary_fused_cast_result_type": (_i, [_i, _i, _i]),
    "dpx_reduce_dtype_supported": (_i, [_i, _i, _i]),
    "dpx_search_dtype_supported": (_i, [_i, _i, _i]),
    "dpx_array_overlap": (_i, [_VP, _VP]),
    "dpx_same_logical": (_i, [_VP, _VP]),
    "dpx_unary": (_i, [_i, _VP, _VP, _vp]),
    "dpx_binary": (_i, [_i, _VP, _VP, _VP, _vp]),
    "dpx_binary_inplace": (_i, [_i, _VP, _VP, _vp]),
    "dpx_where": (_i, [_VP, _VP, _VP, _VP, _vp]),
    "dpx_divide_by_scalar": (_i, [_VP, _d, _VP, _vp]),
    "dpx_nan_to_num": (_i, [_VP, _d, _d, _d, _VP, _vp]),
    "dpx_isclose": (_i, [_VP, _VP, _d, _d, _i, _VP, _vp]),
    "dpx_clip": (_i, [_VP, _VP, _VP, _VP, _vp]),
    "dpx_ldexp_result_type": (_i, [_i, _i]),
    "dpx_ldexp": (_i, [_VP, _VP, _VP, _vp]),
    "dpx_frexp": (_i, [_VP, _VP, _VP, _vp]),
    "dpx_copy_cast": (_i, [_VP, _VP, _vp]),
    "dpx_copy_from_host": (_i, [_vp, _vp, ctypes.c_size_t, _vp]),
    "dpx_copy_to_host": (_i, [_vp, _vp, ctypes.c_size_t, _vp]),
    "dpx_device_count": (_i, [ctypes.POINTER(_i)]),
    "dpx_device_name": (_i, [_i, ctypes.c_char_p, ctypes.c_size_t]),
    "dpx_stream_create": (_i, [ctypes.POINTER(_vp)]),
    "dpx_stream_synchronize": (_i, [_vp]),
    "dpx_stream_destroy": (_i, [_vp]),
    "dpx_mem_alloc": (_i, [ctypes.POINTER(_vp), ctypes.c_size_t, _vp]),
    "dpx_mem_free": (_i, [_vp, _vp]),
    "dpx_mem_release_cached": (_i, []),
    "dpx_mem_stats": (_i, [ctypes.POINTER(ctypes.c_size_t), ctypes.POINTER(ctypes.c_size_t)]),
    "dpx_fill": (_i, [_VP, _d, _d, _i64, _i, _vp]),
    "dpx_unary_plan": (_i, [_i, _VP, _VP, _PP]),
    "dpx_binary_plan": (_i, [_i, _VP, _VP, _VP, _PP]),
    "dpx_where_plan": (_i, [_VP, _VP, _VP, _VP, _PP]),
    "dpx_where_compare": (_i, [_i, _VP, _VP, _VP, _VP, _VP, _vp]),
    "dpx_black_scholes": (_i, [_vp, _vp, _vp, _d, _d, _vp, _vp, _i64, _i, _vp]),
    "dpx_reduce": (_i, [_i, _VP, _i, _VP, _VP, _vp]),
    "dpx_reduce_noalloc": (_i, [_i, _VP, _i, _VP, _VP, _vp]),
    "dpx_nan_variance": (_i, [_VP, _i, _VP, _d, _VP, _vp]),
    "dpx_argreduce": (_i, [_i, _VP, _i, _VP, _vp]),
    "dpx_reduce_plan": (_i, [_i, _VP, _i, _VP, _PP]),
    "dpx_argreduce_plan": (_i, [_i, _VP, _i, _VP, _PP]),
    "dpx_collapse": (_i, [_i, _i, ctypes.POINTER(_i64), ctypes.POINTER(_i64),
                          ctypes.POINTER(_i64), _i]),
}

LIB_PATH = os.path.join(os.path.dirname(os.path.abspath(__file__)), "libdpnp_amd.so")


def _load():
    if not os.path.exists(LIB_PATH):
        raise ImportError(
            f"{LIB_PATH} is not built. Run `python -c 'import __graft_entry__ as g; "
            "g.build()'` or `make -C dpnp_amd/csrc` (needs hipcc); there is no fallback path."
        )
    lib = ctypes.CDLL(LIB_PATH)
    for name, (res, args) in SIGNATURES.items():
        fn = getattr(lib, name)  # AttributeError if the library lacks a declared symbol
        fn.restype = res
        fn.argtypes = args
    return lib


lib = _load()


try:
    from . import _dpx_ext as ext  # noqa: E402  (the pybind11 binding; links the library loaded above)
except ImportError as e:  # pragma: no cover
    raise ImportError(
        "dpnp_amd/_dpx_ext extension module is not built (or was built for another Python): run "
        "`make -C dpnp_amd/csrc`; there is no fallback path.  " + str(e)) from e


class DpxError(Exception):
    """Base for errors reported by the library."""


_STATUS_EXC = {
    ERR_BAD_DTYPE: ValueError,
    ERR_SHAPE_MISMATCH: ValueError,
    ERR_RANK_MISMATCH: ValueError,
    ERR_NOT_WRITABLE: ValueError,
    ERR_OVERLAP: ValueError,
    ERR_NOT_AMPLE: ValueError,
    ERR_NOT_IMPLEMENTED: RuntimeError,
    ERR_HIP: RuntimeError,
    ERR_BAD_ARGUMENT: ValueError,
}


def check(status):
    """Raise the exception class the reference raises for this kind of failure."""
    if status == OK:
        return
    msg = lib.dpx_last_error().decode("utf-8", "replace")
    raise _STATUS_EXC.get(status, RuntimeError)(msg)


def make_view(ptr, shape, strides, dtype_id, flags):
    v = ArrayView()
    v.data = ptr
    v.nd = len(shape)
    v.dtype = dtype_id
    v.flags = flags
    for k, (s, st) in enumerate(zip(shape, strides)):
        v.shape[k] = s
        v.strides[k] = st
    return v
