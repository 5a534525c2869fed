"""Drop-in for the reference's `_tensor_elementwise_impl` extension module
(libtensor/source/elementwise_functions/elementwise_common.cpp:118-188): for every
op `X` it exposes `_X(src[, src2], dst, sycl_queue, depends)`, `_X_result_type(dt[, dt2])`
and, for binary ops, `_X_inplace(lhs, rhs, sycl_queue, depends)`, all backed by the C ABI.
"""
from .. import _lib
from ._dtypes import dtype_from_id, dtype_id
from ._tensor_impl import _events, _stream

lib = _lib.lib
ext = _lib.ext


def _make_unary(name, op_id):
    fn = ext.make_unary(op_id, "_" + name)  # _X(src, dst, sycl_queue=None, depends=()) -> (event, event)

    def result_type(dt):
        return dtype_from_id(lib.dpx_unary_result_type(op_id, dtype_id(dt)))

    result_type.__name__ = f"_{name}_result_type"
    return fn, result_type


def _make_binary(name, op_id):
    fn = ext.make_binary(op_id, "_" + name)  # _X(src1, src2, dst, sycl_queue=None, depends=())
    inplace = ext.make_binary_inplace(op_id, f"_{name}_inplace")  # _X_inplace(lhs, rhs, sycl_queue=None, depends=())

    def result_type(dt1, dt2):
        return dtype_from_id(lib.dpx_binary_result_type(op_id, dtype_id(dt1), dtype_id(dt2)))

    result_type.__name__ = f"_{name}_result_type"
    return fn, result_type, inplace


for _n, _i in _lib.UNARY_ID.items():
    _f, _r = _make_unary(_n, _i)
    globals()["_" + _n] = _f
    globals()[f"_{_n}_result_type"] = _r
for _n, _i in _lib.BINARY_ID.items():
    _f, _r, _ip = _make_binary(_n, _i)
    globals()["_" + _n] = _f
    globals()[f"_{_n}_result_type"] = _r
    globals()[f"_{_n}_inplace"] = _ip


_divide_by_scalar = ext._divide_by_scalar  # (src, scalar, dst, sycl_queue=None, depends=())


def _fused_cast_result_type(name, dt1, dt2):
    """Result dtype of binary function `name` for two different operand dtypes when the library
    converts one operand while reading it (no counterpart in the reference), else None."""
    op = _lib.BINARY_ID.get(name)
    if op is None:
        return None
    r = lib.dpx_binary_fused_cast_result_type(op, dtype_id(dt1), dtype_id(dt2))
    return None if r < 0 else dtype_from_id(r)


def _nan_to_num(src, nan, posinf, neginf, dst, sycl_queue=None, depends=()):
    """ufi._nan_to_num of the reference's ufunc extension
    (dpnp/backend/extensions/ufunc/elementwise_functions/nan_to_num.cpp): scalar replacements."""
    vs, vd = src._as_view(), dst._as_view()
    _lib.check(lib.dpx_nan_to_num(vs, float(nan), float(posinf), float(neginf), vd, _stream(sycl_queue)))
    return _events(sycl_queue)


def _isclose_scalar(a, b, rtol, atol, equal_nan, dst, sycl_queue=None, depends=()):
    """ufi._isclose_scalar (dpnp/backend/extensions/ufunc/elementwise_functions/isclose.cpp)."""
    va, vb, vd = a._as_view(), b._as_view(), dst._as_view()
    _lib.check(lib.dpx_isclose(va, vb, float(rtol), float(atol), int(bool(equal_nan)), vd, _stream(sycl_queue)))
    return _events(sycl_queue)


def _ldexp_result_type(dt1, dt2):
    """ufi._ldexp_result_type (dpnp/backend/extensions/ufunc/elementwise_functions/ldexp.cpp:62-93)."""
    r = lib.dpx_ldexp_result_type(dtype_id(dt1), dtype_id(dt2))
    return None if r < 0 else dtype_from_id(r)


def _ldexp(x1, x2, dst, sycl_queue=None, depends=()):
    """ufi._ldexp: dst = x1 * 2**x2, operands already broadcast to dst's shape."""
    _lib.check(lib.dpx_ldexp(x1._as_view(), x2._as_view(), dst._as_view(), _stream(sycl_queue)))
    return _events(sycl_queue)


def _frexp_result_type(dt):
    """ufi._frexp_result_type (frexp.cpp:70-86): (mantissa dtype, exponent dtype) or None."""
    import numpy as np

    dt = np.dtype(dt)
    return (dt, np.dtype("i4")) if dt.kind == "f" else None


def _frexp(x, mantissa, exponent, sycl_queue=None, depends=()):
    """ufi._frexp: x = mantissa * 2**exponent."""
    _lib.check(lib.dpx_frexp(x._as_view(), mantissa._as_view(), exponent._as_view(), _stream(sycl_queue)))
    return _events(sycl_queue)


def _black_scholes(price, strike, t, rate, vol, call, put, sycl_queue=None, depends=()):
    """Fused Black-Scholes pricing over 1-D contiguous arrays (no counterpart in the reference)."""
    arrs = (price, strike, t, call, put)
    n = price.size
    dt = price.dtype
    for a in arrs:
        if a.ndim != 1 or a.size != n or a.dtype != dt or not a.flags.c_contiguous:
            raise ValueError("black_scholes expects five 1-D contiguous arrays of one size and dtype")
    if not (call.flags.writable and put.flags.writable):
        raise ValueError("output array is read-only.")
    _lib.check(lib.dpx_black_scholes(price._pointer, strike._pointer, t._pointer, float(rate), float(vol),
                                     call._pointer, put._pointer, n, dtype_id(dt), _stream(sycl_queue)))
    return _events(sycl_queue)
