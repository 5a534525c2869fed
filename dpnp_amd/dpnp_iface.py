"""NumPy-flavoured functions over dpnp_array: the dpnp-level wrappers on the hot path.

Keyword handling follows DPNPUnaryFunc / DPNPBinaryFunc
(dpnp/dpnp_algo/dpnp_elementwise_common.py:167-235,647-739), dpnp_wrap_reduction_call
(dpnp/dpnp_utils/dpnp_utils_reduction.py:35-53) and the public functions in
dpnp/dpnp_iface_{mathematical,trigonometric,statistics,searching,bitwise,logic}.py:
`where=`, `subok=`, `initial=` other than their defaults raise NotImplementedError, `dtype=`
casts the inputs and excludes `out=`, `out is x1` runs the in-place kernel, a reduction's
`out` of another dtype receives an unsafe cast of the result.
"""
import builtins as _builtins

import numpy as np

from . import tensor as dpt
from .dpnp_array import dpnp_array
from .tensor import _elementwise_funcs as ef
from .tensor import _tensor_elementwise_impl as tei
from .tensor import _tensor_impl as ti
from .tensor._type_utils import _default_accumulation_dtype
from .tensor._usmarray import usm_ndarray
from . import _lib

_ext = _lib.ext

# dtypes and constants under their NumPy names
bool = bool_ = dpt.bool  # noqa: A001
int8, uint8, int16, uint16 = dpt.int8, dpt.uint8, dpt.int16, dpt.uint16
int32, uint32, int64, uint64 = dpt.int32, dpt.uint32, dpt.int64, dpt.uint64
float16, float32, float64 = dpt.float16, dpt.float32, dpt.float64
complex64, complex128 = dpt.complex64, dpt.complex128
nan, inf, pi, e, newaxis = np.nan, np.inf, np.pi, np.e, None


def is_supported_array_type(a):
    return isinstance(a, (dpnp_array, usm_ndarray))


def isscalar(x):
    return np.isscalar(x)


def get_usm_ndarray(a):
    if isinstance(a, dpnp_array):
        return a.get_array()
    if isinstance(a, usm_ndarray):
        return a
    raise TypeError(f"An array must be any of supported type, but got {type(a)}")


def get_usm_ndarray_or_scalar(a):
    return a if np.isscalar(a) else get_usm_ndarray(a)


def check_supported_arrays_type(*arrays, scalar_type=False, all_scalars=False):
    any_is_array = False
    for a in arrays:
        if is_supported_array_type(a):
            any_is_array = True
            continue
        if scalar_type and np.isscalar(a):
            continue
        raise TypeError(f"An array must be any of supported type, but got {type(a)}")
    if len(arrays) > 1 and not (all_scalars or any_is_array):
        raise TypeError("At least one input must be of supported array type, but got all scalars.")
    return True


def check_limitations(**kwargs):
    """Raise NotImplementedError for NumPy keywords that only work at their default."""
    defaults = {"where": True, "initial": None, "subok": True, "order": None}
    for k, v in kwargs.items():
        d = defaults.get(k)
        if not (v is d or (k == "order" and v in ("C", "K", None))):
            raise NotImplementedError(f"Parameter `{k}` is supported only with default value `{d}`, "
                                      f"but got {v}.")


def _check_creation_subok(subok):
    """Array creation functions take `subok` only at its default (dpnp/dpnp_iface.py:196-236)."""
    if subok is not False:
        raise NotImplementedError(f"Keyword argument `subok` is supported only with default value ``False``, "
                                  f"but got {subok}.")


def get_result_array(a, out=None, casting="safe"):
    """`out` filled with `a` (cast by `casting`), or `a` wrapped when there is no `out`."""
    if out is None:
        return dpnp_array._create_from_usm_ndarray(a) if isinstance(a, usm_ndarray) else a
    out_w = dpnp_array._create_from_usm_ndarray(out) if isinstance(out, usm_ndarray) else out
    a_usm, out_usm = get_usm_ndarray(a), get_usm_ndarray(out_w)
    if a_usm is out_usm or ti._same_logical_tensors(a_usm, out_usm):
        return out_w
    if out_usm.shape != a_usm.shape:
        raise ValueError(f"Output array of shape {a_usm.shape} is needed, got {out_usm.shape}.")
    if not np.can_cast(a_usm.dtype, out_usm.dtype, casting=casting):
        raise TypeError(f"Cannot cast from {a_usm.dtype} to {out_usm.dtype} according to the rule {casting}.")
    if a_usm.size:
        ti._copy_usm_ndarray_into_usm_ndarray(src=a_usm, dst=out_usm)
    return out_w


# -- array creation / transfer ------------------------------------------------------------------------
def _wrap(u):
    return dpnp_array._create_from_usm_ndarray(u)


def array(a, dtype=None, *, copy=True, order="K", subok=False, ndmin=0, like=None, device=None,
          usm_type=None, sycl_queue=None):
    _check_creation_subok(subok)
    src = a.get_array() if isinstance(a, dpnp_array) else a
    r = dpt.asarray(src, dtype=dtype, copy=True if copy else None, order=order)
    if ndmin > r.ndim:
        r = dpt.reshape(r, (1,) * (ndmin - r.ndim) + r.shape)
    return _wrap(r)


def asarray(a, dtype=None, order=None, *, device=None, usm_type=None, sycl_queue=None, copy=None, like=None):
    src = a.get_array() if isinstance(a, dpnp_array) else a
    return _wrap(dpt.asarray(src, dtype=dtype, copy=copy, order=order or "K"))


def asanyarray(a, dtype=None, order=None, *, like=None, device=None, usm_type=None, sycl_queue=None):
    # dpnp/dpnp_iface_arraycreation.py:422-520
    check_limitations(like=like)
    return asarray(a, dtype=dtype, order=order)


def ascontiguousarray(a, dtype=None, *, like=None, device=None, usm_type=None, sycl_queue=None):
    # dpnp/dpnp_iface_arraycreation.py:648-763: C order, at least one dimension
    check_limitations(like=like)
    r = asarray(a, dtype=dtype, order="C")
    return reshape(r, (1,)) if r.ndim == 0 else r


def asfortranarray(a, dtype=None, *, like=None, device=None, usm_type=None, sycl_queue=None):
    # dpnp/dpnp_iface_arraycreation.py:766-880: Fortran order, at least one dimension
    check_limitations(like=like)
    r = asarray(a, dtype=dtype, order="F")
    return reshape(r, (1,)) if r.ndim == 0 else r


def copy(a, order="K", subok=False, device=None, usm_type=None, sycl_queue=None):
    # dpnp/dpnp_iface_arraycreation.py:977-1070: always a new array
    _check_creation_subok(subok)
    if isinstance(a, (dpnp_array, usm_ndarray)):
        return _wrap(dpt.copy(get_usm_ndarray(a), order=order or "K"))
    return array(a, order=order, copy=True)


def asnumpy(a, order="C"):
    if isinstance(a, (dpnp_array, usm_ndarray)):
        return np.asarray(dpt.asnumpy(get_usm_ndarray(a)), order=order)
    return np.asarray(a, order=order)


def empty(shape, *, dtype=None, order="C", like=None, device=None, usm_type="device", sycl_queue=None):
    return _wrap(dpt.empty(shape, dtype=dtype, order=order or "C"))


def zeros(shape, *, dtype=None, order="C", like=None, device=None, usm_type="device", sycl_queue=None):
    return _wrap(dpt.zeros(shape, dtype=dtype, order=order or "C"))


def ones(shape, *, dtype=None, order="C", like=None, device=None, usm_type="device", sycl_queue=None):
    return _wrap(dpt.ones(shape, dtype=dtype, order=order or "C"))


def full(shape, fill_value, *, dtype=None, order="C", like=None, device=None, usm_type=None, sycl_queue=None):
    fv = fill_value.get_array() if isinstance(fill_value, dpnp_array) else fill_value
    return _wrap(dpt.full(shape, fv, dtype=dtype, order=order or "C"))


def empty_like(a, /, *, dtype=None, order="C", subok=False, shape=None, device=None, usm_type=None,
               sycl_queue=None):
    _check_creation_subok(subok)
    u = get_usm_ndarray(a)
    if shape is not None:
        return _wrap(dpt.empty(shape, dtype=dtype or u.dtype, order="C" if order in ("K", "A") else order))
    return _wrap(dpt.empty_like(u, dtype=dtype, order=order))


def zeros_like(a, /, *, dtype=None, order="C", subok=False, shape=None, device=None, usm_type=None,
               sycl_queue=None):
    r = empty_like(a, dtype=dtype, order=order, shape=shape)
    r.fill(0)
    return r


def ones_like(a, /, *, dtype=None, order="C", subok=False, shape=None, device=None, usm_type=None,
              sycl_queue=None):
    r = empty_like(a, dtype=dtype, order=order, shape=shape)
    r.fill(1)
    return r


def full_like(a, /, fill_value, *, dtype=None, order="K", subok=False, shape=None, device=None, usm_type=None,
              sycl_queue=None):
    _check_creation_subok(subok)
    # dpnp/dpnp_iface_arraycreation.py:2426-2530
    r = empty_like(a, dtype=dtype, order=order, shape=shape)
    r.fill(fill_value.get_array() if isinstance(fill_value, dpnp_array) else fill_value)
    return r


def linspace(start, stop, /, num, *, dtype=None, device=None, usm_type=None, sycl_queue=None, endpoint=True,
             retstep=False, axis=0):
    # dpnp/dpnp_iface_arraycreation.py:2789-2900, scalar end points (the tensor-level constructor)
    if not (isscalar(start) and isscalar(stop)):
        raise NotImplementedError("linspace: only scalar start and stop are supported")
    if axis != 0:
        raise NotImplementedError("linspace: axis must be 0 for scalar end points")
    r = _wrap(dpt.linspace(start, stop, num, dtype=dtype, endpoint=endpoint))
    if retstep:
        div = (num - 1) if endpoint else num
        return r, ((stop - start) / div if div > 0 else float("nan"))
    return r


def arange(start, /, stop=None, step=1, *, dtype=None, like=None, device=None, usm_type="device",
           sycl_queue=None):
    return _wrap(dpt.arange(start, stop, step, dtype=dtype))


def broadcast_to(a, /, shape, subok=False):
    return _wrap(dpt.broadcast_to(get_usm_ndarray(a), shape))


def reshape(a, /, shape=None, order="C", *, copy=None):
    return _wrap(dpt.reshape(get_usm_ndarray(a), shape, order=order or "C", copy=copy))


def transpose(a, axes=None):
    u = get_usm_ndarray(a)
    return _wrap(u.T if axes is None else dpt.permute_dims(u, axes))


def astype(x, dtype, /, *, order="K", casting="unsafe", copy=True, device=None):
    return _wrap(dpt.astype(get_usm_ndarray(x), dtype, order=order, casting=casting, copy=copy))


def copyto(dst, src, casting="same_kind", where=True):
    check_limitations(where=where)
    d = get_usm_ndarray(dst)
    s = src if np.isscalar(src) else get_usm_ndarray(src)
    if not np.isscalar(src) and not np.can_cast(s.dtype, d.dtype, casting=casting):
        raise TypeError(f"Cannot cast from {s.dtype} to {d.dtype} according to the rule {casting}.")
    d[...] = s


def can_cast(from_, to, casting="safe"):
    f = from_.dtype if is_supported_array_type(from_) else from_
    return np.can_cast(f, to, casting=casting)


def result_type(*args):
    return dpt.result_type(*[get_usm_ndarray(a) if is_supported_array_type(a) else a for a in args])


# -- elementwise functions ----------------------------------------------------------------------------------
def _norm_order(order):
    if order is None:
        return "K"
    if isinstance(order, str) and len(order) == 1 and order in "afkcAFKC":
        return order.upper()
    raise ValueError(f"order must be one of 'C', 'F', 'A', or 'K' (got '{order}')")


def _check_ufunc_kwargs(name, where, subok, dtype, out, kwargs):
    if kwargs:
        raise NotImplementedError(f"Requested function={name} with kwargs={kwargs} isn't currently supported.")
    if where is not True:
        raise NotImplementedError(f"Requested function={name} with where={where} isn't currently supported.")
    if subok is not True:
        raise NotImplementedError(f"Requested function={name} with subok={subok} isn't currently supported.")
    if dtype is not None and out is not None:
        raise TypeError(f"Requested function={name} only takes `out` or `dtype` as an argument, "
                        "but both were provided.")


def _unpack_out(out, nout=1):
    if isinstance(out, tuple):
        if len(out) != nout:
            raise ValueError("'out' tuple must have exactly one entry per ufunc output")
        return out[0]
    return out


class DPNPUnaryFunc:
    """NumPy-style unary ufunc over a tensor-level elementwise function."""

    def __init__(self, name, tensor_fn):
        self.name_ = self.__name__ = name
        self._fn = tensor_fn
        self.__doc__ = tensor_fn.__doc__
        self.nin, self.nout = 1, 1

    @property
    def types(self):
        return self._fn.types

    def __call__(self, x, /, out=None, *, where=True, order="K", dtype=None, subok=True, **kwargs):
        if (out is None or type(out) is dpnp_array) and dtype is None and where is True and order == "K" \
                and subok is True and not kwargs and type(x) is dpnp_array:
            fn = self._fn
            if not fn._ext_types_known:
                fn._tell_ext_types()
            res = _ext.unary_call(fn._op_id, x, out)  # the plain case, checked on the descriptors
            if res is not NotImplemented:
                return res
            res = self._fn._fast(x._array_obj, None if out is None else out._array_obj)
            if res is not None:
                return _wrap(res) if out is None else out
        _check_ufunc_kwargs(self.name_, where, subok, dtype, out, kwargs)
        if not is_supported_array_type(x):
            raise TypeError(f"Input array must be any of supported type, but got {type(x)}")
        order = _norm_order(order)
        x_usm = get_usm_ndarray(x)
        if dtype is not None:
            x_usm = dpt.astype(x_usm, dtype, copy=False)
        out = _unpack_out(out)
        out_usm = None if out is None else get_usm_ndarray(out)
        res = self._fn(x_usm, out=out_usm, order=order)
        if out is not None and isinstance(out, dpnp_array):
            return out
        return _wrap(res)


class DPNPBinaryFunc:
    """NumPy-style binary ufunc over a tensor-level elementwise function."""

    def __init__(self, name, tensor_fn):
        self.name_ = self.__name__ = name
        self._fn = tensor_fn
        self.__doc__ = tensor_fn.__doc__
        self.nin, self.nout = 2, 1

    @property
    def types(self):
        return self._fn.types

    def __call__(self, x1, x2, /, out=None, *, where=True, order="K", dtype=None, subok=True, **kwargs):
        if (out is None or (type(out) is dpnp_array and out is not x1)) and dtype is None and where is True \
                and order == "K" and subok is True and not kwargs:
            # arrays and Python numbers, the keywords at their defaults: the tensor function's own short path
            t1, t2 = type(x1), type(x2)
            if t1 is dpnp_array and t2 is dpnp_array:
                fn = self._fn
                if not fn._ext_types_known:
                    fn._tell_ext_types()
                res = _ext.binary_call(fn._op_id, x1, x2, out)  # the plain case, checked on the descriptors
                if res is not NotImplemented:
                    return res
            uo = None if out is None else out._array_obj
            res = None
            if t1 is dpnp_array:
                if t2 is dpnp_array:
                    res = self._fn._fast(x1._array_obj, x2._array_obj, uo)
                elif t2 is float or t2 is int:
                    res = self._fn._fast(x1._array_obj, x2, uo)
            elif t2 is dpnp_array and (t1 is float or t1 is int):
                res = self._fn._fast(x1, x2._array_obj, uo)
            if res is not None:
                return _wrap(res) if out is None else out
        check_supported_arrays_type(x1, x2, scalar_type=True, all_scalars=False)
        _check_ufunc_kwargs(self.name_, where, subok, dtype, out, kwargs)
        u1, u2 = get_usm_ndarray_or_scalar(x1), get_usm_ndarray_or_scalar(x2)
        u1 = u1.item() if isinstance(u1, np.generic) else u1
        u2 = u2.item() if isinstance(u2, np.generic) else u2
        out = _unpack_out(out)
        out_usm = None if out is None else get_usm_ndarray(out)
        if isinstance(x1, dpnp_array) and x1 is out and order == "K" and dtype is None:
            self._fn._inplace_op(u1, u2)
            return x1
        order = _norm_order(order)
        if dtype is not None:
            u1 = dpt.asarray(u1, dtype=dtype) if np.isscalar(u1) else dpt.astype(u1, dtype, copy=False)
            u2 = dpt.asarray(u2, dtype=dtype) if np.isscalar(u2) else dpt.astype(u2, dtype, copy=False)
        res = self._fn(u1, u2, out=out_usm, order=order)
        if out is not None and isinstance(out, dpnp_array):
            return out
        return _wrap(res)

    def outer(self, x1, x2, out=None, where=True, order="K", dtype=None, subok=True, **kwargs):
        """The op over all pairs (a, b), a in x1 and b in x2: result shape x1.shape + x2.shape (a broadcast call on
        x1[..., None * x2.ndim] and x2[None * x1.ndim, ...]; DPNPBinaryFunc.outer,
        dpnp/dpnp_algo/dpnp_elementwise_common.py:741-847)."""
        check_supported_arrays_type(x1, x2, scalar_type=True, all_scalars=False)
        if not (np.isscalar(x1) or np.isscalar(x2)):
            n1, n2 = x1.ndim, x2.ndim
            x1 = x1[(Ellipsis,) + (None,) * n2]
            x2 = x2[(None,) * n1 + (Ellipsis,)]
        return self.__call__(x1, x2, out=out, where=where, order=order, dtype=dtype, subok=subok, **kwargs)


_UNARY = {
    "abs": ef.abs, "absolute": ef.abs, "negative": ef.negative, "positive": ef.positive,
    "square": ef.square, "sqrt": ef.sqrt, "exp": ef.exp, "log": ef.log, "erf": ef.erf, "sin": ef.sin,
    "cos": ef.cos, "tan": ef.tan, "tanh": ef.tanh, "exp2": ef.exp2, "expm1": ef.expm1, "log2": ef.log2,
    "log10": ef.log10, "log1p": ef.log1p, "rsqrt": ef.rsqrt, "cbrt": ef.cbrt, "reciprocal": ef.reciprocal,
    "floor": ef.floor, "ceil": ef.ceil, "trunc": ef.trunc, "sign": ef.sign, "isnan": ef.isnan,
    "isinf": ef.isinf, "isfinite": ef.isfinite, "logical_not": ef.logical_not, "invert": ef.bitwise_invert,
    "bitwise_not": ef.bitwise_invert, "bitwise_invert": ef.bitwise_invert, "signbit": ef.signbit,
    "arcsin": ef.asin, "asin": ef.asin, "arccos": ef.acos, "acos": ef.acos, "arctan": ef.atan, "atan": ef.atan,
    "sinh": ef.sinh, "cosh": ef.cosh, "arcsinh": ef.asinh, "asinh": ef.asinh, "arccosh": ef.acosh,
    "acosh": ef.acosh, "arctanh": ef.atanh, "atanh": ef.atanh, "rint": ef.round, "conj": ef.conj,
    "conjugate": ef.conj, "real": ef.real, "imag": ef.imag, "proj": ef.proj, "angle": ef.angle,
    "fabs": ef.fabs, "degrees": ef.degrees, "rad2deg": ef.degrees, "radians": ef.radians, "deg2rad": ef.radians,
    "sinc": ef.sinc, "spacing": ef.spacing, "bitwise_count": ef.bitwise_count, "erfc": ef.erfc, "erfcx": ef.erfcx,
    "erfinv": ef.erfinv, "erfcinv": ef.erfcinv, "i0": ef.i0,
}
_BINARY = {
    "add": ef.add, "subtract": ef.subtract, "multiply": ef.multiply, "divide": ef.divide,
    "true_divide": ef.divide, "bitwise_and": ef.bitwise_and, "bitwise_or": ef.bitwise_or,
    "bitwise_xor": ef.bitwise_xor, "equal": ef.equal, "not_equal": ef.not_equal, "less": ef.less,
    "less_equal": ef.less_equal, "greater": ef.greater, "greater_equal": ef.greater_equal,
    "maximum": ef.maximum, "minimum": ef.minimum, "logical_and": ef.logical_and,
    "logical_or": ef.logical_or, "logical_xor": ef.logical_xor, "power": ef.pow, "pow": ef.pow,
    "floor_divide": ef.floor_divide, "remainder": ef.remainder, "mod": ef.remainder,
    "arctan2": ef.atan2, "atan2": ef.atan2, "hypot": ef.hypot, "copysign": ef.copysign,
    "left_shift": ef.bitwise_left_shift, "bitwise_left_shift": ef.bitwise_left_shift,
    "right_shift": ef.bitwise_right_shift, "bitwise_right_shift": ef.bitwise_right_shift,
    "logaddexp": ef.logaddexp, "nextafter": ef.nextafter, "fmax": ef.fmax, "fmin": ef.fmin, "fmod": ef.fmod,
    "logaddexp2": ef.logaddexp2, "heaviside": ef.heaviside, "gcd": ef.gcd, "lcm": ef.lcm,
}
for _n, _f in _UNARY.items():
    globals()[_n] = DPNPUnaryFunc(_n, _f)
for _n, _f in _BINARY.items():
    globals()[_n] = DPNPBinaryFunc(_n, _f)


def float_power(x1, x2, /, out=None, *, where=True, order="K", dtype=None, subok=True, **kwargs):
    """x1 ** x2 computed in at least float64 (complex128 for complex operands), as
    dpnp.float_power (dpnp/dpnp_iface_mathematical.py:1952-2030)."""
    _check_ufunc_kwargs("float_power", where, subok, dtype, out, kwargs)
    if dtype is not None:
        tgt = dpt.dtype(dtype)
    else:
        kinds = [get_usm_ndarray(v).dtype if is_supported_array_type(v) else np.result_type(v) for v in (x1, x2)]
        tgt = dpt.dtype("c16" if _builtins.any(k.kind == "c" for k in kinds) else "f8")
    if tgt.kind not in "fc":
        raise TypeError(f"float_power needs a floating or complex result type, got {tgt}")
    return globals()["power"](x1, x2, out=out, order=order, dtype=tgt)


def divmod(x1, x2, /, out1=None, out2=None, *, out=(None, None), where=True, order="K", dtype=None,  # noqa: A001
           subok=True, **kwargs):
    """(x1 // x2, x1 % x2): dpnp.divmod (dpnp/dpnp_iface_mathematical.py:1619-1700); the reference
    runs one two-output kernel, here the two existing kernels run back to back."""
    o1, o2 = (out1, out2) if (out1 is not None or out2 is not None) else tuple(out)
    q = globals()["floor_divide"](x1, x2, out=o1, where=where, order=order, dtype=dtype, subok=subok, **kwargs)
    r = globals()["remainder"](x1, x2, out=o2, where=where, order=order, dtype=dtype, subok=subok, **kwargs)
    return q, r


def modf(x, /, out1=None, out2=None, *, out=(None, None), where=True, order="K", dtype=None, subok=True,
         **kwargs):
    """(fractional part, integral part), both with the sign of x: dpnp.modf
    (dpnp/dpnp_iface_mathematical.py:3494-3560)."""
    o1, o2 = (out1, out2) if (out1 is not None or out2 is not None) else tuple(out)
    u = get_usm_ndarray(x)
    if u.dtype.kind not in "f":
        if u.dtype.kind == "c":
            raise ValueError("modf does not support complex input")
        x = astype(x, "f8" if u.dtype.itemsize >= 4 else ("f4" if u.dtype.itemsize == 2 else "f2"))
    whole = globals()["trunc"](x, out=o2, where=where, order=order, dtype=dtype, subok=subok, **kwargs)
    frac = globals()["subtract"](x, whole, out=o1, order=order)
    # inf - inf is NaN but the fractional part of an infinity is a zero; zeros keep the sign of x
    fu = get_usm_ndarray(frac)
    xu = get_usm_ndarray(x)
    fixed = dpt.where(dpt.isinf(xu), dpt.asarray(0, dtype=fu.dtype), fu)
    dpt.copysign(fixed, xu, out=fu)
    return frac, whole


def _checked_out(out, shape, dt, name):
    """The usm_ndarray behind a user-supplied `out`, validated as the ufunc wrappers do."""
    u = get_usm_ndarray(out)
    if tuple(u.shape) != tuple(shape):
        raise ValueError(f"The shape of input and output arrays are inconsistent. Expected output shape is "
                         f"{tuple(shape)}, got {tuple(u.shape)}")
    if u.dtype != dt:
        raise ValueError(f"Output array of type {dt} is needed, got {u.dtype}")
    if not u.flags.writable:
        raise ValueError(f"{name}: output array is read-only")
    return u


def ldexp(x1, x2, /, out=None, *, where=True, order="K", dtype=None, subok=True, **kwargs):
    """x1 * 2**x2 for a floating x1 and an integer x2: dpnp.ldexp
    (dpnp/dpnp_iface_mathematical.py:3150-3220).  Integer x1 converts to the smallest float type that
    holds it, unsigned x2 to the next signed type; a Python int as x2 is the default integer type."""
    _check_ufunc_kwargs("ldexp", where, subok, dtype, out, kwargs)
    check_supported_arrays_type(x1, x2, scalar_type=True)

    def bad(d1, d2):
        return ValueError(f"function 'ldexp' does not support input types ({d1}, {d2}), and the inputs could not "
                          "be safely coerced to any supported types according to the casting rule ''safe''.")

    d1 = get_usm_ndarray(x1).dtype if is_supported_array_type(x1) else np.result_type(x1)
    d2 = get_usm_ndarray(x2).dtype if is_supported_array_type(x2) else np.result_type(x2)
    if d1.kind in "biu":
        f1 = np.dtype("f2" if d1.itemsize == 1 else ("f4" if d1.itemsize == 2 else "f8"))
        if not is_supported_array_type(x1):
            f1 = np.dtype("f8")
    elif d1.kind == "f":
        f1 = d1 if is_supported_array_type(x1) else np.dtype("f8")
    else:
        raise bad(d1, d2)
    if not is_supported_array_type(x2):
        if d2.kind not in "biu":
            raise bad(d1, d2)
        i2 = np.dtype("i8")
    elif d2.kind == "i":
        i2 = d2
    elif d2.kind in "bu" and d2.itemsize < 8:
        i2 = np.dtype("i1" if d2.kind == "b" else "i" + str(2 * d2.itemsize))
    else:
        raise bad(d1, d2)
    u1 = dpt.astype(get_usm_ndarray(x1), f1, copy=False) if is_supported_array_type(x1) else dpt.asarray(x1, dtype=f1)
    u2 = dpt.astype(get_usm_ndarray(x2), i2, copy=False) if is_supported_array_type(x2) else dpt.asarray(x2, dtype=i2)
    shape = np.broadcast_shapes(u1.shape, u2.shape)
    u1, u2 = dpt.broadcast_to(u1, shape), dpt.broadcast_to(u2, shape)
    res = None
    if out is not None:
        ou = get_usm_ndarray(_unpack_out(out))
        if tuple(ou.shape) == tuple(shape) and ou.dtype == f1 and ou.flags.writable and not (
                ti._array_overlap(ou, u1) and not ti._same_logical_tensors(ou, u1)) and not ti._array_overlap(ou, u2):
            res = ou
    if res is None:
        res = dpt.empty(shape, dtype=f1, order="F" if order == "F" else "C")
    if res.size:
        tei._ldexp(u1, u2, res)
    if dtype is not None and np.dtype(dtype) != f1:
        if not np.can_cast(f1, np.dtype(dtype), "same_kind"):
            raise TypeError(f"Cannot cast ufunc 'ldexp' output from dtype({f1}) to dtype({np.dtype(dtype)})")
        res = dpt.astype(res, dtype)
    if out is not None:
        return get_result_array(_wrap(res), _unpack_out(out), casting="same_kind")
    return _wrap(res)


def frexp(x, out1=None, out2=None, /, *, out=(None, None), where=True, order="K", dtype=None, subok=True,
          **kwargs):
    """(mantissa, exponent) with x = mantissa * 2**exponent and |mantissa| in [0.5, 1): dpnp.frexp
    (dpnp/dpnp_iface_mathematical.py:2395-2457); the exponent is int32."""
    _check_ufunc_kwargs("frexp", where, subok, None, None, kwargs)
    if dtype is not None:
        raise NotImplementedError("frexp: the `dtype` keyword is not supported")
    check_supported_arrays_type(x)
    o1, o2 = (out1, out2) if (out1 is not None or out2 is not None) else tuple(out)
    u = get_usm_ndarray(x)
    if u.dtype.kind == "c":
        raise ValueError(f"function 'frexp' does not support input type ({u.dtype}), and the input could not be "
                         "safely coerced to any supported types according to the casting rule ''safe''.")
    if u.dtype.kind != "f":
        u = dpt.astype(u, "f2" if u.dtype.itemsize == 1 else ("f4" if u.dtype.itemsize == 2 else "f8"))
    mant = _checked_out(o1, u.shape, u.dtype, "frexp") if o1 is not None else dpt.empty_like(u, order=order or "K")
    expo = _checked_out(o2, u.shape, np.dtype("i4"), "frexp") if o2 is not None else dpt.empty_like(
        u, dtype="i4", order=order or "K")
    if u.size:
        tei._frexp(u, mant, expo)
    return (o1 if isinstance(o1, dpnp_array) else _wrap(mant)), (o2 if isinstance(o2, dpnp_array) else _wrap(expo))


def clip(a, /, min=None, max=None, *, out=None, order="K", **kwargs):  # noqa: A002
    """Values of `a` limited to [min, max]: dpnp.clip (dpnp/dpnp_iface_mathematical.py:722-830)."""
    if kwargs:
        raise NotImplementedError(f"kwargs={kwargs} is currently not supported")
    order = order if order is not None else "K"
    usm_min = None if min is None else get_usm_ndarray_or_scalar(min)
    usm_max = None if max is None else get_usm_ndarray_or_scalar(max)
    usm_out = None if out is None else get_usm_ndarray(out)
    res = dpt.clip(get_usm_ndarray(a), usm_min, usm_max, out=usm_out, order=order)
    if out is not None and isinstance(out, dpnp_array):
        return out
    return _wrap(res)


def nan_to_num(x, copy=True, nan=0.0, posinf=None, neginf=None):
    """NaN -> `nan`, +inf -> `posinf` (largest finite value by default), -inf -> `neginf`:
    dpnp.nan_to_num (dpnp/dpnp_iface_mathematical.py:3584-3760), scalar replacement values."""
    check_supported_arrays_type(x)
    u = get_usm_ndarray(x)
    if u.dtype.kind not in "fc":
        return _wrap(dpt.copy(u)) if copy else get_result_array(x)
    for v in (nan, posinf, neginf):
        if v is not None and not isinstance(v, (int, float)):
            raise NotImplementedError("nan_to_num with array replacement values is outside this library's scope")
    real_dt = np.dtype("f" + str(u.dtype.itemsize // 2)) if u.dtype.kind == "c" else u.dtype
    info = np.finfo(real_dt)
    hi = float(info.max) if posinf is None else posinf
    lo = float(info.min) if neginf is None else neginf
    if copy:
        out = dpt.empty_like(u)
    else:
        if not u.flags.writable:
            raise ValueError("copy is required for read-only array `x`")
        out = u
    if u.size:
        tei._nan_to_num(u, nan, hi, lo, out)
    return _wrap(out) if copy else get_result_array(x)


def isclose(a, b, rtol=1e-05, atol=1e-08, equal_nan=False):
    """|a - b| <= atol + rtol * |b| elementwise, infinities equal to themselves, NaNs equal when
    equal_nan: dpnp.isclose with scalar tolerances (dpnp/dpnp_iface_logic.py:824-960)."""
    check_supported_arrays_type(a, b, scalar_type=True)
    if not (np.isscalar(rtol) and np.isscalar(atol)):
        raise NotImplementedError("isclose with array tolerances is outside this library's scope")
    dt = result_type(a, b, 1.0)
    ua = dpt.asarray(a, dtype=dt) if np.isscalar(a) else dpt.astype(get_usm_ndarray(a), dt, copy=False)
    ub = dpt.asarray(b, dtype=dt) if np.isscalar(b) else dpt.astype(get_usm_ndarray(b), dt, copy=False)
    rtol = rtol.real if isinstance(rtol, complex) else rtol
    atol = atol.real if isinstance(atol, complex) else atol
    shape = np.broadcast_shapes(ua.shape, ub.shape)
    ua, ub = dpt.broadcast_to(ua, shape), dpt.broadcast_to(ub, shape)
    out = dpt.empty(shape, dtype="?")
    if out.size:
        tei._isclose_scalar(ua, ub, rtol, atol, True if equal_nan else False, out)
    return _wrap(out)


def where(condition, x=None, y=None, /, *, order="K", out=None):
    """Elements of `x` where `condition` holds, else of `y`."""
    if order == "K" and x is not None and y is not None:
        r = _ext.where_call(condition, x, y, out)  # arrays with branches of one dtype, on the descriptors
        if r is not NotImplemented:
            return r
    if out is None and type(condition) is dpnp_array and type(x) is dpnp_array and type(y) is dpnp_array:
        return _wrap(dpt.where(condition._array_obj, x._array_obj, y._array_obj, order=order))
    missing = (x is None, y is None).count(True)
    if missing == 1:
        raise ValueError("Must provide both 'x' and 'y' or neither.")
    if missing == 2:
        raise NotImplementedError("where(condition) without x and y (nonzero) is outside this library's scope")
    ux, uy = get_usm_ndarray_or_scalar(x), get_usm_ndarray_or_scalar(y)
    ux = ux.item() if isinstance(ux, np.generic) else ux
    uy = uy.item() if isinstance(uy, np.generic) else uy
    out_usm = None if out is None else get_usm_ndarray(out)
    res = dpt.where(get_usm_ndarray(condition), ux, uy, order=order, out=out_usm)
    return get_result_array(res, out)


# -- reductions ---------------------------------------------------------------------------------------------
_R_SUM, _R_PROD, _R_MAX, _R_MIN = (_lib.REDUCE_ID[n] for n in ("sum", "prod", "max", "min"))
_S_ARGMAX, _S_ARGMIN = _lib.SEARCH_ID["argmax"], _lib.SEARCH_ID["argmin"]
def _wrap_reduction_call(usm_a, out, fn, res_dt, **kwargs):
    """Run a tensor-level reduction; an `out` of another dtype gets an unsafe cast of the result."""
    usm_out = None
    if out is not None:
        check_supported_arrays_type(out)
        usm_out = get_usm_ndarray(out)
        if usm_out.dtype != res_dt:
            usm_out = None  # compute into a fresh array of the kernel's dtype, cast into `out` below
    res = fn(usm_a, out=usm_out, **kwargs)
    return get_result_array(res, out, casting="unsafe")


def _reduction_res_dt(a, dtype):
    return _default_accumulation_dtype(a.dtype) if dtype is None else dpt.dtype(dtype)


def sum(a, axis=None, dtype=None, out=None, keepdims=False, initial=None, where=True):  # noqa: A001
    if dtype is None and keepdims is False and initial is None and where is True:
        r = _ext.reduce_call(_R_SUM, a, axis, out)  # the plain call, on the descriptors; else the general path
        if r is not NotImplemented:
            return r
    check_limitations(initial=initial, where=where)
    u = get_usm_ndarray(a)
    return _wrap_reduction_call(u, out, dpt.sum, _reduction_res_dt(u, dtype), axis=axis, dtype=dtype,
                                keepdims=keepdims)


def prod(a, axis=None, dtype=None, out=None, keepdims=False, initial=None, where=True):
    if dtype is None and keepdims is False and initial is None and where is True:
        r = _ext.reduce_call(_R_PROD, a, axis, out)
        if r is not NotImplemented:
            return r
    check_limitations(initial=initial, where=where)
    u = get_usm_ndarray(a)
    return _wrap_reduction_call(u, out, dpt.prod, _reduction_res_dt(u, dtype), axis=axis, dtype=dtype,
                                keepdims=keepdims)


def max(a, axis=None, out=None, keepdims=False, initial=None, where=True):  # noqa: A001
    if keepdims is False and initial is None and where is True:
        r = _ext.reduce_call(_R_MAX, a, axis, out)
        if r is not NotImplemented:
            return r
    check_limitations(initial=initial, where=where)
    u = get_usm_ndarray(a)
    return _wrap_reduction_call(u, out, dpt.max, u.dtype, axis=axis, keepdims=keepdims)


def min(a, axis=None, out=None, keepdims=False, initial=None, where=True):  # noqa: A001
    if keepdims is False and initial is None and where is True:
        r = _ext.reduce_call(_R_MIN, a, axis, out)
        if r is not NotImplemented:
            return r
    check_limitations(initial=initial, where=where)
    u = get_usm_ndarray(a)
    return _wrap_reduction_call(u, out, dpt.min, u.dtype, axis=axis, keepdims=keepdims)


amax, amin = max, min


def all(a, /, axis=None, out=None, keepdims=False, *, where=True):  # noqa: A001
    check_limitations(where=where)
    u = get_usm_ndarray(a)
    return _wrap_reduction_call(u, out, dpt.all, dpt.bool, axis=axis, keepdims=keepdims)


def any(a, /, axis=None, out=None, keepdims=False, *, where=True):  # noqa: A001
    check_limitations(where=where)
    u = get_usm_ndarray(a)
    return _wrap_reduction_call(u, out, dpt.any, dpt.bool, axis=axis, keepdims=keepdims)


def count_nonzero(a, axis=None, *, keepdims=False, out=None):
    u = get_usm_ndarray(a)
    return _wrap_reduction_call(u, out, dpt.count_nonzero, dpt.int64, axis=axis, keepdims=keepdims)


def logsumexp(x, /, *, axis=None, out=None, dtype=None, keepdims=False):
    u = get_usm_ndarray(x)
    res_dt = dpt.dtype(dtype) if dtype is not None else (u.dtype if u.dtype.kind == "f" else dpt.float64)
    return _wrap_reduction_call(u, out, dpt.logsumexp, res_dt, axis=axis, dtype=dtype, keepdims=keepdims)


def reduce_hypot(x, /, *, axis=None, out=None, dtype=None, keepdims=False):
    u = get_usm_ndarray(x)
    res_dt = dpt.dtype(dtype) if dtype is not None else (u.dtype if u.dtype.kind == "f" else dpt.float64)
    return _wrap_reduction_call(u, out, dpt.reduce_hypot, res_dt, axis=axis, dtype=dtype, keepdims=keepdims)


def _search_res_dt(out):
    res_dt = dpt.dtype(ti.default_device_index_type())
    if out is not None and not np.can_cast(out.dtype, res_dt, casting="safe"):
        raise TypeError(f"Cannot cast from {out.dtype} to {res_dt} according to the rule safe.")
    return res_dt


def argmax(a, axis=None, out=None, *, keepdims=False):
    if keepdims is False:
        r = _ext.search_call(_S_ARGMAX, a, axis, out)
        if r is not NotImplemented:
            return r
    u = get_usm_ndarray(a)
    return _wrap_reduction_call(u, out, dpt.argmax, _search_res_dt(out), axis=axis, keepdims=keepdims)


def argmin(a, axis=None, out=None, *, keepdims=False):
    if keepdims is False:
        r = _ext.search_call(_S_ARGMIN, a, axis, out)
        if r is not NotImplemented:
            return r
    u = get_usm_ndarray(a)
    return _wrap_reduction_call(u, out, dpt.argmin, _search_res_dt(out), axis=axis, keepdims=keepdims)


def _wider_float(u, dtype):
    """dtype to accumulate in when the caller asks for a wider floating result than the
    input's: the statistics then run in that type end to end.  (The reference computes in
    the input's type and casts the result, dpnp/dpnp_iface_statistics.py:1203-1205; this is
    never less accurate.)"""
    if dtype is None:
        return None
    d = dpt.dtype(dtype)
    if u.dtype.kind == "f" and d.kind == "f" and d.itemsize > u.dtype.itemsize:
        return d
    return None


def mean(a, /, axis=None, dtype=None, out=None, keepdims=False, *, where=True):
    check_limitations(where=where)
    u = get_usm_ndarray(a)
    res = dpt.mean(u, axis=axis, keepdims=keepdims, dtype=_wider_float(u, dtype))
    if dtype is not None:
        res = dpt.astype(res, dtype, copy=False)
    return get_result_array(res, out, casting="unsafe")


_mean = mean  # (var and std have a parameter of that name)


def _check_ddof(ddof, correction):
    if correction is not None:
        if ddof != 0:
            raise ValueError("ddof and correction can't be provided simultaneously.")
        ddof = correction
    if not isinstance(ddof, (int, float)):
        raise TypeError(f"An integer or float is required, but got {type(ddof)}")
    return ddof


def _var_around_mean(a, u, axis, dtype, out, ddof, keepdims, mean):
    """Variance of complex data, or around a mean the caller brings: dpnp/dpnp_iface_statistics.py:1832-1869.

    sum(|a - mean|**2) / (N - ddof), with the reference's dtype rules (integer and bool input computes in
    the default floating type; the deviations live in the type `a - mean` promotes to; the sum is taken
    in `dtype` when given) and its divisor (N - ddof as it comes, NaN when that is zero).  The common
    shapes run as one kernel (tensor._sum_abs_sqdev); anything else as the reference's own sequence of calls.
    """
    if dtype is None and u.dtype.kind not in "fc":
        dtype = dpt.float64
    um = None if mean is None else get_usm_ndarray(mean)
    fused = None
    if u.dtype.kind == "c":
        if dtype is None:
            m = um if um is not None else dpt.mean(u, axis=axis, keepdims=True)
            fused = dpt._statistical_functions._sum_abs_sqdev(u, m, axis, keepdims)
    elif um is not None and um.dtype.kind != "c":
        # the type the reference's deviations and their sum would have
        res_dt = dpt.dtype(dtype) if dtype is not None else np.result_type(u.dtype, um.dtype)
        if res_dt.kind == "f":
            fused = dpt._statistical_functions._sum_abs_sqdev(u, um, axis, keepdims, dtype=res_dt)
    if fused is not None:
        result = get_result_array(fused, out, casting="unsafe")
    else:
        arrmean = mean if mean is not None else _mean(a, axis=axis, dtype=dtype, keepdims=True)
        x = subtract(a, arrmean)
        if x.dtype.kind == "c":
            x = multiply(x, x.conj(), out=x).real
        else:
            x = square(x, out=x)
        result = sum(x, axis=axis, dtype=dtype, out=out, keepdims=keepdims)
    axes = range(u.ndim) if axis is None else (axis if isinstance(axis, (tuple, list)) else (axis,))
    items = 1
    for ax in axes:
        items *= u.shape[ax]
    # (the reference writes numpy.max(items - ddof, 0): the 0 is an axis, nothing is clamped)
    cnt = np.asarray(np.intp(items) - ddof).astype(result.dtype, casting="same_kind").item()
    ur = get_usm_ndarray(result)
    if ur.size:
        tei._divide_by_scalar(src=ur, scalar=cnt if cnt else np.nan, dst=ur)
    return result


def var(a, /, axis=None, dtype=None, out=None, ddof=0, keepdims=False, *, where=True, mean=None,
        correction=None):
    check_supported_arrays_type(a)
    check_limitations(where=where)
    ddof = _check_ddof(ddof, correction)
    u = get_usm_ndarray(a)
    if u.dtype.kind == "c" or mean is not None:
        result = _var_around_mean(a, u, axis, dtype, out, ddof, keepdims, mean)
    else:
        res = dpt.var(u, axis=axis, correction=ddof, keepdims=keepdims, dtype=_wider_float(u, dtype))
        result = get_result_array(res, out)
    if out is None and dtype is not None:
        result = result.astype(dtype, casting="same_kind")
    return result


def std(a, /, axis=None, dtype=None, out=None, ddof=0, keepdims=False, *, where=True, mean=None,
        correction=None):
    check_supported_arrays_type(a)
    check_limitations(where=where)
    ddof = _check_ddof(ddof, correction)
    u = get_usm_ndarray(a)
    if u.dtype.kind == "c" or mean is not None:
        # dpnp/dpnp_iface_statistics.py:1644-1656: the variance in its own type, then the root in place
        result = var(a, axis=axis, dtype=None, out=out, ddof=ddof, keepdims=keepdims, where=where, mean=mean)
        sqrt(result, out=result)
    else:
        res = dpt.std(u, axis=axis, correction=ddof, keepdims=keepdims, dtype=_wider_float(u, dtype))
        result = get_result_array(res, out)
    if out is None and dtype is not None:
        result = result.astype(dtype, casting="same_kind")
    return result


# -- fused chains (extensions: one kernel where the reference runs a sequence) ---------------------------------
def where_compare(cmp_name, lhs, rhs, x, y, out=None):
    """`where(lhs CMP rhs, x, y)` in one pass; cmp_name in equal/not_equal/less/less_equal/
    greater/greater_equal.  All four operands must share a shape after broadcasting; lhs/rhs
    share a dtype and x/y share a dtype (scalars adopt the array operand's dtype)."""
    from .tensor._elementwise_common import _scalar_operand

    us = [o._array_obj if type(o) is dpnp_array else (o if type(o) is usm_ndarray else None) for o in (lhs, rhs, x, y)]
    if us[0] is None and us[1] is None or us[2] is None and us[3] is None:
        if not _builtins.any(u is not None for u in us):
            raise TypeError("at least one operand must be an array")
        raise TypeError("each of (lhs, rhs) and (x, y) needs an array operand")
    shapes = [u._shape for u in us if u is not None]
    shape = shapes[0]
    if _builtins.any(sh != shape for sh in shapes[1:]):
        from .tensor._manipulation_functions import _broadcast_shape_impl

        shape = _broadcast_shape_impl(shapes)

    def pair(a, b, ua, ub):
        dt = (ua if ua is not None else ub)._dtype
        # a Python number becomes the kept 0-d device array of that value, seen with the result's shape
        ua = _scalar_operand(a, dt, shape) if ua is None else (ua if ua._shape == shape else dpt.broadcast_to(ua, shape))
        ub = _scalar_operand(b, dt, shape) if ub is None else (ub if ub._shape == shape else dpt.broadcast_to(ub, shape))
        if ua._dtype != ub._dtype:
            raise ValueError("operands of a pair must have one dtype")
        return ua, ub

    ul, ur = pair(lhs, rhs, us[0], us[1])
    ux, uy = pair(x, y, us[2], us[3])
    res = usm_ndarray._new_contiguous(tuple(shape), ux._dtype) if out is None else get_usm_ndarray(out)
    ti._where_compare(cmp_name, ul, ur, ux, uy, res)
    return out if out is not None else _wrap(res)


def black_scholes(price, strike, t, rate, vol, call=None, put=None):
    """Call and put prices of European options (one fused kernel); returns (call, put)."""
    up, us, ut = get_usm_ndarray(price), get_usm_ndarray(strike), get_usm_ndarray(t)
    uc = dpt.empty_like(up) if call is None else get_usm_ndarray(call)
    uq = dpt.empty_like(up) if put is None else get_usm_ndarray(put)
    tei._black_scholes(up, us, ut, rate, vol, uc, uq)
    return (call if call is not None else _wrap(uc)), (put if put is not None else _wrap(uq))


def synchronize():
    """Wait for all work queued by this library (and torch) on the current stream."""
    dpt._device.default_queue().wait()


__all__ = [n for n in list(globals()) if not n.startswith("_") and n not in (
    "np", "dpt", "ef", "tei", "ti", "usm_ndarray", "dpnp_array")]
