"""where(condition, x1, x2): behaviour of dpnp/tensor/_search_functions.py:126-415."""
import numpy as np

from . import _tensor_impl as ti
from ._copy_utils import _empty_like_orderK, _empty_like_triple_orderK
from ._ctors import empty, empty_like
from ._dtypes import bool as _bool_dt
from ._dtypes import complex128, dtype as _as_dtype, float64, int64
from ._elementwise_common import _as_device_array, _operand_dtype, _operand_shape
from ._manipulation_functions import _broadcast_shape_impl, broadcast_to
from ._type_utils import (
    WeakBooleanType,
    WeakComplexType,
    WeakFloatingType,
    WeakIntegralType,
    _is_weak_dtype,
    _resolve_weak_types,
)
from ._usmarray import usm_ndarray


def _default_dtype_from_weak_type(d):
    if isinstance(d, WeakBooleanType):
        return _bool_dt
    if isinstance(d, WeakIntegralType):
        return int64
    if isinstance(d, WeakFloatingType):
        return float64
    if isinstance(d, WeakComplexType):
        return complex128
    raise TypeError(d)


def _resolve_two_weak_types(d1, d2):
    if _is_weak_dtype(d1) and _is_weak_dtype(d2):
        return _default_dtype_from_weak_type(d1), _default_dtype_from_weak_type(d2)
    return _resolve_weak_types(d1, d2)


def where(condition, x1, x2, /, *, order="K", out=None):
    """Elements of `x1` where `condition` is true, of `x2` elsewhere; the three operands
    broadcast together and the result has the promoted dtype of `x1` and `x2`."""
    if out is None and order == "K" and type(condition) is usm_ndarray and type(x1) is usm_ndarray \
            and type(x2) is usm_ndarray and x1._dtype == x2._dtype and condition._shape == x1._shape == x2._shape \
            and condition._is_c_contiguous() and x1._is_c_contiguous() and x2._is_c_contiguous() and x1.size:
        # three C-contiguous arrays of one shape, branches of one dtype: nothing to promote, broadcast or lay out
        r = usm_ndarray._new_contiguous(x1._shape, x1._dtype)
        ti._where(condition=condition, x1=x1, x2=x2, dst=r)
        return r
    if not isinstance(condition, usm_ndarray):
        raise TypeError(f"Expecting dpnp_amd.tensor.usm_ndarray type, got {type(condition)}")
    if order not in ("K", "C", "F", "A"):
        order = "K"
    sc, s1, s2 = condition.shape, _operand_shape(x1), _operand_shape(x2)
    if s1 is None or s2 is None:
        raise TypeError("Shape of arguments can not be inferred. Arguments are expected to be "
                        "lists, tuples, or both")
    try:
        res_shape = _broadcast_shape_impl([sc, s1, s2])
    except ValueError:
        raise ValueError(f"operands could not be broadcast together with shapes {sc}, {s1}, and {s2}")
    d1, d2 = _operand_dtype(x1), _operand_dtype(x2)
    if d1 is None or d2 is None:
        raise ValueError("Operands have unsupported data types")
    d1, d2 = _resolve_two_weak_types(d1, d2)
    out_dt = _as_dtype(np.result_type(d1, d2))

    orig_out = out
    if out is not None:
        if not isinstance(out, usm_ndarray):
            raise TypeError(f"output array must be of usm_ndarray type, got {type(out)}")
        if not out.flags.writable:
            raise ValueError("provided `out` array is read-only")
        if out.shape != res_shape:
            raise ValueError("The shape of input and output arrays are inconsistent. "
                             f"Expected output shape is {res_shape}, got {out.shape}")
        if out_dt != out.dtype:
            raise ValueError(f"Output array of type {out_dt} is needed, got {out.dtype}")
        clash = ti._array_overlap(condition, out) and not ti._same_logical_tensors(condition, out)
        for xo, xd in ((x1, d1), (x2, d2)):
            if isinstance(xo, usm_ndarray) and xd == out_dt:
                clash = clash or (ti._array_overlap(xo, out) and not ti._same_logical_tensors(xo, out))
        if clash:
            out = empty_like(out)

    x1 = _as_device_array(x1, d1)
    x2 = _as_device_array(x2, d2)
    if order == "A":
        order = "F" if all(a.flags.f_contiguous for a in (condition, x1, x2)) else "C"

    def alloc():
        if order == "K":
            return _empty_like_triple_orderK(condition, x1, x2, out_dt, res_shape)
        return empty(res_shape, dtype=out_dt, order=order)

    if condition.size == 0:
        return out if out is not None else alloc()

    def cast(x):
        if x.dtype == out_dt:
            return x
        b = _empty_like_orderK(x, out_dt) if order == "K" else empty_like(x, dtype=out_dt, order=order)
        ti._copy_usm_ndarray_into_usm_ndarray(src=x, dst=b)
        return b

    x1, x2 = cast(x1), cast(x2)
    if out is None:
        out = alloc()
    cond = condition if sc == res_shape else broadcast_to(condition, res_shape)
    if x1.shape != res_shape:
        x1 = broadcast_to(x1, res_shape)
    if x2.shape != res_shape:
        x2 = broadcast_to(x2, res_shape)
    ti._where(condition=cond, x1=x1, x2=x2, dst=out)
    if orig_out is not None and orig_out is not out:
        ti._copy_usm_ndarray_into_usm_ndarray(src=out, dst=orig_out)
        out = orig_out
    return out
