"""clip(x, min, max): behaviour of dpnp/tensor/_clip.py:54-771 (one bound: 75-270, both: 273-771).

The result always has the dtype of `x`; a bound must cast safely to it.  With both bounds one native
call computes min(max(x, lo), hi); with one bound the call is maximum / minimum; with none a copy."""

from . import _tensor_impl as ti
from ._copy_utils import _empty_like_orderK, _empty_like_pair_orderK, _empty_like_triple_orderK
from ._ctors import empty, empty_like
from ._dtypes import iinfo
from ._elementwise_common import _as_device_array, _operand_dtype, _operand_shape
from ._manipulation_functions import _broadcast_shape_impl, broadcast_to
from ._type_utils import _can_cast, _resolve_one_strong_two_weak_types, _resolve_weak_types
from ._usmarray import usm_ndarray


def _checked_out(out, res_shape, res_dt, operands):
    """`out` itself, or a temporary of its layout when it overlaps an operand it is not identical to."""
    if not isinstance(out, usm_ndarray):
        raise TypeError(f"output array must be of usm_ndarray type, got {type(out)}")
    if not out.flags.writable:
        raise ValueError("provided `out` array is read-only")
    if out.shape != res_shape:
        raise ValueError("The shape of input and output arrays are inconsistent. "
                         f"Expected output shape is {res_shape}, got {out.shape}")
    if res_dt != out.dtype:
        raise ValueError(f"Output array of type {res_dt} is needed, got {out.dtype}")
    for o in operands:
        if isinstance(o, usm_ndarray) and ti._array_overlap(o, out) and not ti._same_logical_tensors(o, out):
            return empty_like(out)
    return out


def _unsupported(*dts):
    return ValueError(f"function 'clip' does not support input types ({', '.join(str(d) for d in dts)}), "
                      "and the inputs could not be safely coerced to any supported types according to the "
                      "casting rule ''safe''.")


def _bound_as_array(val, val_dt, res_dt, order):
    """The bound as a device array of the result dtype (converted through a copy when it is not)."""
    a = _as_device_array(val, val_dt)
    if a.dtype == res_dt:
        return a
    b = _empty_like_orderK(a, res_dt) if order == "K" else empty_like(a, dtype=res_dt, order=order)
    ti._copy_usm_ndarray_into_usm_ndarray(src=a, dst=b)
    return b


def _clip_one_bound(x, val, out, order, lower):
    # dpnp/tensor/_clip.py:75-270
    val_shape = _operand_shape(val)
    if val_shape is None:
        raise TypeError("Shape of arguments can not be inferred. Arguments are expected to be "
                        "lists, tuples, or both")
    try:
        res_shape = _broadcast_shape_impl([x.shape, val_shape])
    except ValueError:
        raise ValueError(f"operands could not be broadcast together with shapes {x.shape} and {val_shape}")
    val_dt = _operand_dtype(val)
    if val_dt is None:
        raise ValueError("Operands have unsupported data types")
    _, val_dt = _resolve_weak_types(x.dtype, val_dt)
    res_dt = x.dtype
    if not _can_cast(val_dt, res_dt):
        raise _unsupported(x.dtype, val_dt)
    orig_out = out
    if out is not None:
        out = _checked_out(out, res_shape, res_dt, (x, val))
    if order == "A":
        vf = val.flags.f_contiguous if isinstance(val, usm_ndarray) else True
        order = "F" if (x.flags.f_contiguous and vf) else "C"
    b = _bound_as_array(val, val_dt, res_dt, order)
    if out is None:
        out = _empty_like_pair_orderK(x, b, res_dt, res_shape) if order == "K" else empty(res_shape, dtype=res_dt, order=order)
    if out.size:
        xb = x if x.shape == res_shape else broadcast_to(x, res_shape)
        bb = b if b.shape == res_shape else broadcast_to(b, res_shape)
        from . import _tensor_elementwise_impl as tei

        (tei._maximum if lower else tei._minimum)(xb, bb, out)
    if orig_out is not None and orig_out is not out:
        ti._copy_usm_ndarray_into_usm_ndarray(src=out, dst=orig_out)
        out = orig_out
    return out


def clip(x, /, min=None, max=None, out=None, order="K"):  # noqa: A002
    """Elements of `x` limited to [min, max]; the bounds broadcast against `x`, may be arrays or Python
    scalars, and the result has the dtype of `x`."""
    if not isinstance(x, usm_ndarray):
        raise TypeError(f"Expected `x` to be of dpnp.tensor.usm_ndarray type, got {type(x)}")
    if order not in ("K", "C", "F", "A"):
        order = "K"
    if x.dtype.kind in "iu":
        # integer bounds at or beyond the range of the dtype do nothing
        if isinstance(min, int) and min <= iinfo(x.dtype).min:
            min = None
        if isinstance(max, int) and max >= iinfo(x.dtype).max:
            max = None
    if min is None and max is None:
        orig_out = out
        if out is not None:
            if not isinstance(out, usm_ndarray):
                raise TypeError(f"output array must be of usm_ndarray type, got {type(out)}")
            if not out.flags.writable:
                raise ValueError("provided `out` array is read-only")
            if out.shape != x.shape:
                raise ValueError("The shape of input and output arrays are inconsistent. "
                                 f"Expected output shape is {x.shape}, got {out.shape}")
            if x.dtype != out.dtype:
                raise ValueError(f"Output array of type {x.dtype} is needed, got {out.dtype}")
            if ti._array_overlap(x, out):
                if ti._same_logical_tensors(x, out):
                    return out
                out = empty_like(out)
        else:
            out = _empty_like_orderK(x, x.dtype) if order == "K" else empty_like(x, order=order)
        if x.size:
            ti._copy_usm_ndarray_into_usm_ndarray(src=x, dst=out)
        if orig_out is not None and orig_out is not out:
            ti._copy_usm_ndarray_into_usm_ndarray(src=out, dst=orig_out)
            out = orig_out
        return out
    if max is None:
        return _clip_one_bound(x, min, out, order, True)
    if min is None:
        return _clip_one_bound(x, max, out, order, False)

    # both bounds: dpnp/tensor/_clip.py:372-771
    lo_shape, hi_shape = _operand_shape(min), _operand_shape(max)
    if lo_shape is None or hi_shape is None:
        raise TypeError("Shape of arguments can not be inferred. Arguments are expected to be "
                        "lists, tuples, or both")
    try:
        res_shape = _broadcast_shape_impl([x.shape, lo_shape, hi_shape])
    except ValueError:
        raise ValueError(f"operands could not be broadcast together with shapes {x.shape}, {lo_shape}, and {hi_shape}")
    lo_dt, hi_dt = _operand_dtype(min), _operand_dtype(max)
    if lo_dt is None or hi_dt is None:
        raise ValueError("Operands have unsupported data types")
    lo_dt, hi_dt = _resolve_one_strong_two_weak_types(x.dtype, lo_dt, hi_dt)
    res_dt = x.dtype
    if not (_can_cast(lo_dt, res_dt) and _can_cast(hi_dt, res_dt)):
        raise _unsupported(x.dtype, lo_dt, hi_dt)
    orig_out = out
    if out is not None:
        out = _checked_out(out, res_shape, res_dt, (x, min, max))
    if order == "A":
        fs = [a.flags.f_contiguous for a in (x, min, max) if isinstance(a, usm_ndarray)]
        order = "F" if all(fs) else "C"
    lo = _bound_as_array(min, lo_dt, res_dt, order)
    hi = _bound_as_array(max, hi_dt, res_dt, order)
    if out is None:
        out = (_empty_like_triple_orderK(x, lo, hi, res_dt, res_shape) if order == "K"
               else empty(res_shape, dtype=res_dt, order=order))
    if out.size:
        xb = x if x.shape == res_shape else broadcast_to(x, res_shape)
        lo = lo if lo.shape == res_shape else broadcast_to(lo, res_shape)
        hi = hi if hi.shape == res_shape else broadcast_to(hi, res_shape)
        ti._clip(src=xb, min=lo, max=hi, dst=out)
    if orig_out is not None and orig_out is not out:
        ti._copy_usm_ndarray_into_usm_ndarray(src=out, dst=orig_out)
        out = orig_out
    return out
