"""Views, shape queries and joins of the dpnp surface that callers put around the elementwise and reduction
calls (dpnp/dpnp_iface_manipulation.py).  The views move no data; `ravel` of an array that cannot be flattened
in place, `concatenate` / `stack` / `hstack` / `vstack` and `diff` / `trapezoid` (dpnp/dpnp_iface_mathematical.py)
run on the copy / cast and elementwise kernels.  Splitting, repeating and the other functions of that file that
need kernels of their own are outside this library."""
import math

import numpy as np

from . import tensor as dpt
from .dpnp_iface import (
    _wrap,
    ascontiguousarray,
    check_supported_arrays_type,
    get_usm_ndarray,
    is_supported_array_type,
    reshape,
)
from .tensor._manipulation_functions import normalize_axis_index, normalize_axis_tuple

__all__ = ["atleast_1d", "atleast_2d", "atleast_3d", "broadcast_arrays", "broadcast_shapes", "concat", "concatenate",
           "diff", "expand_dims", "flip", "fliplr", "flipud", "hstack", "matrix_transpose", "moveaxis", "ndim",
           "permute_dims", "ravel", "rollaxis", "shape", "size", "squeeze", "stack", "swapaxes", "trapezoid", "vstack"]


def _atleast(arys, fn):
    check_supported_arrays_type(*arys)
    res = []
    for ary in arys:
        r = fn(ary)
        res.append(_wrap(r) if isinstance(r, dpt.usm_ndarray) else r)
    return res[0] if len(res) == 1 else tuple(res)


def atleast_1d(*arys):
    return _atleast(arys, lambda a: a.reshape(1) if a.ndim == 0 else a)


def atleast_2d(*arys):
    return _atleast(arys, lambda a: a.reshape(1, 1) if a.ndim == 0 else (a[None, :] if a.ndim == 1 else a))


def atleast_3d(*arys):
    def fn(a):
        if a.ndim == 0:
            return a.reshape(1, 1, 1)
        if a.ndim == 1:
            return a[None, :, None]
        if a.ndim == 2:
            return a[:, :, None]
        return a

    return _atleast(arys, fn)


def broadcast_arrays(*args, subok=False):
    if subok is not False:
        raise NotImplementedError(f"subok={subok} is currently not supported")
    if len(args) == 0:
        return ()
    return tuple(_wrap(a) for a in dpt.broadcast_arrays(*[get_usm_ndarray(a) for a in args]))


def broadcast_shapes(*args):
    return np.broadcast_shapes(*args)


def expand_dims(a, /, axis):
    return _wrap(dpt.expand_dims(get_usm_ndarray(a), axis=axis))


def squeeze(a, /, axis=None):
    return _wrap(dpt.squeeze(get_usm_ndarray(a), axis=axis))


def flip(m, axis=None):
    return _wrap(dpt.flip(get_usm_ndarray(m), axis=axis))


def fliplr(m):
    check_supported_arrays_type(m)
    if m.ndim < 2:
        raise ValueError(f"Input must be >= 2-d, but got {m.ndim}")
    return m[:, ::-1]


def flipud(m):
    check_supported_arrays_type(m)
    if m.ndim < 1:
        raise ValueError(f"Input must be >= 1-d, but got {m.ndim}")
    return m[::-1, ...]


def matrix_transpose(x, /):
    check_supported_arrays_type(x)
    if x.ndim < 2:
        raise ValueError(f"Input array must be at least 2-dimensional, but it is {x.ndim}")
    return _wrap(dpt.matrix_transpose(get_usm_ndarray(x)))


def moveaxis(a, source, destination):
    return _wrap(dpt.moveaxis(get_usm_ndarray(a), source, destination))


def permute_dims(a, axes=None):
    u = get_usm_ndarray(a)
    return _wrap(u.T if axes is None else dpt.permute_dims(u, axes))


def swapaxes(a, axis1, axis2):
    return _wrap(dpt.swapaxes(get_usm_ndarray(a), axis1=axis1, axis2=axis2))


def rollaxis(x, axis, start=0):
    n = x.ndim
    axis = normalize_axis_index(axis, n)
    if start < 0:
        start += n
    if not 0 <= start < n + 1:
        raise ValueError("'%s' arg requires %d <= %s < %d, but %d was passed in" % ("start", -n, "start", n + 1, start))
    if axis < start:
        start -= 1
    if axis == start:
        return x
    return moveaxis(get_usm_ndarray(x), source=axis, destination=start)


def ravel(a, order="C"):
    """The elements as a 1-D array: a view when the array can be flattened in place, else a copy."""
    if order in "kK":
        raise NotImplementedError("Keyword argument `order` is supported only with values None, 'C', 'F', and 'A', "
                                  f"but got '{order}'")
    if order in "aA":
        u = get_usm_ndarray(a)
        order = "F" if u.flags.fnc else "C"
    result = reshape(a, -1, order=order)
    return result if result.flags.c_contiguous else ascontiguousarray(result)


def ndim(a):
    return a.ndim if is_supported_array_type(a) else np.ndim(a)


def shape(a):
    return a.shape if is_supported_array_type(a) else np.shape(a)


def size(a, axis=None):
    if is_supported_array_type(a):
        if axis is None:
            return a.size
        return math.prod(a.shape[ax] for ax in normalize_axis_tuple(axis, a.ndim))
    return np.size(a, axis)


# -- joining (copies through the cast / copy kernel into slices of the result) ---------------------------
def _check_stack_arrays(arrays):
    if not hasattr(arrays, "__getitem__"):
        raise TypeError('arrays to stack must be passed as a "sequence" type such as list or tuple.')


def _joined(res, out, dtype, casting):
    from .dpnp_iface import copyto

    if dtype is not None:
        return res.astype(dtype, casting=casting, copy=False)
    if out is not None:
        copyto(out, res, casting=casting)
        return out
    return res


def concatenate(arrays, /, *, axis=0, out=None, dtype=None, casting="same_kind"):
    """Join arrays along an existing axis (dpnp/dpnp_iface_manipulation.py, `concatenate`)."""
    if dtype is not None and out is not None:
        raise TypeError("concatenate() only takes `out` or `dtype` as an argument, but both were provided.")
    return _joined(_wrap(dpt.concat([get_usm_ndarray(x) for x in arrays], axis=axis)), out, dtype, casting)


concat = concatenate


def stack(arrays, /, *, axis=0, out=None, dtype=None, casting="same_kind"):
    """Join arrays of one shape along a new axis."""
    _check_stack_arrays(arrays)
    if dtype is not None and out is not None:
        raise TypeError("stack() only takes `out` or `dtype` as an argument, but both were provided.")
    return _joined(_wrap(dpt.stack([get_usm_ndarray(x) for x in arrays], axis=axis)), out, dtype, casting)


def hstack(tup, *, dtype=None, casting="same_kind"):
    _check_stack_arrays(tup)
    arrs = atleast_1d(*tup)
    if not isinstance(arrs, tuple):
        arrs = (arrs,)
    if arrs and arrs[0].ndim == 1:
        return concatenate(arrs, axis=0, dtype=dtype, casting=casting)
    return concatenate(arrs, axis=1, dtype=dtype, casting=casting)


def vstack(tup, *, dtype=None, casting="same_kind"):
    _check_stack_arrays(tup)
    arrs = atleast_2d(*tup)
    if not isinstance(arrs, tuple):
        arrs = (arrs,)
    return concatenate(arrs, axis=0, dtype=dtype, casting=casting)


# -- differences and the trapezoid rule (dpnp/dpnp_iface_mathematical.py, `diff`, `trapezoid`) ----------
def diff(a, n=1, axis=-1, prepend=None, append=None):
    from .dpnp_iface import get_usm_ndarray_or_scalar

    pre = None if prepend is None else get_usm_ndarray_or_scalar(prepend)
    app = None if append is None else get_usm_ndarray_or_scalar(append)
    return _wrap(dpt.diff(get_usm_ndarray(a), axis=axis, n=n, prepend=pre, append=app))


def trapezoid(y, x=None, dx=1.0, axis=-1):
    """Integral along `axis` by the trapezoid rule: sum(d * (y[1:] + y[:-1]) / 2)."""
    check_supported_arrays_type(y)
    nd = y.ndim
    if x is None:
        d = dx
    else:
        check_supported_arrays_type(x)
        if x.ndim == 1:
            d = diff(x)
            shape = [1] * nd
            shape[axis] = d.shape[0]
            d = d.reshape(shape)
        else:
            d = diff(x, axis=axis)
    slice1, slice2 = [slice(None)] * nd, [slice(None)] * nd
    slice1[axis] = slice(1, None)
    slice2[axis] = slice(None, -1)
    return (d * (y[tuple(slice1)] + y[tuple(slice2)]) / 2.0).sum(axis)
