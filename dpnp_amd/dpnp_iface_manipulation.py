"""Views and shape queries of the dpnp surface that callers put around the elementwise and reduction
calls (dpnp/dpnp_iface_manipulation.py): nothing here moves data except `ravel` of an array that
cannot be flattened in place.  Joining, splitting, repeating and the other functions of that file
that need kernels of their own are outside this library."""
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

__all__ = ["atleast_1d", "atleast_2d", "atleast_3d", "broadcast_arrays", "broadcast_shapes", "expand_dims", "flip",
           "fliplr", "flipud", "matrix_transpose", "moveaxis", "ndim", "permute_dims", "ravel", "rollaxis", "shape",
           "size", "squeeze", "swapaxes"]


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
