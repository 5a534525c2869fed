"""Allocation in the layout of an existing array (order="K"), cast-copies, host transfers.
Behaviour of dpnp/tensor/_copy_utils.py:811-911 (order-K allocators), astype/copy, and the
host<->device copies of dpnp.tensor.asnumpy / from_numpy."""
import numpy as np

from . import _device
from . import _tensor_impl as ti
from ._dtypes import dtype as _as_dtype
from ._manipulation_functions import broadcast_to, permute_dims
from ._usmarray import usm_ndarray


def _empty(shape, dtype, order="C"):
    return usm_ndarray._new_contiguous(tuple(shape), _as_dtype(dtype), order)


def _like_strides(shape, stride_lists, dt):
    """New array whose dims are nested in the order of the given arrays' |strides|
    (first list is the primary key); dims that all given arrays walk backwards stay reversed."""
    nd = len(shape)
    perm = sorted(range(nd),
                  key=lambda d: tuple(abs(st[d]) if shape[d] > 1 else 0 for st in stride_lists),
                  reverse=True)
    inv = sorted(range(nd), key=lambda i: perm[i])
    r = _empty(tuple(shape[i] for i in perm), dt, "C")
    flips = [all(st[i] < 0 for st in stride_lists) for i in perm]
    if any(flips):
        r = r[tuple(slice(None, None, -1) if f else slice(None) for f in flips)]
    return permute_dims(r, inv)


def _empty_like_orderK(x, dt, usm_type=None, dev=None):
    """Same shape as `x`, dtype `dt`, strides ordered like x's (C stays C, F stays F)."""
    if not isinstance(x, usm_ndarray):
        raise TypeError(f"Expected usm_ndarray, got {type(x)}")
    fl = x.flags
    if fl.c_contiguous or x.size <= 1:
        return _empty(x.shape, dt, "C")
    if fl.f_contiguous:
        return _empty(x.shape, dt, "F")
    return _like_strides(x.shape, [x.strides], dt)


def _empty_like_pair_orderK(x1, x2, dt, res_shape, usm_type=None, dev=None):
    for x in (x1, x2):
        if not isinstance(x, usm_ndarray):
            raise TypeError(f"Expected usm_ndarray, got {type(x)}")
    nd1, nd2 = x1.ndim, x2.ndim
    if nd1 > nd2 and x1.shape == res_shape:
        return _empty_like_orderK(x1, dt)
    if nd1 < nd2 and x2.shape == res_shape:
        return _empty_like_orderK(x2, dt)
    f1, f2 = x1.flags, x2.flags
    if f1.c_contiguous or f2.c_contiguous:
        return _empty(res_shape, dt, "C")
    if f1.f_contiguous and f2.f_contiguous:
        return _empty(res_shape, dt, "F")
    nd = max(nd1, nd2)
    if nd1 != nd2 or x1.shape != tuple(res_shape) or x2.shape != tuple(res_shape):
        x1 = broadcast_to(x1, res_shape)
        x2 = broadcast_to(x2, res_shape)
    return _like_strides(tuple(res_shape), [x1.strides, x2.strides], dt) if nd else _empty(res_shape, dt)


def _empty_like_triple_orderK(x1, x2, x3, dt, res_shape):
    """Layout of a result of three operands (dpnp/tensor/_copy_utils.py:914-987): two operands of
    the full shape decide when the third has fewer dims; else C if any operand is C-contiguous,
    F if all are F-contiguous, else dims nested by the operands' strides."""
    res_shape = tuple(res_shape)
    nd = len(res_shape)
    if x1.shape == res_shape and x2.shape == res_shape and nd > x3.ndim:
        return _empty_like_pair_orderK(x1, x2, dt, res_shape)
    if x2.shape == res_shape and x3.shape == res_shape and nd > x1.ndim:
        return _empty_like_pair_orderK(x2, x3, dt, res_shape)
    if x1.shape == res_shape and x3.shape == res_shape and nd > x2.ndim:
        return _empty_like_pair_orderK(x1, x3, dt, res_shape)
    arrs = [x1, x2, x3]
    if any(a.flags.c_contiguous for a in arrs):
        return _empty(res_shape, dt, "C")
    if all(a.flags.f_contiguous for a in arrs):
        return _empty(res_shape, dt, "F")
    b = [broadcast_to(a, res_shape) for a in arrs]
    return _like_strides(res_shape, [a.strides for a in b], dt) if nd else _empty(res_shape, dt)


def _copy_into(src, dst):
    ti._copy_usm_ndarray_into_usm_ndarray(src=src, dst=dst)


def copy(x, /, *, order="K"):
    if not isinstance(x, usm_ndarray):
        raise TypeError(f"Expected instance of `usm_ndarray`, got {type(x)}.")
    if order not in ("C", "F", "A", "K"):
        raise ValueError("Unrecognized value of the order keyword. Recognized values are 'A', 'C', 'F', or 'K'")
    if order == "A":
        order = "F" if x.flags.fnc else "C"
    r = _empty_like_orderK(x, x.dtype) if order == "K" else _empty(x.shape, x.dtype, order)
    if x.size:
        _copy_into(x, r)
    return r


def astype(x, newdtype, /, *, order="K", casting="unsafe", copy=True, device=None):
    if not isinstance(x, usm_ndarray):
        raise TypeError(f"Expected instance of `usm_ndarray`, got {type(x)}.")
    if order not in ("C", "F", "A", "K"):
        raise ValueError("Unrecognized value of the order keyword. Recognized values are 'A', 'C', 'F', or 'K'")
    tgt = _as_dtype(newdtype)
    if not np.can_cast(x.dtype, tgt, casting=casting):
        raise TypeError(f"Can not cast from {x.dtype} to {tgt} according to rule {casting}.")
    c, f = x.flags.c_contiguous, x.flags.f_contiguous
    layout_ok = order == "K" or (order == "C" and c) or (order == "F" and f) or (order == "A" and (c or f))
    if tgt == x.dtype and layout_ok and not copy:
        return x
    if order == "A":
        order = "F" if x.flags.fnc else "C"
    r = _empty_like_orderK(x, tgt) if order == "K" else _empty(x.shape, tgt, order)
    if x.size:
        _copy_into(x, r)
    return r


def from_numpy(np_ary, /, *, dtype=None, order="K"):
    """New device array with the contents of a NumPy array."""
    a = np.asarray(np_ary)
    src_dt = _as_dtype(a.dtype)
    keep_nesting = order == "K" and a.ndim > 1 and a.size > 1 and not (a.flags.c_contiguous or a.flags.f_contiguous)
    if order == "K":
        order = "F" if (a.flags.f_contiguous and not a.flags.c_contiguous) else "C"
    elif order == "A":
        order = "F" if (a.flags.f_contiguous and not a.flags.c_contiguous) else "C"
    if keep_nesting:
        # order "K" of an array that is neither C- nor F-contiguous: keep the nesting of its axes
        # (a permuted contiguous array gets the same strides: dpnp/tensor/_copy_utils.py:837-856)
        perm = sorted(range(a.ndim), key=lambda d: (-abs(a.strides[d]) if a.shape[d] > 1 else 0, d))
        inv = sorted(range(a.ndim), key=lambda i: perm[i])
        r = from_numpy(np.ascontiguousarray(a.transpose(perm)), dtype=dtype, order="C")
        return permute_dims(r, inv)
    host = np.asarray(a, dtype=src_dt, order=order)
    if not (host.flags.c_contiguous or host.flags.f_contiguous):
        host = np.ascontiguousarray(host)
        order = "C"
    flat = host.reshape(-1, order=order) if host.ndim else host.reshape(1)
    buf = _device.to_device_bytes(np.ascontiguousarray(flat).view(np.uint8).reshape(-1))
    r = usm_ndarray(a.shape, dtype=src_dt, buffer=buf, order=order)
    if dtype is not None and _as_dtype(dtype) != src_dt:
        r = astype(r, dtype)
    return r


def asnumpy(x):
    """NumPy copy of a device array (synchronises with the stream)."""
    if not isinstance(x, usm_ndarray):
        raise TypeError(f"Expected instance of `usm_ndarray`, got {type(x)}.")
    if x.size == 0:
        return np.empty(x.shape, dtype=x.dtype)
    src = x
    order = "C"
    if x.flags.f_contiguous and not x.flags.c_contiguous:
        order = "F"
    elif not x.flags.c_contiguous:
        src = copy(x, order="C")
    host = _device.to_host_bytes(src._buf, src._offset * src.itemsize, src.size * src.itemsize)
    flat = host.view(x.dtype)
    return flat.reshape(x.shape, order=order).copy(order="K") if order == "F" else flat.reshape(x.shape)


to_numpy = asnumpy


def _assign(dst_view, value):
    """dst_view[...] = value with broadcasting and casting (usm_ndarray.__setitem__)."""
    if isinstance(value, usm_ndarray):
        src = value
    elif isinstance(value, (bool, int, float, complex, np.generic)) and dst_view.size:
        ti._full_usm_ndarray(value.item() if isinstance(value, np.generic) else value, dst_view)
        return
    else:
        src = from_numpy(np.asarray(value))
    if src.ndim > dst_view.ndim and all(s == 1 for s in src.shape[: src.ndim - dst_view.ndim]):
        src = src._view(src.shape[src.ndim - dst_view.ndim:], src.strides[src.ndim - dst_view.ndim:], src._offset)
    if src.shape != dst_view.shape:
        try:
            src = broadcast_to(src, dst_view.shape)
        except ValueError:
            raise ValueError(f"Shape of the value {src.shape} can not be broadcast to {dst_view.shape}")
    if dst_view.size == 0:
        return
    if ti._array_overlap(src, dst_view) and not ti._same_logical_tensors(src, dst_view):
        src = copy(src)
        if src.shape != dst_view.shape:
            src = broadcast_to(src, dst_view.shape)
    elif ti._same_logical_tensors(src, dst_view):
        return
    _copy_into(src, dst_view)
