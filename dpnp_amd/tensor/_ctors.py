"""Array constructors needed around the hot path (dpnp/tensor/_ctors.py): empty, zeros,
ones, full, asarray, arange, linspace-free minimal set and their *_like forms."""
import numpy as np

from . import _tensor_impl as ti
from ._copy_utils import _empty_like_orderK, asnumpy, astype, copy, from_numpy
from ._dtypes import dtype as _as_dtype
from ._usmarray import usm_ndarray


def _norm_order(order):
    if order in ("C", "c"):
        return "C"
    if order in ("F", "f"):
        return "F"
    raise ValueError("Unrecognized order keyword value, expecting 'F' or 'C'.")


def _dtype_or_default(dtype, default="f8"):
    return _as_dtype(default if dtype is None else dtype)


def empty(shape, *, dtype=None, order="C", device=None, usm_type="device", sycl_queue=None):
    return usm_ndarray(shape, dtype=_dtype_or_default(dtype), order=_norm_order(order))


def full(shape, fill_value, *, dtype=None, order="C", device=None, usm_type=None, sycl_queue=None):
    if dtype is None:
        if isinstance(fill_value, usm_ndarray):
            dtype = fill_value.dtype
        elif isinstance(fill_value, bool):
            dtype = "?"
        elif isinstance(fill_value, int):
            dtype = "i8"
        elif isinstance(fill_value, complex):
            dtype = "c16"
        elif isinstance(fill_value, (np.generic, np.ndarray)):
            dtype = fill_value.dtype
        else:
            dtype = "f8"
    dt = _as_dtype(dtype)
    if dt.kind in "iu" and isinstance(fill_value, int) and not isinstance(fill_value, bool):
        info = np.iinfo(dt)
        if not (info.min <= fill_value <= info.max):
            raise OverflowError(f"Python integer {fill_value} out of bounds for {dt}")
    r = usm_ndarray(shape, dtype=dt, order=_norm_order(order))
    if r.size:
        if isinstance(fill_value, (usm_ndarray, np.ndarray)):
            r[...] = fill_value
        else:
            ti._full_usm_ndarray(fill_value.item() if isinstance(fill_value, np.generic) else fill_value, r)
    return r


def zeros(shape, *, dtype=None, order="C", device=None, usm_type="device", sycl_queue=None):
    return full(shape, 0, dtype=_dtype_or_default(dtype), order=order)


def ones(shape, *, dtype=None, order="C", device=None, usm_type="device", sycl_queue=None):
    return full(shape, 1, dtype=_dtype_or_default(dtype), order=order)


def _like(x, dtype, order):
    if not isinstance(x, usm_ndarray):
        raise TypeError(f"Expected instance of usm_ndarray, got {type(x)}.")
    dt = x.dtype if dtype is None else _as_dtype(dtype)
    if order in ("K", "k"):
        return _empty_like_orderK(x, dt)
    if order in ("A", "a"):
        order = "F" if x.flags.fnc else "C"
    return usm_ndarray(x.shape, dtype=dt, order=_norm_order(order))


def empty_like(x, /, *, dtype=None, order="K", device=None, usm_type=None, sycl_queue=None):
    return _like(x, dtype, order)


def full_like(x, /, fill_value, *, dtype=None, order="K", device=None, usm_type=None, sycl_queue=None):
    r = _like(x, dtype, order)
    if r.size:
        r[...] = fill_value
    return r


def zeros_like(x, /, *, dtype=None, order="K", device=None, usm_type=None, sycl_queue=None):
    return full_like(x, 0, dtype=dtype, order=order)


def ones_like(x, /, *, dtype=None, order="K", device=None, usm_type=None, sycl_queue=None):
    return full_like(x, 1, dtype=dtype, order=order)


def _host_image(obj):
    """Nested sequences with device arrays replaced by their host copies (for np.asarray)."""
    if isinstance(obj, usm_ndarray):
        return asnumpy(obj)
    if hasattr(obj, "get_array") and isinstance(obj.get_array(), usm_ndarray):
        return asnumpy(obj.get_array())
    if isinstance(obj, (list, tuple)):
        return [_host_image(o) for o in obj]
    return obj


def asarray(obj, /, *, dtype=None, device=None, copy=None, usm_type=None, sycl_queue=None, order="K"):
    """Convert `obj` (device array, NumPy array, nested sequence or scalar) to a device array
    (dpnp/tensor/_ctors.py:560-760)."""
    if copy is not None and not isinstance(copy, bool):
        raise TypeError(f"Argument 'copy' is expected to be a boolean or None, got {type(copy)}")
    if not isinstance(order, str):
        raise TypeError(f"Expected order keyword to be of type str, got {type(order)}")
    if order.upper() not in ("K", "C", "F", "A"):
        raise ValueError("Unrecognized order keyword value, expecting 'K', 'A', 'F', or 'C'.")
    if usm_type is not None:
        if not isinstance(usm_type, str):
            raise TypeError(f"Expected usm_type to be a str or None, got {type(usm_type)}")
        if usm_type not in ("device", "shared", "host"):
            raise ValueError(f"Unrecognized value of usm_type={usm_type}, expected 'device', 'shared', 'host'")
    if dtype is not None:
        dtype = _as_dtype(dtype)
    if isinstance(obj, usm_ndarray):
        tgt = obj.dtype if dtype is None else dtype
        c, f = obj.flags.c_contiguous, obj.flags.f_contiguous
        layout_ok = order in ("K", "k") or (order in ("A", "a") and (c or f)) or \
            (order in ("C", "c") and c) or (order in ("F", "f") and f)
        if tgt == obj.dtype and layout_ok:
            return globals()["copy_"](obj) if copy else obj
        if copy is False:
            raise ValueError("asarray(..., copy=False) needs a copy to satisfy dtype or order")
        return astype(obj, tgt, order=order.upper(), copy=True)
    if hasattr(obj, "get_array") and isinstance(obj.get_array(), usm_ndarray):  # dpnp_amd.ndarray
        return asarray(obj.get_array(), dtype=dtype, copy=copy, order=order)
    if copy is False:
        raise ValueError("Converting a host object to a device array requires a copy")
    if isinstance(obj, (list, tuple)):
        obj = _host_image(obj)
    if isinstance(obj, int) and not isinstance(obj, bool) and dtype is not None:
        a = np.asarray(obj, dtype=dtype)  # raises OverflowError for values outside the dtype
    else:
        a = np.asarray(obj)
    if a.dtype == object:
        if isinstance(obj, int):
            raise OverflowError("Python int too large to convert to a device integer")
        raise TypeError("object arrays are not supported")
    if dtype is None:
        # Python scalars and sequences: NumPy's defaults (int64, float64, complex128)
        dtype = a.dtype
    return from_numpy(a, dtype=dtype, order=order.upper() if order else "K")


copy_ = copy


def arange(start, /, stop=None, step=1, *, dtype=None, device=None, usm_type="device", sycl_queue=None):
    host = np.arange(start, stop, step) if stop is not None else np.arange(start)
    if dtype is None:
        dtype = host.dtype if host.dtype.kind != "i" else "i8"
    return from_numpy(host.astype(_as_dtype(dtype), copy=False))


def linspace(start, stop, /, num, *, dtype=None, device=None, endpoint=True, sycl_queue=None, usm_type="device"):
    host = np.linspace(start, stop, num, endpoint=endpoint)
    return from_numpy(host.astype(_dtype_or_default(dtype), copy=False))
