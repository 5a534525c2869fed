"""NaN-ignoring reductions of the dpnp surface: nansum, nanprod, nanmax, nanmin, nanargmax,
nanargmin, nanmean, nanvar, nanstd.

Arguments, result dtypes, errors and warnings follow dpnp/dpnp_iface_nanfunctions.py:119-284,
427-636,743-1390.  The reference copies the input, overwrites the NaNs (`_replace_nan`, :48-116)
and calls the plain reduction, several passes over the data per call; here floating input goes
through kernels that skip NaNs while reading (dpnp_amd/tensor/_nan_reductions.py), and input of
any other dtype, which holds no NaN, goes straight to the plain function, as in the reference.
"""
import math
import warnings

from . import tensor as dpt
from .dpnp_iface import (
    _search_res_dt,
    _wrap,
    _wrap_reduction_call,
    argmax,
    argmin,
    check_limitations,
    check_supported_arrays_type,
    get_result_array,
    get_usm_ndarray,
    max,  # noqa: A004
    mean,
    min,  # noqa: A004
    prod,
    std,
    sum,  # noqa: A004
    var,
)
from .tensor import _nan_reductions as nr
from .tensor import _tensor_elementwise_impl as tei
from .tensor import _tensor_reductions_impl as tri
from .tensor._manipulation_functions import normalize_axis_tuple

__all__ = ["nanargmax", "nanargmin", "nanmax", "nanmean", "nanmin", "nanprod", "nanstd", "nansum", "nanvar"]


def _inexact(dt):
    return dt.kind in "fc"


def _any_true(u):
    return bool(dpt.any(u)) if u.size else False


def _nanarg(a, axis, out, keepdims, fused, plain):
    u = get_usm_ndarray(a)
    if not _inexact(u.dtype):
        return plain(a, axis=axis, out=out, keepdims=keepdims)
    if u.dtype.kind == "c":
        # complex: replace and search, as the reference does
        fill = -math.inf if fused is nr.nanargmax else math.inf
        nan = dpt.isnan(u)
        if _any_true(dpt.all(nan, axis=axis)):
            raise ValueError("All-NaN slice encountered")
        return plain(_wrap(dpt.where(nan, dpt.asarray(fill, dtype=u.dtype), u)), axis=axis, out=out,
                     keepdims=keepdims)
    if u.size == 0:
        return _wrap_reduction_call(u, out, fused, _search_res_dt(out), axis=axis, keepdims=keepdims)
    if out is not None:
        check_supported_arrays_type(out)
        _search_res_dt(out)  # rejects an `out` that cannot hold indices before anything is computed
    # one pass: the search marks the runs that may be all NaN (their extreme is the infinity NaNs are
    # read as) with negative results; only then is the input read again to tell which they are
    marked = nr.nanargmax_marked if fused is nr.nanargmax else nr.nanargmin_marked
    res = marked(u, axis=axis, keepdims=keepdims)
    doubtful = dpt.less(res, 0)
    if _any_true(doubtful):
        if _any_true(dpt.equal(nr.nancount(u, axis=axis), 0)):
            raise ValueError("All-NaN slice encountered")
        res = dpt.where(doubtful, dpt.subtract(-1, res), res)
    return get_result_array(_wrap(res), out, casting="unsafe")


def nanargmax(a, axis=None, out=None, *, keepdims=False):
    """Indices of the maximum values along an axis, ignoring NaNs; an all-NaN slice raises
    ValueError (dpnp/dpnp_iface_nanfunctions.py:119-200)."""
    return _nanarg(a, axis, out, keepdims, nr.nanargmax, argmax)


def nanargmin(a, axis=None, out=None, *, keepdims=False):
    """Indices of the minimum values along an axis, ignoring NaNs; an all-NaN slice raises
    ValueError (dpnp/dpnp_iface_nanfunctions.py:203-284)."""
    return _nanarg(a, axis, out, keepdims, nr.nanargmin, argmin)


def _nanextremum(a, axis, out, keepdims, fused, plain):
    u = get_usm_ndarray(a)
    if not _inexact(u.dtype):
        return plain(a, axis=axis, out=out, keepdims=keepdims)
    if u.dtype.kind == "c":
        nan = dpt.isnan(u)
        fill = -math.inf if fused is nr.nanmax else math.inf
        res = get_usm_ndarray(plain(_wrap(dpt.where(nan, dpt.asarray(fill, dtype=u.dtype), u)), axis=axis,
                                    keepdims=keepdims))
        bad = dpt.all(nan, axis=axis, keepdims=keepdims)
        if _any_true(bad):
            res = dpt.where(bad, dpt.asarray(math.nan, dtype=res.dtype), res)
            warnings.warn("All-NaN slice encountered", RuntimeWarning, stacklevel=3)
        return get_result_array(res, out, casting="unsafe")
    res = _wrap_reduction_call(u, out, fused, u.dtype, axis=axis, keepdims=keepdims)
    # a result is NaN exactly where the slice held nothing but NaN
    r = get_usm_ndarray(res)
    if r.size and r.dtype.kind == "f" and _any_true(dpt.isnan(r)):
        warnings.warn("All-NaN slice encountered", RuntimeWarning, stacklevel=3)
    return res


def nanmax(a, axis=None, out=None, keepdims=False, initial=None, where=True):
    """Maximum along an axis, ignoring NaNs; NaN (with a RuntimeWarning) for an all-NaN slice
    (dpnp/dpnp_iface_nanfunctions.py:427-518)."""
    check_limitations(initial=initial, where=where)
    return _nanextremum(a, axis, out, keepdims, nr.nanmax, max)


def nanmin(a, axis=None, out=None, keepdims=False, initial=None, where=True):
    """Minimum along an axis, ignoring NaNs; NaN (with a RuntimeWarning) for an all-NaN slice
    (dpnp/dpnp_iface_nanfunctions.py:743-834)."""
    check_limitations(initial=initial, where=where)
    return _nanextremum(a, axis, out, keepdims, nr.nanmin, min)


def _nansumprod(a, axis, dtype, out, keepdims, fused, plain):
    u = get_usm_ndarray(a)
    if not _inexact(u.dtype):
        return plain(a, axis=axis, dtype=dtype, out=out, keepdims=keepdims)
    res_dt = u.dtype if dtype is None else dpt.dtype(dtype)
    return _wrap_reduction_call(u, out, fused, res_dt, axis=axis, dtype=res_dt, keepdims=keepdims)


def nansum(a, axis=None, dtype=None, out=None, keepdims=False, initial=None, where=True):
    """Sum along an axis with NaNs counted as zero (dpnp/dpnp_iface_nanfunctions.py:934-1035)."""
    check_limitations(initial=initial, where=where)
    return _nansumprod(a, axis, dtype, out, keepdims, nr.nansum, sum)


def nanprod(a, axis=None, dtype=None, out=None, keepdims=False, initial=None, where=True):
    """Product along an axis with NaNs counted as one (dpnp/dpnp_iface_nanfunctions.py:837-931)."""
    check_limitations(initial=initial, where=where)
    return _nansumprod(a, axis, dtype, out, keepdims, nr.nanprod, prod)


def _check_inexact_targets(dtype, out):
    if dtype is not None:
        dtype = dpt.dtype(dtype)
        if not _inexact(dtype):
            raise TypeError("If input is inexact, then dtype must be inexact.")
    if out is not None:
        if not _inexact(get_usm_ndarray(out).dtype):
            raise TypeError("If input is inexact, then out must be inexact.")
    return dtype


def nanmean(a, axis=None, dtype=None, out=None, keepdims=False, *, where=True):
    """Mean along an axis over the elements that are not NaN; NaN where there is none
    (dpnp/dpnp_iface_nanfunctions.py:521-635)."""
    check_limitations(where=where)
    u = get_usm_ndarray(a)
    if not _inexact(u.dtype):
        return mean(a, axis=axis, dtype=dtype, out=out, keepdims=keepdims)
    dtype = _check_inexact_targets(dtype, out)
    res_dt = u.dtype if dtype is None else dtype
    usm_out = None if out is None else get_usm_ndarray(out)
    direct = usm_out is not None and usm_out.dtype == res_dt
    # sum and count of the numbers in one pass; 0 / 0 -> NaN for an all-NaN slice
    avg = nr.nanmean(u, axis=axis, dtype=res_dt, keepdims=keepdims, out=usm_out if direct else None)
    return get_result_array(avg, out, casting="unsafe")


def nanvar(a, axis=None, dtype=None, out=None, ddof=0, keepdims=False, *, where=True, mean=None,  # noqa: A002
           correction=None):
    """Variance along an axis over the elements that are not NaN; NaN where their number does
    not exceed ddof (dpnp/dpnp_iface_nanfunctions.py:1188-1391)."""
    check_limitations(where=where)
    if not isinstance(ddof, (int, float)):
        raise TypeError(f"An integer or float is required, but got {type(ddof)}")
    u = get_usm_ndarray(a)
    if not _inexact(u.dtype):
        return var(a, axis=axis, dtype=dtype, out=out, ddof=ddof, keepdims=keepdims, correction=correction)
    dtype = _check_inexact_targets(dtype, out)
    if correction is not None:
        if ddof != 0:
            raise ValueError("ddof and correction can't be provided simultaneously.")
        ddof = correction
    if u.dtype.kind == "c":
        raise NotImplementedError("nanvar of complex input is outside this library's scope")
    res_dt = u.dtype if dtype is None else dtype
    if res_dt.kind == "c":
        raise NotImplementedError("nanvar with a complex dtype is outside this library's scope")
    nd = u.ndim
    axes = tuple(range(nd)) if axis is None else normalize_axis_tuple(
        axis if isinstance(axis, (tuple, list)) else (axis,), nd, "axis")
    kept_shape = tuple(1 if d in axes else u.shape[d] for d in range(nd))
    if mean is not None:
        avg = dpt.astype(get_usm_ndarray(mean), res_dt, copy=False)
        if avg.shape != kept_shape:
            avg = dpt.broadcast_to(avg, kept_shape)
    else:
        avg = nr.nanmean(u, axis=axis, dtype=res_dt, keepdims=True)
    # squared deviations and count of the non-NaN elements travel together: one pass gives
    # sum / (count - ddof), NaN where count <= ddof
    perm = [i for i in range(nd) if i not in axes] + list(axes)
    red_nd = len(axes)
    src = u
    if not tri._sumsqdev_over_axis_dtype_supported(u.dtype, res_dt):
        src = dpt.astype(u, res_dt)
    arr = dpt.permute_dims(src, perm)
    res_shape = arr.shape[: nd - red_nd]
    ssq = dpt.empty(res_shape, dtype=res_dt)
    avg_flat = dpt.reshape(dpt.permute_dims(avg, perm), res_shape)
    if avg_flat.dtype != res_dt:
        avg_flat = dpt.astype(avg_flat, res_dt)
    if ssq.size:
        tri._nanvar_over_axis(src=arr, mean=avg_flat, trailing_dims_to_reduce=red_nd, ddof=ddof, dst=ssq)
    if keepdims:
        inv = sorted(range(nd), key=lambda d: perm[d])
        ssq = dpt.permute_dims(dpt.reshape(ssq, tuple(res_shape) + (1,) * red_nd), inv)
    return get_result_array(ssq, out, casting="unsafe")


def nanstd(a, axis=None, dtype=None, out=None, ddof=0, keepdims=False, *, where=True, mean=None,  # noqa: A002
           correction=None):
    """Standard deviation along an axis over the elements that are not NaN
    (dpnp/dpnp_iface_nanfunctions.py:1038-1185)."""
    check_limitations(where=where)
    if not isinstance(ddof, (int, float)):
        raise TypeError(f"An integer or float is required, but got {type(ddof)}")
    u = get_usm_ndarray(a)
    if not _inexact(u.dtype):
        return std(a, axis=axis, dtype=dtype, out=out, ddof=ddof, keepdims=keepdims, correction=correction)
    res = nanvar(a, axis=axis, dtype=dtype, out=out, ddof=ddof, keepdims=keepdims, where=where, mean=mean,
                 correction=correction)
    r = get_usm_ndarray(res)
    if r.size:
        tei._sqrt(src=r, dst=r)
    return res
