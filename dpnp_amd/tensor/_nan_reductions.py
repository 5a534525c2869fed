"""NaN-ignoring reductions of floating arrays in one pass over the data.

The reference has no tensor-level functions for these: dpnp.nansum, nanmax, nanmean, ... copy
the input, overwrite its NaNs and call the plain reduction
(dpnp/dpnp_iface_nanfunctions.py:48-116).  The kernels behind this module skip NaNs as they
read, so nothing is copied.  Inputs must be of a floating (or, for sum/prod/count, complex)
dtype; other dtypes hold no NaN and belong to the plain functions.
"""
from . import _tensor_reductions_impl as tri
from ._reduction import _comparison_over_axis, _reduction_over_axis, _search_over_axis


def _same_dtype(inp_dt, _queue=None):
    return inp_dt


def nansum(x, /, *, axis=None, dtype=None, keepdims=False, out=None):
    """Sum over `axis` with NaN counted as zero."""
    return _reduction_over_axis(x, axis, dtype, keepdims, out, tri._nansum_over_axis,
                                tri._nansum_over_axis_dtype_supported, _same_dtype)


def nanprod(x, /, *, axis=None, dtype=None, keepdims=False, out=None):
    """Product over `axis` with NaN counted as one."""
    return _reduction_over_axis(x, axis, dtype, keepdims, out, tri._nanprod_over_axis,
                                tri._nanprod_over_axis_dtype_supported, _same_dtype)


def nanmax(x, /, *, axis=None, keepdims=False, out=None):
    """Maximum over `axis` of the elements that are not NaN; NaN where there is none."""
    return _comparison_over_axis(x, axis, keepdims, out, tri._nanmax_over_axis)


def nanmin(x, /, *, axis=None, keepdims=False, out=None):
    """Minimum over `axis` of the elements that are not NaN; NaN where there is none."""
    return _comparison_over_axis(x, axis, keepdims, out, tri._nanmin_over_axis)


def nancount(x, /, *, axis=None, keepdims=False, out=None):
    """Number of elements over `axis` that are not NaN (int64)."""
    return _reduction_over_axis(x, axis, "i8", keepdims, out, tri._nancount_over_axis,
                                tri._nancount_over_axis_dtype_supported, _same_dtype)


def nanmean(x, /, *, axis=None, dtype=None, keepdims=False, out=None):
    """Mean over `axis` of the elements that are not NaN, NaN where there is none: sum and count in
    one pass, divided in the accumulation type."""
    return _reduction_over_axis(x, axis, dtype, keepdims, out, tri._nanmean_over_axis,
                                tri._nanmean_over_axis_dtype_supported, _same_dtype)


def nanargmax(x, /, *, axis=None, keepdims=False, out=None):
    """Index of the maximum along `axis` with NaN read as -inf (first occurrence)."""
    return _search_over_axis(x, axis, keepdims, out, tri._nanargmax_over_axis)


def nanargmin(x, /, *, axis=None, keepdims=False, out=None):
    """Index of the minimum along `axis` with NaN read as +inf (first occurrence)."""
    return _search_over_axis(x, axis, keepdims, out, tri._nanargmin_over_axis)


def nanargmax_marked(x, /, *, axis=None, keepdims=False):
    """nanargmax in which a run that is all NaN, or whose maximum is -inf, reports -1 - index: a
    caller that must raise on all-NaN runs looks at the input again only when a result is negative."""
    return _search_over_axis(x, axis, keepdims, None, tri._nanargmax_marked_over_axis)


def nanargmin_marked(x, /, *, axis=None, keepdims=False):
    """nanargmin in which a run that is all NaN, or whose minimum is +inf, reports -1 - index."""
    return _search_over_axis(x, axis, keepdims, None, tri._nanargmin_marked_over_axis)
