"""mean, var, std over axes.

Results and dtypes as dpnp/tensor/_statistical_functions.py:38-321 (floating input keeps its
dtype, integer and bool input gives float64; N - correction <= 0 gives NaN; complex input is
rejected for var/std).  The variance is computed in two passes over the data (mean, then
sum of squared deviations in one kernel) instead of the reference's five kernels and a
full-size temporary; the arithmetic per element is the same (x - mean, squared, summed).
"""
import math

from . import _tensor_elementwise_impl as tei
from . import _tensor_impl as ti
from . import _tensor_reductions_impl as tri
from ._copy_utils import astype
from ._ctors import empty, empty_like
from ._dtypes import dtype as _as_dtype
from ._dtypes import float64
from ._manipulation_functions import normalize_axis_tuple, permute_dims, reshape
from ._usmarray import usm_ndarray


def _split_axes(x, axis):
    nd = x.ndim
    if axis is None:
        axis = tuple(range(nd))
    if not isinstance(axis, (tuple, list)):
        axis = (axis,)
    axis = normalize_axis_tuple(axis, nd, "axis")
    nelems = 1
    for a in axis:
        nelems *= x.shape[a]
    perm = [i for i in range(nd) if i not in axis] + list(axis)
    return axis, perm, nelems


def _keepdims_view(res, res_shape, red_nd, perm, nd):
    inv = sorted(range(nd), key=lambda d: perm[d])
    return permute_dims(reshape(res, tuple(res_shape) + (1,) * red_nd), inv)


def _sum_as(arr, red_nd, res_shape, res_dt):
    """Sum of the trailing axes of `arr` accumulated in res_dt."""
    res = empty(res_shape, dtype=res_dt)
    if tri._sum_over_axis_dtype_supported(arr.dtype, res_dt):
        tri._sum_over_axis(src=arr, trailing_dims_to_reduce=red_nd, dst=res)
    else:
        tmp = empty(arr.shape, dtype=res_dt)
        ti._copy_usm_ndarray_into_usm_ndarray(src=arr, dst=tmp)
        tri._sum_over_axis(src=tmp, trailing_dims_to_reduce=red_nd, dst=res)
    return res


def mean(x, axis=None, keepdims=False, *, dtype=None):
    """Arithmetic mean over `axis`.

    `dtype` (an extension used by the NumPy-flavoured front end) asks for accumulation in a
    wider floating type than the input's, e.g. float64 for a float32 array.
    """
    if not isinstance(x, usm_ndarray):
        raise TypeError(f"Expected dpnp_amd.tensor.usm_ndarray, got {type(x)}")
    nd = x.ndim
    axis, perm, nelems = _split_axes(x, axis)
    red_nd = len(axis)
    res_dt = x.dtype if x.dtype.kind in "fc" else float64
    if dtype is not None:
        res_dt = _as_dtype(dtype)
    if red_nd == 0:
        return astype(x, res_dt, copy=True)
    arr = permute_dims(x, perm)
    res_shape = arr.shape[: nd - red_nd]
    res = _sum_as(arr, red_nd, res_shape, res_dt)
    if keepdims:
        res = _keepdims_view(res, res_shape, red_nd, perm, nd)
    if res.size:
        tei._divide_by_scalar(src=res, scalar=nelems if nelems else math.nan, dst=res)
    return res


def _var_impl(x, axis, correction, keepdims, dtype=None):
    nd = x.ndim
    axis, perm, nelems = _split_axes(x, axis)
    red_nd = len(axis)
    res_dt = x.dtype if x.dtype.kind == "f" else float64
    if dtype is not None:
        res_dt = _as_dtype(dtype)
    div = max(nelems - correction, 0)
    div = div if div else math.nan
    if red_nd == 0:
        # every element is its own mean: zeros (or NaN when the divisor is not positive)
        res = empty_like(x, dtype=res_dt)
        if res.size:
            ti._full_usm_ndarray(0, res)
            tei._divide_by_scalar(src=res, scalar=div, dst=res)
        return res
    # float64 accumulation: one pass over the input, whatever its layout, instead of the mean's pass plus the
    # deviations' (the reference, dpnp/tensor/_statistical_functions.py:140-230, reads the
    # input twice and a full-size temporary three times)
    # A float32 result of float32 input (a float16 one of float16 input) goes the same way: accumulated in float64
    # (never less accurate than the float32 / float16 accumulation of the reference, whose float16 sums overflow
    # beyond 65504), then rounded; the result arrays are small.
    acc_dt = float64 if (x.dtype in (_as_dtype("f4"), _as_dtype("f2")) and res_dt == x.dtype) else res_dt
    if nelems > 0 and x.size and tri._sqdev_onepass_dtype_supported(x.dtype, acc_dt):
        arr = permute_dims(x, perm)
        res_shape = arr.shape[: nd - red_nd]
        res = empty(res_shape, dtype=acc_dt)
        tri._sqdev_onepass_over_axis(src=arr, trailing_dims_to_reduce=red_nd, dst=res)
        tei._divide_by_scalar(src=res, scalar=div, dst=res)
        if acc_dt != res_dt:
            res = astype(res, res_dt, copy=False)
        if keepdims:
            res = _keepdims_view(res, res_shape, red_nd, perm, nd)
        return res
    buf = x
    if not tri._sumsqdev_over_axis_dtype_supported(x.dtype, res_dt):
        buf = empty_like(x, dtype=res_dt)
        ti._copy_usm_ndarray_into_usm_ndarray(src=x, dst=buf)
    arr = permute_dims(buf, perm)
    res_shape = arr.shape[: nd - red_nd]
    mean_ary = _sum_as(arr, red_nd, res_shape, res_dt)
    res = empty(res_shape, dtype=res_dt)
    if res.size:
        tei._divide_by_scalar(src=mean_ary, scalar=nelems if nelems else math.nan, dst=mean_ary)
        tri._sumsqdev_over_axis(src=arr, mean=mean_ary, trailing_dims_to_reduce=red_nd, dst=res)
        tei._divide_by_scalar(src=res, scalar=div, dst=res)
    if keepdims:
        res = _keepdims_view(res, res_shape, red_nd, perm, nd)
    return res


def _sum_abs_sqdev(x, mean, axis=None, keepdims=False, *, dtype=None):
    """sum(|x - mean|**2) over `axis` in ONE kernel, or None when this call has no fused form.

    The tail of dpnp.var when the caller brings the mean or the data is complex
    (dpnp/dpnp_iface_statistics.py:1843-1860: subtract, square or multiply by the conjugate, real part,
    sum: three or four kernels over full-size temporaries there).  Fused when `mean` broadcasts against
    `x` with extent 1 along every reduced axis (the keepdims=True shape the reference documents, or fewer
    dims), the result type is a real floating one with a kernel for this input type, and a complex mean
    meets complex data; the mean is cast to the result's precision (a small array).
    """
    nd = x.ndim
    axis, perm, nelems = _split_axes(x, axis)
    red_nd = len(axis)
    if red_nd == 0 or nelems == 0 or x.size == 0 or mean.ndim > nd:
        return None
    if x.dtype.kind == "c":
        res_dt = _as_dtype("f4" if x.dtype == _as_dtype("c8") else "f8") if dtype is None else _as_dtype(dtype)
    else:
        if mean.dtype.kind == "c":
            return None
        res_dt = _as_dtype(dtype) if dtype is not None else None
        if res_dt is None:
            return None
    if res_dt.kind != "f" or not tri._sumsqdev_over_axis_dtype_supported(x.dtype, res_dt):
        return None
    mshape = (1,) * (nd - mean.ndim) + tuple(mean.shape)
    for d in range(nd):
        if mshape[d] != 1 and (d in axis or mshape[d] != x.shape[d]):
            return None
    aux_dt = res_dt if x.dtype.kind != "c" else _as_dtype("c8" if res_dt == _as_dtype("f4") else "c16")
    if mean.dtype != aux_dt:
        mean = astype(mean, aux_dt)
    mstrides = (0,) * (nd - mean.ndim) + tuple(mean.strides)
    arr = permute_dims(x, perm)
    res_shape = arr.shape[: nd - red_nd]
    keep = [d for d in range(nd) if d not in axis]
    aux = mean._view(list(res_shape), [0 if mshape[d] == 1 else mstrides[d] for d in keep], mean._offset)
    res = empty(res_shape, dtype=res_dt)
    tri._sumsqdev_over_axis(src=arr, mean=aux, trailing_dims_to_reduce=red_nd, dst=res)
    if keepdims:
        res = _keepdims_view(res, res_shape, red_nd, perm, nd)
    return res


def _check_var_args(x, correction, name):
    if not isinstance(x, usm_ndarray):
        raise TypeError(f"Expected dpnp_amd.tensor.usm_ndarray, got {type(x)}")
    if not isinstance(correction, (int, float)):
        raise TypeError(f"Expected a Python integer or float for `correction`, got{type(x)}")
    if x.dtype.kind == "c":
        raise ValueError(f"`{name}` does not support complex types")


def var(x, axis=None, correction=0.0, keepdims=False, *, dtype=None):
    """Variance over `axis` with divisor N - correction."""
    _check_var_args(x, correction, "var")
    return _var_impl(x, axis, correction, keepdims, dtype)


def std(x, axis=None, correction=0.0, keepdims=False, *, dtype=None):
    """Standard deviation over `axis` with divisor N - correction."""
    _check_var_args(x, correction, "std")
    res = _var_impl(x, axis, correction, keepdims, dtype)
    if res.size:
        tei._sqrt(src=res, dst=res)
    return res
