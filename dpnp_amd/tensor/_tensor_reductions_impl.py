"""Drop-in for the reference's `_tensor_reductions_impl` extension module
(libtensor/source/reductions/{sum,prod,max,min,argmax,argmin}.cpp): `_X_over_axis(src,
trailing_dims_to_reduce, dst, sycl_queue, depends)` and `_X_over_axis_dtype_supported`.
"""
from .. import _lib
from ._dtypes import dtype_id
from ._tensor_impl import _events, _stream

lib = _lib.lib


def _make_reduction(name, op_id):
    # _X_over_axis(src, trailing_dims_to_reduce, dst, sycl_queue=None, depends=()) -> (event, event)
    fn = _lib.ext.make_reduction(op_id, f"_{name}_over_axis")

    def supported(arg_dtype, out_dtype, dst_usm_type=None, sycl_queue=None):
        return bool(lib.dpx_reduce_dtype_supported(op_id, dtype_id(arg_dtype), dtype_id(out_dtype)))

    return fn, supported


def _make_search(name, op_id):
    return _lib.ext.make_search(op_id, f"_{name}_over_axis")


_sum_over_axis, _sum_over_axis_dtype_supported = _make_reduction("sum", _lib.REDUCE_ID["sum"])
_prod_over_axis, _prod_over_axis_dtype_supported = _make_reduction("prod", _lib.REDUCE_ID["prod"])
_max_over_axis, _max_over_axis_dtype_supported = _make_reduction("max", _lib.REDUCE_ID["max"])
_min_over_axis, _min_over_axis_dtype_supported = _make_reduction("min", _lib.REDUCE_ID["min"])
_logsumexp_over_axis, _logsumexp_over_axis_dtype_supported = _make_reduction("logsumexp", _lib.REDUCE_ID["logsumexp"])
_hypot_over_axis, _hypot_over_axis_dtype_supported = _make_reduction("hypot", _lib.REDUCE_ID["hypot"])
# all / any of any dtype (tri._all, tri._any) and the one-pass count of non-zero elements
_any, _any_dtype_supported = _make_reduction("any", _lib.REDUCE_ID["any"])
_all, _all_dtype_supported = _make_reduction("all", _lib.REDUCE_ID["all"])
_count_nonzero_over_axis, _count_nonzero_over_axis_dtype_supported = _make_reduction(
    "count_nonzero", _lib.REDUCE_ID["count_nonzero"])
_argmax_over_axis = _make_search("argmax", _lib.SEARCH_ID["argmax"])
_argmin_over_axis = _make_search("argmin", _lib.SEARCH_ID["argmin"])


# NaN-ignoring forms (no counterpart among the reference's extension functions: dpnp builds
# nansum, nanmax, ... from a masked copy and the plain reductions,
# dpnp/dpnp_iface_nanfunctions.py:48-116)
_nansum_over_axis, _nansum_over_axis_dtype_supported = _make_reduction("nansum", _lib.REDUCE_ID["nansum"])
_nanprod_over_axis, _nanprod_over_axis_dtype_supported = _make_reduction("nanprod", _lib.REDUCE_ID["nanprod"])
_nanmax_over_axis, _nanmax_over_axis_dtype_supported = _make_reduction("nanmax", _lib.REDUCE_ID["nanmax"])
_nanmin_over_axis, _nanmin_over_axis_dtype_supported = _make_reduction("nanmin", _lib.REDUCE_ID["nanmin"])
_nancount_over_axis, _nancount_over_axis_dtype_supported = _make_reduction("nancount", _lib.REDUCE_ID["nancount"])
_nanmean_over_axis, _nanmean_over_axis_dtype_supported = _make_reduction("nanmean", _lib.REDUCE_ID["nanmean"])
_nanargmax_over_axis = _make_search("nanargmax", _lib.SEARCH_ID["nanargmax"])
_nanargmin_over_axis = _make_search("nanargmin", _lib.SEARCH_ID["nanargmin"])
# the same, with results of runs whose extreme is the infinity NaNs are read as stored as -1 - index
_nanargmax_marked_over_axis = _make_search("nanargmax_marked", _lib.SEARCH_ID["nanargmax_marked"])
_nanargmin_marked_over_axis = _make_search("nanargmin_marked", _lib.SEARCH_ID["nanargmin_marked"])


def _sumsqdev_over_axis(src, mean, trailing_dims_to_reduce, dst, sycl_queue=None, depends=(), nan=False):
    """dst[i] = sum_j (src[i, j] - mean[i])**2: the second pass of var in one kernel
    (the reference runs subtract, square and sum kernels over a full-size temporary,
    dpnp/tensor/_statistical_functions.py:38-163)."""
    vs, vm, vd = src._as_view(), mean._as_view(), dst._as_view()
    op = _lib.REDUCE_ID["nansumsqdev" if nan else "sumsqdev"]
    _lib.check(lib.dpx_reduce(op, vs, int(trailing_dims_to_reduce), vd, vm, _stream(sycl_queue)))
    return _events(sycl_queue)


def _sqdev_onepass_over_axis(src, trailing_dims_to_reduce, dst, sycl_queue=None, depends=()):
    """dst[i] = sum_j (src[i, j] - mean_i)**2 with mean_i the mean of row i, in ONE pass over src (float32 or
    float64 in, float64 out): count, mean and squared deviations travel together and are merged pairwise.  Fast
    for a contiguous reduced run only (see DPX_R_SQDEV_ONEPASS)."""
    vs, vd = src._as_view(), dst._as_view()
    _lib.check(lib.dpx_reduce(_lib.REDUCE_ID["sqdev_onepass"], vs, int(trailing_dims_to_reduce), vd, None,
                              _stream(sycl_queue)))
    return _events(sycl_queue)


def _sqdev_onepass_dtype_supported(arg_dtype, out_dtype):
    return bool(lib.dpx_reduce_dtype_supported(_lib.REDUCE_ID["sqdev_onepass"], dtype_id(arg_dtype),
                                               dtype_id(out_dtype)))


def _sumsqdev_over_axis_dtype_supported(arg_dtype, out_dtype, dst_usm_type=None, sycl_queue=None):
    return bool(lib.dpx_reduce_dtype_supported(_lib.REDUCE_ID["sumsqdev"], dtype_id(arg_dtype),
                                               dtype_id(out_dtype)))


def _nanvar_over_axis(src, mean, trailing_dims_to_reduce, ddof, dst, sycl_queue=None, depends=()):
    """dst[i] = sum_j (src[i, j] - mean[i])**2 / (count_i - ddof) over the elements that are not NaN, NaN where
    count_i <= ddof: the second pass of nanvar in one kernel (dpnp/dpnp_iface_nanfunctions.py:1318-1390 runs
    count, subtract, square, sum and divide as separate calls)."""
    vs, vm, vd = src._as_view(), mean._as_view(), dst._as_view()
    _lib.check(lib.dpx_nan_variance(vs, int(trailing_dims_to_reduce), vm, float(ddof), vd, _stream(sycl_queue)))
    return _events(sycl_queue)
