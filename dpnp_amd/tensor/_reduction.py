"""sum, prod, max, min, argmax, argmin over axes.

Host logic of dpnp/tensor/_reduction.py:43-138,141-296,299-395 restated around one
skeleton: move the reduced axes last (a view), allocate or validate `out`, run the
kernel on (array, number of trailing axes, destination), undo the permutation for
keepdims.  Result dtypes: sum/prod use the default accumulation dtype unless `dtype`
is given; max/min keep the dtype; argmax/argmin give int64.
"""
import builtins

from . import _tensor_impl as ti
from . import _tensor_reductions_impl as tri
from ._ctors import empty, empty_like
from ._dtypes import dtype as _as_dtype
from ._manipulation_functions import normalize_axis_tuple, permute_dims, reshape, squeeze
from ._type_utils import _default_accumulation_dtype, _default_accumulation_dtype_fp_types
from ._usmarray import usm_ndarray


def _move_reduced_axes_last(x, axis, int_only=False):
    nd = x.ndim
    if axis is None:
        return x, tuple(range(nd)), list(range(nd))
    if int_only:
        if not isinstance(axis, int):
            raise TypeError("'axis' argument expected to have type 'int' or be `None`, "
                            f"got type {type(axis)}")
        axis = (axis,)
    axis = normalize_axis_tuple(axis, nd, "axis")
    perm = [i for i in range(nd) if i not in axis] + list(axis)
    if perm == list(range(nd)):
        return x, axis, perm  # the reduced axes are the last ones already: x and its cached descriptor serve
    # the permuted view of an array is kept with it: the next call with the same axes finds the view and the
    # descriptor it has built
    cache = x.__dict__.get("_perm_views")
    if cache is None:
        cache = x.__dict__["_perm_views"] = {}
    key = tuple(perm)
    arr = cache.get(key)
    if arr is None:
        arr = x._view([x._shape[a] for a in perm], [x._strides[a] for a in perm], x._offset)
        if arr._base is x:
            # an internal view, never handed out: it holds the allocation itself, not the array that keeps it
            # (x -> cache -> view -> x would be a cycle, and the memory of a dropped array would wait for the
            # cycle collector instead of being freed with the last reference)
            arr._base = None
        cache[key] = arr
    return arr, axis, perm


def _prepare_out(x, out, axis, keepdims, res_shape, res_dt, guard_overlap):
    """Validate a user `out`; returns (array the kernel writes, array the user gets back)."""
    if out is None:
        r = usm_ndarray._new_contiguous(tuple(res_shape), res_dt)
        return r, r
    if not isinstance(out, usm_ndarray):
        raise TypeError(f"output array must be of usm_ndarray type, got {type(out)}")
    if not out.flags.writable:
        raise ValueError("provided `out` array is read-only")
    final_shape = res_shape if not keepdims else tuple(
        x.shape[i] if i not in axis else 1 for i in range(x.ndim))
    if out.shape != final_shape:
        raise ValueError("The shape of input and output arrays are inconsistent. "
                         f"Expected output shape is {final_shape}, got {out.shape}")
    if res_dt != out.dtype:
        raise ValueError(f"Output array of type {res_dt} is needed, got {out.dtype}")
    if keepdims:
        out = squeeze(out, axis=axis)
    user = out
    if guard_overlap and ti._array_overlap(x, out):
        out = empty_like(out)
    return out, user


def _finish(out, user, keepdims, res_shape, red_nd, perm, nd):
    if user is not out:
        ti._copy_usm_ndarray_into_usm_ndarray(src=out, dst=user)
        out = user
    if keepdims:
        inv = sorted(range(nd), key=lambda d: perm[d])
        out = permute_dims(reshape(out, res_shape + (1,) * red_nd), inv)
    return out


def _reduction_over_axis(x, axis, dtype, keepdims, out, _reduction_fn, _dtype_supported,
                         _default_reduction_type_fn):
    if not isinstance(x, usm_ndarray):
        raise TypeError(f"Expected dpnp_amd.tensor.usm_ndarray, got {type(x)}")
    nd = x.ndim
    arr, axis, perm = _move_reduced_axes_last(x, axis)
    red_nd = len(axis)
    res_shape = arr.shape[: nd - red_nd]
    inp_dt = x.dtype
    res_dt = _default_reduction_type_fn(inp_dt, None) if dtype is None else _as_dtype(dtype)
    direct = _dtype_supported(inp_dt, res_dt, "device", None)
    if dtype is None and not direct and not _dtype_supported(res_dt, res_dt, "device", None):
        raise RuntimeError("Automatically determined reduction data type does not have direct implementation")
    out, user = _prepare_out(x, out, axis, keepdims, res_shape, res_dt, guard_overlap=direct)
    if red_nd == 0:
        ti._copy_usm_ndarray_into_usm_ndarray(src=arr, dst=out)
        return _finish(out, user, False, res_shape, red_nd, perm, nd)
    if direct:
        _reduction_fn(src=arr, trailing_dims_to_reduce=red_nd, dst=out)
    elif _dtype_supported(res_dt, res_dt, "device", None):
        # no (input, result) kernel: cast the input to the result type first
        tmp = empty(arr.shape, dtype=res_dt)
        ti._copy_usm_ndarray_into_usm_ndarray(src=arr, dst=tmp)
        _reduction_fn(src=tmp, trailing_dims_to_reduce=red_nd, dst=out)
    else:
        # reduce in the default type of the input, cast the (small) result
        buf_dt = _default_reduction_type_fn(inp_dt, None)
        tmp = empty(arr.shape, dtype=buf_dt)
        ti._copy_usm_ndarray_into_usm_ndarray(src=arr, dst=tmp)
        tmp_res = empty(res_shape, dtype=buf_dt)
        _reduction_fn(src=tmp, trailing_dims_to_reduce=red_nd, dst=tmp_res)
        ti._copy_usm_ndarray_into_usm_ndarray(src=tmp_res, dst=out)
    return _finish(out, user, keepdims, res_shape, red_nd, perm, nd)


def _comparison_over_axis(x, axis, keepdims, out, _reduction_fn):
    if not isinstance(x, usm_ndarray):
        raise TypeError(f"Expected dpnp_amd.tensor.usm_ndarray, got {type(x)}")
    nd = x.ndim
    arr, axis, perm = _move_reduced_axes_last(x, axis)
    red_nd = len(axis)
    if builtins.any(arr.shape[i] == 0 for i in range(nd - red_nd, nd)):
        raise ValueError("reduction cannot be performed over zero-size axes")
    res_shape = arr.shape[: nd - red_nd]
    out, user = _prepare_out(x, out, axis, keepdims, res_shape, x.dtype, guard_overlap=True)
    if red_nd == 0:
        ti._copy_usm_ndarray_into_usm_ndarray(src=arr, dst=out)
        return _finish(out, user, False, res_shape, red_nd, perm, nd)
    _reduction_fn(src=arr, trailing_dims_to_reduce=red_nd, dst=out)
    return _finish(out, user, keepdims, res_shape, red_nd, perm, nd)


def _search_over_axis(x, axis, keepdims, out, _reduction_fn):
    if not isinstance(x, usm_ndarray):
        raise TypeError(f"Expected dpnp_amd.tensor.usm_ndarray, got {type(x)}")
    nd = x.ndim
    arr, axis, perm = _move_reduced_axes_last(x, axis, int_only=True)
    red_nd = len(axis)
    if builtins.any(arr.shape[i] == 0 for i in range(nd - red_nd, nd)):
        raise ValueError("reduction cannot be performed over zero-size axes")
    res_shape = arr.shape[: nd - red_nd]
    res_dt = _as_dtype(ti.default_device_index_type())
    out, user = _prepare_out(x, out, axis, keepdims, res_shape, res_dt, guard_overlap=red_nd > 0)
    if red_nd == 0:
        ti._full_usm_ndarray(fill_value=0, dst=out)
        return out
    _reduction_fn(src=arr, trailing_dims_to_reduce=red_nd, dst=out)
    return _finish(out, user, keepdims, res_shape, red_nd, perm, nd)


def _fill_ext_type_tables():
    """Default result dtype of each reduction per input dtype, for the extension module's plain-call path
    (reduce_call / search_call): only pairs with a direct kernel are entered."""
    from .. import _lib
    from ._dtypes import ALL_DTYPES, bool as _bool, dtype_id, int64

    ext, lib = _lib.ext, _lib.lib
    rules = {"sum": _default_accumulation_dtype, "prod": _default_accumulation_dtype,
             "max": lambda dt, q: dt, "min": lambda dt, q: dt,
             "logsumexp": _default_accumulation_dtype_fp_types, "hypot": _default_accumulation_dtype_fp_types,
             "any": lambda dt, q: _bool, "all": lambda dt, q: _bool, "count_nonzero": lambda dt, q: int64}
    for name, rule in rules.items():
        op = _lib.REDUCE_ID[name]
        for dt in ALL_DTYPES:
            if name in ("logsumexp", "hypot") and dt.kind == "c":
                continue
            res = rule(dt, None)
            ok = res is not None and lib.dpx_reduce_dtype_supported(op, dtype_id(dt), dtype_id(res))
            ext.set_reduce_type(op, dtype_id(dt), dtype_id(res) if ok else -1)
    for name in ("argmax", "argmin"):
        op = _lib.SEARCH_ID[name]
        for dt in ALL_DTYPES:
            ok = lib.dpx_search_dtype_supported(op, dtype_id(dt), dtype_id(int64))
            ext.set_search_type(op, dtype_id(dt), dtype_id(int64) if ok else -1)
    return ext.reduce_call, ext.search_call, _lib.REDUCE_ID, _lib.SEARCH_ID


_ext_reduce, _ext_search, _RID, _SID = _fill_ext_type_tables()


def _plain(op, x, axis, dtype, keepdims, out, search=False):
    """The call for the plain case (default result dtype, no keepdims), done on the descriptors by the extension
    module; NotImplemented for anything else."""
    if dtype is not None or keepdims is not False:
        return NotImplemented
    return _ext_search(op, x, axis, out) if search else _ext_reduce(op, x, axis, out)


def sum(x, /, *, axis=None, dtype=None, keepdims=False, out=None):  # noqa: A001
    """Sum of the elements of `x` over `axis` (all axes when None)."""
    r = _plain(_RID["sum"], x, axis, dtype, keepdims, out)
    if r is not NotImplemented:
        return r
    return _reduction_over_axis(x, axis, dtype, keepdims, out, tri._sum_over_axis,
                                tri._sum_over_axis_dtype_supported, _default_accumulation_dtype)


def prod(x, /, *, axis=None, dtype=None, keepdims=False, out=None):
    """Product of the elements of `x` over `axis`."""
    r = _plain(_RID["prod"], x, axis, dtype, keepdims, out)
    if r is not NotImplemented:
        return r
    return _reduction_over_axis(x, axis, dtype, keepdims, out, tri._prod_over_axis,
                                tri._prod_over_axis_dtype_supported, _default_accumulation_dtype)


def max(x, /, *, axis=None, keepdims=False, out=None):  # noqa: A001
    """Maximum over `axis`; NaN propagates."""
    r = _plain(_RID["max"], x, axis, None, keepdims, out)
    if r is not NotImplemented:
        return r
    return _comparison_over_axis(x, axis, keepdims, out, tri._max_over_axis)


def min(x, /, *, axis=None, keepdims=False, out=None):  # noqa: A001
    """Minimum over `axis`; NaN propagates."""
    r = _plain(_RID["min"], x, axis, None, keepdims, out)
    if r is not NotImplemented:
        return r
    return _comparison_over_axis(x, axis, keepdims, out, tri._min_over_axis)


def argmax(x, /, *, axis=None, keepdims=False, out=None):
    """Index of the maximum along `axis` (flat C-order index when None); first occurrence,
    NaN counts as the maximum."""
    r = _plain(_SID["argmax"], x, axis, None, keepdims, out, search=True)
    if r is not NotImplemented:
        return r
    return _search_over_axis(x, axis, keepdims, out, tri._argmax_over_axis)


def argmin(x, /, *, axis=None, keepdims=False, out=None):
    """Index of the minimum along `axis`; first occurrence, NaN counts as the minimum."""
    r = _plain(_SID["argmin"], x, axis, None, keepdims, out, search=True)
    if r is not NotImplemented:
        return r
    return _search_over_axis(x, axis, keepdims, out, tri._argmin_over_axis)


def _boolean_reduction(x, axis, keepdims, out, fn):
    """all / any of an array of any dtype in one pass (an element is true when it is not zero):
    _boolean_reduction, dpnp/tensor/_utility_functions.py:31-85."""
    from ._dtypes import bool as _bool

    if not isinstance(x, usm_ndarray):
        raise TypeError(f"Expected dpnp_amd.tensor.usm_ndarray, got {type(x)}")
    nd = x.ndim
    arr, axis, perm = _move_reduced_axes_last(x, axis)
    red_nd = len(axis)
    res_shape = arr.shape[: nd - red_nd]
    out, user = _prepare_out(x, out, axis, keepdims, res_shape, _bool, guard_overlap=True)
    if red_nd == 0:
        ti._copy_usm_ndarray_into_usm_ndarray(src=arr, dst=out)  # a cast to bool
        return _finish(out, user, False, res_shape, red_nd, perm, nd)
    fn(src=arr, trailing_dims_to_reduce=red_nd, dst=out)  # an empty run gives the identity
    return _finish(out, user, keepdims, res_shape, red_nd, perm, nd)


def all(x, /, *, axis=None, keepdims=False, out=None):  # noqa: A001
    """True where every element along `axis` is non-zero."""
    return _boolean_reduction(x, axis, keepdims, out, tri._all)


def any(x, /, *, axis=None, keepdims=False, out=None):  # noqa: A001
    """True where some element along `axis` is non-zero."""
    return _boolean_reduction(x, axis, keepdims, out, tri._any)


def logsumexp(x, /, *, axis=None, dtype=None, keepdims=False, out=None):
    """log(sum(exp(x))) over `axis`, combined pairwise with logaddexp (no overflow)."""
    return _reduction_over_axis(x, axis, dtype, keepdims, out, tri._logsumexp_over_axis,
                                lambda i, o, u=None, q=None: i.kind != "c" and o.kind != "c"
                                and tri._logsumexp_over_axis_dtype_supported(i, o),
                                _default_accumulation_dtype_fp_types)


def reduce_hypot(x, /, *, axis=None, dtype=None, keepdims=False, out=None):
    """sqrt(sum(x**2)) over `axis`, combined pairwise with hypot (no overflow)."""
    return _reduction_over_axis(x, axis, dtype, keepdims, out, tri._hypot_over_axis,
                                lambda i, o, u=None, q=None: i.kind != "c" and o.kind != "c"
                                and tri._hypot_over_axis_dtype_supported(i, o),
                                _default_accumulation_dtype_fp_types)


def count_nonzero(x, /, *, axis=None, keepdims=False, out=None):
    """Number of non-zero elements over `axis` (int64), counted while reading `x` (the reference
    casts to bool and sums, dpnp/tensor/_reduction.py:472-512)."""
    return _reduction_over_axis(x, axis, "i8", keepdims, out, tri._count_nonzero_over_axis,
                                tri._count_nonzero_over_axis_dtype_supported, lambda dt, q=None: dt)
