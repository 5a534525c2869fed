"""View-making helpers the hot path relies on: broadcast_to, permute_dims, reshape,
squeeze, expand_dims (behaviour of dpnp/tensor/_manipulation_functions.py and
dpnp/tensor/_reshape.py for these five)."""
import operator

import numpy as np

from ._usmarray import usm_ndarray


def normalize_axis_index(axis, ndim, name="axis"):
    axis = operator.index(axis)
    if axis < -ndim or axis >= ndim:
        raise np.exceptions.AxisError(f"{name} {axis} is out of bounds for array of dimension {ndim}")
    return axis + ndim if axis < 0 else axis


def normalize_axis_tuple(axis, ndim, argname="axis", allow_duplicate=False):
    if not isinstance(axis, (tuple, list)):
        axis = (axis,)
    axes = tuple(normalize_axis_index(a, ndim, argname) for a in axis)
    if not allow_duplicate and len(set(axes)) != len(axes):
        raise ValueError(f"repeated axis in `{argname}` argument")
    return axes


def _broadcast_shape_impl(shapes):
    nd = max((len(s) for s in shapes), default=0)
    out = [1] * nd
    for s in shapes:
        for i, ext in enumerate(reversed(s)):
            j = nd - 1 - i
            if ext == 1 or ext == out[j]:
                continue
            if out[j] == 1:
                out[j] = ext
            else:
                raise ValueError("shape mismatch: objects cannot be broadcast to a single shape")
    return tuple(out)


def broadcast_to(x, shape):
    """A read-only-safe view of `x` with `shape`: new and stretched dims get stride 0."""
    if not isinstance(x, usm_ndarray):
        raise TypeError(f"Expected usm_ndarray type; got {type(x)}.")
    shape = tuple(shape) if isinstance(shape, (tuple, list)) else (shape,)
    nd = len(shape)
    if nd < x.ndim:
        raise ValueError(f"array of shape {x.shape} cannot be broadcast to shape {shape}")
    strides = [0] * nd
    for i in range(x.ndim):
        j = nd - x.ndim + i
        if x.shape[i] == shape[j]:
            strides[j] = x.strides[i] if shape[j] != 1 else 0
        elif x.shape[i] == 1:
            strides[j] = 0
        else:
            raise ValueError(f"array of shape {x.shape} cannot be broadcast to shape {shape}")
    return x._view(shape, strides, x._offset)


def permute_dims(x, axes):
    if not isinstance(x, usm_ndarray):
        raise TypeError(f"Expected usm_ndarray type; got {type(x)}.")
    axes = normalize_axis_tuple(axes, x.ndim, "axes")
    if sorted(axes) != list(range(x.ndim)):
        raise ValueError("The length of the passed axes does not match to the number of usm_ndarray dimensions.")
    return x._view([x.shape[a] for a in axes], [x.strides[a] for a in axes], x._offset)


def expand_dims(x, axis):
    axes = normalize_axis_tuple(axis, x.ndim + (len(axis) if isinstance(axis, (tuple, list)) else 1))
    nd = x.ndim + len(axes)
    sh, st = [], []
    it_sh, it_st = iter(x.shape), iter(x.strides)
    for d in range(nd):
        if d in axes:
            sh.append(1)
            st.append(0)
        else:
            sh.append(next(it_sh))
            st.append(next(it_st))
    return x._view(sh, st, x._offset)


def squeeze(x, axis=None):
    if axis is None:
        keep = [d for d in range(x.ndim) if x.shape[d] != 1]
    else:
        axes = normalize_axis_tuple(axis, x.ndim)
        for a in axes:
            if x.shape[a] != 1:
                raise ValueError("Cannot select an axis to squeeze out which has size not equal to one.")
        keep = [d for d in range(x.ndim) if d not in axes]
    return x._view([x.shape[d] for d in keep], [x.strides[d] for d in keep], x._offset)


def _reshape_strides(shape, strides, new_shape):
    """Strides of a no-copy reshape, or None when the layout needs a copy (NumPy's rule)."""
    old = [(s, st) for s, st in zip(shape, strides) if s != 1]
    new_strides = [0] * len(new_shape)
    oi = 0
    ni = 0
    nn = len(new_shape)
    while ni < nn:
        if new_shape[ni] == 1:
            new_strides[ni] = 0
            ni += 1
            continue
        if oi >= len(old):
            return None
        # grow groups on both sides until the element counts agree
        np_, op_ = new_shape[ni], old[oi][0]
        nj, oj = ni + 1, oi + 1
        while np_ != op_:
            if np_ < op_:
                if nj >= nn:
                    return None
                np_ *= new_shape[nj]
                nj += 1
            else:
                if oj >= len(old):
                    return None
                op_ *= old[oj][0]
                oj += 1
        # the old group must be internally contiguous (in units of its last stride)
        for k in range(oi, oj - 1):
            if old[k][1] != old[k + 1][0] * old[k + 1][1]:
                return None
        st = old[oj - 1][1]
        for k in range(nj - 1, ni - 1, -1):
            new_strides[k] = st
            st *= new_shape[k]
        ni, oi = nj, oj
    return new_strides


def reshape(x, shape, /, *, order="C", copy=None):
    if not isinstance(x, usm_ndarray):
        raise TypeError(f"Expected usm_ndarray type; got {type(x)}.")
    if order in ("F", "f"):
        # column-major reshape: the row-major reshape of the array with its axes reversed, reversed again
        # (dpnp/tensor/_reshape.py:98-190)
        if isinstance(shape, (tuple, list)):
            rshape = tuple(shape)[::-1]
        else:
            rshape = (shape,)
        r = reshape(permute_dims(x, tuple(range(x.ndim - 1, -1, -1))), rshape, order="C", copy=copy)
        return permute_dims(r, tuple(range(r.ndim - 1, -1, -1)))
    if order not in ("C", "c"):
        raise ValueError(f"Keyword 'order' not recognized. Expecting 'C' or 'F', got {order}")
    shape = [operator.index(s) for s in (shape if isinstance(shape, (tuple, list)) else (shape,))]
    if shape.count(-1) > 1:
        raise ValueError("Only one dimension of the new shape may be -1")
    if -1 in shape:
        known = 1
        for s in shape:
            if s != -1:
                known *= s
        if known == 0 or x.size % known != 0:
            raise ValueError(f"Can not reshape array of size {x.size} into {tuple(shape)}")
        shape[shape.index(-1)] = x.size // known
    n = 1
    for s in shape:
        n *= s
    if n != x.size:
        raise ValueError(f"Can not reshape array of size {x.size} into {tuple(shape)}")
    if x.size == 0:
        from ._usmarray import _contig_strides

        return x._view(shape, _contig_strides(shape), x._offset) if not copy else _copy_reshape(x, shape)
    st = _reshape_strides(x.shape, x.strides, shape)
    if st is not None and not copy:
        return x._view(shape, st, x._offset)
    if copy is False:
        raise ValueError("Reshaping the array requires a copy, but no copying was requested by using copy=False")
    return _copy_reshape(x, shape)


def _copy_reshape(x, shape):
    from ._copy_utils import copy as _copy
    from ._usmarray import _contig_strides

    c = _copy(x, order="C")
    return c._view(shape, _contig_strides(shape), c._offset)


def flip(x, /, *, axis=None):
    """View of `x` with the elements along `axis` (all axes when None) reversed."""
    if not isinstance(x, usm_ndarray):
        raise TypeError(f"Expected usm_ndarray type; got {type(x)}.")
    axes = range(x.ndim) if axis is None else normalize_axis_tuple(axis, x.ndim)
    key = tuple(slice(None, None, -1) if d in axes else slice(None) for d in range(x.ndim))
    return x[key]


def moveaxis(x, source, destination, /):
    """View with the axes `source` moved to the positions `destination`; the other axes keep their
    order (dpnp/tensor/_manipulation_functions.py, `moveaxis`)."""
    if not isinstance(x, usm_ndarray):
        raise TypeError(f"Expected usm_ndarray type; got {type(x)}.")
    source = normalize_axis_tuple(source, x.ndim, "source")
    destination = normalize_axis_tuple(destination, x.ndim, "destination")
    if len(source) != len(destination):
        raise ValueError("`source` and `destination` arguments must have the same number of elements")
    order = [n for n in range(x.ndim) if n not in source]
    for dest, src in sorted(zip(destination, source)):
        order.insert(dest, src)
    return permute_dims(x, tuple(order))


def swapaxes(x, axis1, axis2):
    """View with two axes exchanged (dpnp/tensor/_manipulation_functions.py, `swapaxes`)."""
    if not isinstance(x, usm_ndarray):
        raise TypeError(f"Expected usm_ndarray type; got {type(x)}.")
    axis1 = normalize_axis_index(axis1, x.ndim, "axis1")
    axis2 = normalize_axis_index(axis2, x.ndim, "axis2")
    order = list(range(x.ndim))
    order[axis1], order[axis2] = order[axis2], order[axis1]
    return permute_dims(x, tuple(order))


def matrix_transpose(x):
    """View with the last two axes exchanged; needs at least two dimensions."""
    if not isinstance(x, usm_ndarray):
        raise TypeError(f"Expected usm_ndarray type; got {type(x)}.")
    return x.mT


def broadcast_arrays(*args):
    """Views of the arrays stretched to their common shape."""
    if len(args) == 0:
        raise ValueError("`broadcast_arrays` requires at least one argument")
    for a in args:
        if not isinstance(a, usm_ndarray):
            raise TypeError(f"Expected usm_ndarray type; got {type(a)}.")
    shape = _broadcast_shape_impl([a.shape for a in args])
    return [a if a.shape == shape else broadcast_to(a, shape) for a in args]


# -- joining: copies into slices of the result through the copy / cast kernel ---------------------------
def _arrays_validation(arrays, check_ndim=True):
    """Result dtype of a join; the checks of dpnp/tensor/_manipulation_functions.py:47-88."""
    if not isinstance(arrays, (list, tuple)):
        raise TypeError(f"Expected tuple or list type, got {type(arrays)}.")
    if len(arrays) == 0:
        raise TypeError("Missing 1 required positional argument: 'arrays'.")
    for x in arrays:
        if not isinstance(x, usm_ndarray):
            raise TypeError(f"Expected usm_ndarray type, got {type(x)}.")
    res_dtype = arrays[0].dtype
    for x in arrays[1:]:
        res_dtype = np.promote_types(res_dtype, x.dtype)
    if check_ndim:
        for x in arrays[1:]:
            if x.ndim != arrays[0].ndim:
                raise ValueError(
                    "All the input arrays must have same number of dimensions, but the array at index 0 has "
                    f"{arrays[0].ndim} dimension(s) and the array at index {arrays.index(x)} has {x.ndim} dimension(s).")
    return res_dtype


def concat(arrays, /, *, axis=0):
    """Joins arrays along an existing axis (all of them flattened for axis=None); the result dtype follows
    the promotion rules (dpnp/tensor/_manipulation_functions.py:314-392)."""
    from ._copy_utils import _copy_into
    from ._ctors import empty

    if axis is None:
        res_dtype = _arrays_validation(arrays, check_ndim=False)
        res = empty(sum(x.size for x in arrays), dtype=res_dtype)
        start = 0
        for x in arrays:
            if x.size:
                _copy_into(reshape(x, (-1,)), res[start:start + x.size])
            start += x.size
        return res
    res_dtype = _arrays_validation(arrays)
    x0 = arrays[0]
    if x0.ndim == 0:
        raise ValueError("Zero-dimensional arrays cannot be concatenated")
    axis = normalize_axis_index(axis, x0.ndim)
    for i, x in enumerate(arrays[1:], 1):
        for j, ext in enumerate(x0.shape):
            if ext != x.shape[j] and j != axis:
                raise ValueError(
                    "All the input array dimensions for the concatenation axis must match exactly, but along "
                    f"dimension {j}, the array at index 0 has size {ext} and the array at index {i} has size "
                    f"{x.shape[j]}.")
    shape = list(x0.shape)
    shape[axis] = sum(x.shape[axis] for x in arrays)
    res = empty(tuple(shape), dtype=res_dtype)
    start = 0
    for x in arrays:
        stop = start + x.shape[axis]
        if x.size:
            _copy_into(x, res[(slice(None),) * axis + (slice(start, stop),)])
        start = stop
    return res


def stack(arrays, /, *, axis=0):
    """Joins arrays of one shape along a new axis (dpnp/tensor/_manipulation_functions.py, `stack`)."""
    from ._copy_utils import _copy_into
    from ._ctors import empty

    res_dtype = _arrays_validation(arrays)
    x0 = arrays[0]
    axis = normalize_axis_index(axis, x0.ndim + 1)
    for x in arrays[1:]:
        if x.shape != x0.shape:
            raise ValueError("All input arrays must have the same shape")
    res = empty(x0.shape[:axis] + (len(arrays),) + x0.shape[axis:], dtype=res_dtype)
    for i, x in enumerate(arrays):
        if x.size:
            _copy_into(x, res[(slice(None),) * axis + (i,)])
    return res


def diff(x, /, *, axis=-1, n=1, prepend=None, append=None):
    """n-th forward difference along `axis`; `prepend` / `append` (arrays or scalars) are joined to `x`
    first (dpnp/tensor/_utility_functions.py, `diff`).  Booleans difference with not_equal, as in NumPy."""
    from ._ctors import asarray
    from ._elementwise_funcs import not_equal, subtract

    if not isinstance(x, usm_ndarray):
        raise TypeError(f"Expecting dpnp.tensor.usm_ndarray type, got {type(x)}")
    axis = normalize_axis_index(axis, x.ndim)
    n = int(n)
    if n < 0:
        raise ValueError(f"`n` must be positive, got {n}")

    def side(v):
        if isinstance(v, usm_ndarray):
            return v
        from ._type_utils import result_type  # a Python scalar takes the array's kind where it can

        shape = list(x.shape)
        shape[axis] = 1
        return broadcast_to(asarray(v, dtype=result_type(x, v)), tuple(shape))

    parts = []
    if prepend is not None:
        parts.append(side(prepend))
    parts.append(x)
    if append is not None:
        parts.append(side(append))
    if len(parts) > 1:
        for p in parts:
            if p.ndim != x.ndim:
                raise ValueError("`prepend` and `append` must have the same number of dimensions as `x`")
        x = concat(parts, axis=axis)
    op = not_equal if x.dtype == np.dtype("?") else subtract
    for _ in range(n):
        if x.shape[axis] == 0:
            break
        lead = (slice(None),) * axis
        x = op(x[lead + (slice(1, None),)], x[lead + (slice(None, -1),)])
    return x
