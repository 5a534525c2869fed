"""Type promotion for elementwise calls and reductions.

Kernels exist for exact dtype combinations only; anything else is resolved here by
searching, in a fixed dtype order, for the cheapest safe casts of the operands for which
a kernel exists, with Python scalars taking part as "weak" types (NEP 50).  Restates the
behaviour of dpnp/tensor/_type_utils.py:37-76,157-266,389-485,932-952 for a device that
has both fp16 and fp64 (so device-dependent branches reduce to NumPy's rules).
"""
import numpy as np

from . import _dtypes as dt_
from . import _tensor_impl as ti

_SEARCH_ORDER = list(dt_.ALL_DTYPES)  # bool, ints by width (signed first), floats, complex


class _Weak:
    """Dtype stand-in for a Python scalar operand; keeps the value for range checks."""

    rank = -1

    def __init__(self, value):
        self.value = value

    def get(self):
        return self.value


class WeakBooleanType(_Weak):
    rank = 0


class WeakIntegralType(_Weak):
    rank = 1


class WeakFloatingType(_Weak):
    rank = 2


class WeakComplexType(_Weak):
    rank = 3


_KIND_RANK = {"b": 0, "i": 1, "u": 1, "f": 2, "c": 3}


def _is_weak_dtype(d):
    return isinstance(d, _Weak)


def _default_for_weak(weak, strong):
    """dtype a weak scalar takes when its kind outranks the array's kind."""
    if isinstance(weak, WeakIntegralType):
        return dt_.dtype(ti.default_device_int_type())
    if isinstance(weak, WeakComplexType):
        if strong in (dt_.float16, dt_.float32):
            return dt_.complex64
        return dt_.complex128
    return dt_.float64


def _resolve_weak_types(d1, d2, dev=None):
    """Replace a weak operand type by a concrete dtype (same-kind scalars adopt the
    array's dtype; higher-kind scalars take the default dtype of their kind)."""
    if _is_weak_dtype(d1):
        if _is_weak_dtype(d2):
            raise ValueError("both operands are Python scalars")
        if d1.rank > _KIND_RANK[d2.kind]:
            return _default_for_weak(d1, d2), d2
        return d2, d2
    if _is_weak_dtype(d2):
        if d2.rank > _KIND_RANK[d1.kind]:
            return d1, _default_for_weak(d2, d1)
        return d1, d1
    return d1, d2


def _resolve_weak_types_all_py_ints(d1, d2, dev=None):
    """As above, but a Python int that does not fit the integer array's dtype keeps its
    own minimal dtype so that comparisons and divide see the true value."""
    if _is_weak_dtype(d1) and not _is_weak_dtype(d2):
        if isinstance(d1, WeakIntegralType) and d2.kind in "iu":
            info = np.iinfo(d2)
            if not (info.min <= d1.get() <= info.max):
                return dt_.dtype(np.min_scalar_type(d1.get())), d2
    elif _is_weak_dtype(d2) and not _is_weak_dtype(d1):
        if isinstance(d2, WeakIntegralType) and d1.kind in "iu":
            info = np.iinfo(d1)
            if not (info.min <= d2.get() <= info.max):
                return d1, dt_.dtype(np.min_scalar_type(d2.get()))
    return _resolve_weak_types(d1, d2, dev)


def _resolve_one_strong_two_weak_types(st, d1, d2, dev=None):
    """where(cond, x1, x2) with scalar x1 and/or x2: `st` is the dtype of the array operand
    that anchors the resolution."""
    if _is_weak_dtype(st):
        raise ValueError("anchor dtype must be concrete")
    if _is_weak_dtype(d1) and _is_weak_dtype(d2):
        r1 = _default_for_weak(d1, st) if d1.rank > _KIND_RANK[st.kind] else st
        r2 = _default_for_weak(d2, st) if d2.rank > _KIND_RANK[st.kind] else st
        return r1, r2
    if _is_weak_dtype(d1):
        anchor = max([(_KIND_RANK[st.kind], st), (_KIND_RANK[d2.kind], d2)], key=lambda p: p[0])[1]
        if d1.rank > _KIND_RANK[anchor.kind]:
            return _default_for_weak(d1, anchor), d2
        return anchor, d2
    if _is_weak_dtype(d2):
        anchor = max([(_KIND_RANK[st.kind], st), (_KIND_RANK[d1.kind], d1)], key=lambda p: p[0])[1]
        if d2.rank > _KIND_RANK[anchor.kind]:
            return d1, _default_for_weak(d2, anchor)
        return d1, anchor
    return d1, d2


def _can_cast(from_, to_, casting="safe"):
    return np.can_cast(from_, to_, casting=casting)


def _get_device_default_dtype(kind, dev=None):
    return {"b": dt_.bool, "i": dt_.int64, "u": dt_.uint64, "f": dt_.float64, "c": dt_.complex128}[kind]


# -- acceptance hooks: may veto a candidate found by the search (or raise) ---------------------------
def _acceptance_fn_default_unary(arg_dtype, buf_dt, res_dt, dev=None):
    return True


def _acceptance_fn_default_binary(a1, a2, b1, b2, res_dt, dev=None):
    return True


def _acceptance_fn_divide(a1, a2, b1, b2, res_dt, dev=None):
    # both operands change kind (int / int): use the default floating type, as NumPy does
    if b1.kind != a1.kind and b2.kind != a2.kind:
        return res_dt == _get_device_default_dtype(res_dt.kind)
    return True


def _acceptance_fn_reciprocal(arg_dtype, buf_dt, res_dt, dev=None):
    if buf_dt.kind != arg_dtype.kind:
        return res_dt == _get_device_default_dtype(res_dt.kind)
    return True


def _acceptance_fn_negative(arg_dtype, buf_dt, res_dt, dev=None):
    if arg_dtype.char == "?":
        raise ValueError(
            "The `negative` function, the `-` operator, is not supported for inputs of data type "
            "bool, use the `~` operator or the `logical_not` function instead")
    return True


def _acceptance_fn_subtract(a1, a2, b1, b2, res_dt, dev=None):
    if a1.char == "?" and a2.char == "?":
        raise ValueError(
            "The `subtract` function, the `-` operator, is not supported for inputs of data type "
            "bool, use the `^` operator,  the `bitwise_xor`, or the `logical_xor` function instead")
    return True


def _find_buf_dtype(arg_dtype, query_fn, dev=None, acceptance_fn=_acceptance_fn_default_unary):
    """(cast dtype or None, result dtype) for a unary op; (None, None) if nothing fits."""
    res = query_fn(arg_dtype)
    if res is not None:
        return None, res
    for cand in _SEARCH_ORDER:
        if _can_cast(arg_dtype, cand):
            res = query_fn(cand)
            if res is not None and acceptance_fn(arg_dtype, cand, res, dev):
                return cand, res
    return None, None


def _find_buf_dtype2(d1, d2, query_fn, dev=None, acceptance_fn=_acceptance_fn_default_binary):
    """(cast1 or None, cast2 or None, result dtype) for a binary op; Nones if nothing fits."""
    res = query_fn(d1, d2)
    if res is not None:
        return None, None, res
    for c1 in _SEARCH_ORDER:
        if not _can_cast(d1, c1):
            continue
        for c2 in _SEARCH_ORDER:
            if not _can_cast(d2, c2):
                continue
            res = query_fn(c1, c2)
            if res is None:
                continue
            b1 = None if c1 == d1 else c1
            b2 = None if c2 == d2 else c2
            if b1 is None or b2 is None or acceptance_fn(d1, d2, b1, b2, res, dev):
                return b1, b2, res
    return None, None, None


def _find_buf_dtype_in_place_op(d1, d2, query_fn, dev=None):
    """(cast of rhs or None, result dtype) for `lhs op= rhs`; lhs is never cast."""
    res = query_fn(d1, d2)
    if res is not None:
        return None, res
    if _can_cast(d2, d1, casting="same_kind"):
        res = query_fn(d1, d1)
        if res is not None:
            return d1, res
    return None, None


def _to_device_supported_dtype(d, dev=None):
    return d


def _default_accumulation_dtype(inp_dt, q=None):
    """Result dtype of sum/prod when none is asked for: bool and signed ints widen to int64,
    unsigned to uint64, floating and complex stay."""
    k = inp_dt.kind
    if k in "bi":
        res = dt_.int64
        return inp_dt if inp_dt.itemsize > res.itemsize else res
    if k == "u":
        return dt_.uint64
    return inp_dt


def _default_accumulation_dtype_fp_types(inp_dt, q=None):
    """Result dtype for accumulations defined on floating types only (mean, var, ...)."""
    k = inp_dt.kind
    if k in "biu":
        return dt_.float64  # the device has fp64, so ints never settle for float32
    if k == "c":
        raise ValueError("function not defined for complex types")
    return inp_dt


def result_type(*arrays_and_dtypes):
    """Array-API result_type over arrays, dtypes and Python scalars."""
    from ._usmarray import usm_ndarray

    dtypes, weak = [], []
    for a in arrays_and_dtypes:
        if isinstance(a, usm_ndarray):
            dtypes.append(a.dtype)
        elif isinstance(a, (bool, int, float, complex)):
            weak.append(a)
        else:
            dtypes.append(dt_.dtype(a))
    if not dtypes:
        return np.result_type(*weak)
    res = np.result_type(*dtypes)
    for w in weak:
        res = np.result_type(res, w)
    return dt_.dtype(res)


def can_cast(from_, to, /, *, casting="safe"):
    from ._usmarray import usm_ndarray

    f = from_.dtype if isinstance(from_, usm_ndarray) else dt_.dtype(from_)
    return bool(np.can_cast(f, dt_.dtype(to), casting=casting))
