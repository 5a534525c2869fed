"""dpnp-level functions that the reference builds from elementwise calls and reductions:
round / around / fix (dpnp/dpnp_iface_mathematical.py, DPNPRound in
dpnp/dpnp_algo/dpnp_elementwise_common.py:1296-1341), real_if_close, the predicates and comparisons of
dpnp/dpnp_iface_logic.py (allclose, array_equal, array_equiv, iscomplex, isreal, iscomplexobj,
isrealobj, isfortran, isneginf, isposinf) and ptp / average of dpnp/dpnp_iface_statistics.py.

Argument checks, result dtypes and errors follow those files; where the reference runs several
kernels for one answer (isneginf: isinf, signbit, logical_and) one comparison is used.
"""
import math
import warnings

import numpy as np

from . import tensor as dpt
from .dpnp_array import dpnp_array
from .dpnp_iface import (
    _unpack_out,
    _wrap,
    all,  # noqa: A004
    any,  # noqa: A004
    asarray,
    broadcast_to,
    check_supported_arrays_type,
    equal,
    get_usm_ndarray,
    is_supported_array_type,
    isclose,
    isnan,
    logical_and,
    logical_or,
    max,  # noqa: A004
    mean,
    min,  # noqa: A004
    multiply,
    subtract,
    trunc,
    zeros_like,
    ones_like,
)

__all__ = ["allclose", "around", "array_equal", "array_equiv", "average", "fix", "iscomplex", "iscomplexobj",
           "isfortran", "isneginf", "isposinf", "isreal", "isrealobj", "ptp", "real_if_close", "round"]


# -- rounding -----------------------------------------------------------------------------------------
def round(x, /, decimals=0, out=None, *, dtype=None):  # noqa: A001
    """Round to `decimals` places, halves to even (DPNPRound.__call__,
    dpnp/dpnp_algo/dpnp_elementwise_common.py:1316-1341): for decimals != 0 the array is scaled by
    10**decimals, rounded and scaled back; integers are untouched for decimals > 0."""
    out = _unpack_out(out)
    if dtype is not None and out is not None:
        raise TypeError("Requested function=round only takes `out` or `dtype` as an argument, "
                        "but both were provided.")
    check_supported_arrays_type(x)
    x_usm = get_usm_ndarray(x)
    out_usm = None if out is None else get_usm_ndarray(out)
    if decimals == 0:
        if dtype is not None:
            x_usm = dpt.astype(x_usm, dtype, copy=False)
        res = dpt.round(x_usm, out=out_usm)
    else:
        if x_usm.dtype.kind in "iu":
            if decimals < 0:
                dtype = x_usm.dtype
                scaled = dpt.round(dpt.multiply(x_usm, 10 ** decimals), out=out_usm)
                res = dpt.divide(scaled, 10 ** decimals, out=out_usm)
            else:
                res = dpt.round(x_usm, out=out_usm)
        else:
            scaled = dpt.round(dpt.multiply(x_usm, 10 ** decimals), out=out_usm)
            res = dpt.divide(scaled, 10 ** decimals, out=out_usm)
        if dtype is not None:
            res = dpt.astype(res, dtype, copy=False)
    if out is not None and isinstance(out, dpnp_array):
        return out
    return _wrap(res)


def around(x, /, decimals=0, out=None):
    """Alias of round (dpnp/dpnp_iface_mathematical.py, `around`)."""
    return round(x, decimals, out)


def fix(x, /, out=None, **kwargs):
    """Round towards zero; deprecated in favour of trunc, as in the reference
    (DPNPDeprecatedUnaryFunc, dpnp/dpnp_iface_mathematical.py `fix`)."""
    warnings.warn("dpnp.fix is deprecated in favor of dpnp.trunc", DeprecationWarning, stacklevel=2)
    return trunc(x, out=out, **kwargs)


def real_if_close(a, tol=100):
    """The real part of a complex array whose imaginary parts are all below `tol` machine epsilons
    (or below `tol` itself when tol <= 1); anything else comes back unchanged."""
    check_supported_arrays_type(a)
    if a.dtype.kind != "c":
        return a
    if not np.isscalar(tol):
        raise TypeError(f"Tolerance must be a scalar, but got {type(tol)}")
    if tol > 1:
        tol = float(np.finfo(a.dtype).eps) * tol
    u = get_usm_ndarray(a)
    if bool(dpt.all(dpt.less(dpt.abs(dpt.imag(u)), tol))):
        return _wrap(dpt.real(u))
    return a


# -- predicates ---------------------------------------------------------------------------------------
def _is_signed_inf(x, out, sign):
    check_supported_arrays_type(x)
    if out is not None:
        check_supported_arrays_type(out)
    if x.dtype.kind == "c":
        raise TypeError(f"This operation is not supported for {x.dtype} values because it would be ambiguous.")
    if x.dtype.kind != "f":
        # no infinity among integers and booleans
        out_usm = None if out is None else get_usm_ndarray(out)
        res = dpt.isinf(get_usm_ndarray(x), out=out_usm)
        return out if isinstance(out, dpnp_array) else _wrap(res)
    return equal(x, sign * math.inf, out=out)


def isneginf(x, out=None):
    """True where x is -inf (dpnp/dpnp_iface_logic.py:1406-1482)."""
    return _is_signed_inf(x, out, -1.0)


def isposinf(x, out=None):
    """True where x is +inf (dpnp/dpnp_iface_logic.py:1485-1561)."""
    return _is_signed_inf(x, out, 1.0)


def iscomplex(x):
    """True where the imaginary part is not zero; all False for a real dtype."""
    check_supported_arrays_type(x)
    if x.dtype.kind == "c":
        return _wrap(dpt.not_equal(dpt.imag(get_usm_ndarray(x)), 0))
    return zeros_like(x, dtype="?")


def isreal(x):
    """True where the imaginary part is zero; all True for a real dtype."""
    check_supported_arrays_type(x)
    if x.dtype.kind == "c":
        return _wrap(dpt.equal(dpt.imag(get_usm_ndarray(x)), 0))
    return ones_like(x, dtype="?")


def iscomplexobj(x):
    """Whether x has a complex dtype (numpy.iscomplexobj on the object, as the reference does)."""
    return np.iscomplexobj(x)


def isrealobj(x):
    return not iscomplexobj(x)


def isfortran(a):
    """True for an array that is column-major and not also row-major."""
    check_supported_arrays_type(a)
    return a.flags.fnc


# -- comparisons of whole arrays ------------------------------------------------------------------------
def allclose(a, b, rtol=1e-05, atol=1e-08, equal_nan=False):
    """all(isclose(a, b)) as a 0-d bool array (dpnp/dpnp_iface_logic.py, `allclose`)."""
    return all(isclose(a, b, rtol=rtol, atol=atol, equal_nan=equal_nan))


def _scalar_false():
    return asarray(False)


def array_equal(a1, a2, equal_nan=False):
    """0-d bool array: same shape and equal elements (NaNs in the same places count as equal
    when `equal_nan`)."""
    check_supported_arrays_type(a1, a2, scalar_type=True)
    if np.isscalar(a1):
        a1 = asarray(a1, dtype=dpt.result_type(a1, get_usm_ndarray(a2)))
    elif np.isscalar(a2):
        a2 = asarray(a2, dtype=dpt.result_type(get_usm_ndarray(a1), a2))
    if a1.shape != a2.shape:
        return _scalar_false()
    if not equal_nan:
        return all(equal(a1, a2))
    if a1 is a2:
        return asarray(True)
    if a1.dtype.kind not in "fc" and a2.dtype.kind not in "fc":
        return all(equal(a1, a2))
    # equal, or NaN in both: the same answer as comparing the NaN masks and then the rest
    both_nan = logical_and(isnan(a1), isnan(a2))
    return all(logical_or(equal(a1, a2), both_nan))


def array_equiv(a1, a2):
    """0-d bool array: the arrays broadcast against each other and are equal everywhere."""
    check_supported_arrays_type(a1, a2, scalar_type=True)
    if not np.isscalar(a1) and not np.isscalar(a2):
        try:
            np.broadcast_shapes(a1.shape, a2.shape)
        except ValueError:
            return _scalar_false()
    return all(equal(a1, a2))


# -- statistics -----------------------------------------------------------------------------------------
def ptp(a, /, axis=None, out=None, keepdims=False):
    """max - min along an axis (dpnp/dpnp_iface_statistics.py, `ptp`)."""
    return subtract(max(a, axis=axis, keepdims=keepdims, out=out), min(a, axis=axis, keepdims=keepdims), out=out)


def average(a, axis=None, weights=None, returned=False, *, keepdims=False):
    """Weighted mean along an axis (dpnp/dpnp_iface_statistics.py, `average`): sum(a * w) / sum(w);
    ZeroDivisionError when weights sum to zero; with `returned` also the sum of the weights."""
    check_supported_arrays_type(a)
    if weights is None:
        avg = mean(a, axis=axis, keepdims=keepdims)
        scl = asarray(avg.dtype.type(a.size / avg.size if avg.size else 0))
    else:
        if not is_supported_array_type(weights):
            weights = asarray(weights)
        if a.dtype.kind not in "fc":
            res_dtype = dpt.result_type(a.dtype, weights.dtype, dpt.dtype("f8"))
        else:
            res_dtype = dpt.result_type(a.dtype, weights.dtype)
        if a.shape != weights.shape:
            if axis is None:
                raise TypeError("Axis must be specified when shapes of input array and weights differ.")
            if weights.ndim != 1:
                raise TypeError("1D weights expected when shapes of input array and weights differ.")
            if weights.shape[0] != a.shape[axis]:
                raise ValueError("Length of weights not compatible with specified axis.")
            w = dpt.broadcast_to(get_usm_ndarray(weights), (a.ndim - 1) * (1,) + weights.shape)
            perm = list(range(a.ndim))
            ax = axis % a.ndim
            perm[-1], perm[ax] = perm[ax], perm[-1]
            weights = _wrap(dpt.permute_dims(w, perm))
        scl = weights.sum(axis=axis, dtype=res_dtype, keepdims=keepdims)
        if bool(any(equal(scl, 0.0))):
            raise ZeroDivisionError("Weights sum to zero, can't be normalized")
        avg = multiply(a, weights).sum(axis=axis, dtype=res_dtype, keepdims=keepdims)
        avg /= scl
    if returned:
        if scl.shape != avg.shape:
            scl = broadcast_to(scl, avg.shape).copy()
        return avg, scl
    return avg
