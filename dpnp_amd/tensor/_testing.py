"""allclose for device arrays (dpnp/tensor/_testing.py:31-180):
|a - b| <= max(atol, rtol * max(|a|, |b|)) for finite pairs, infinities equal in place and sign,
NaNs equal when `equal_nan`.  The result is a 0-d bool array, like `dpt.all`."""
import numpy as np

from ._copy_utils import astype
from ._ctors import asarray
from ._elementwise_funcs import (abs, equal, imag, isfinite, isinf, isnan, less_equal, maximum, multiply,  # noqa: A004
                                 real, subtract)
from ._manipulation_functions import _broadcast_shape_impl, broadcast_to
from ._reduction import all as all_  # noqa: A004
from ._reduction import any as any_
from ._search_functions import where
from ._usmarray import usm_ndarray


def _false():
    return asarray(False)


def _allclose_real_fp(r1, r2, atol, rtol, equal_nan):
    n1, n2 = isnan(r1), isnan(r2)
    if equal_nan:
        if not all_(equal(n1, n2)):
            return _false()
    elif any_(n1) or any_(n2):
        return _false()
    i1 = isinf(r1)
    if not all_(equal(i1, isinf(r2))):
        return _false()
    true = asarray(True)
    if not all_(where(i1, equal(r1, r2), true)):
        return _false()
    bound = maximum(multiply(maximum(abs(r1), abs(r2)), rtol), atol)
    close = less_equal(abs(subtract(r1, r2)), bound)
    return all_(where(isfinite(r1), close, true))


def allclose(a1, a2, atol=1e-8, rtol=1e-5, equal_nan=False):
    """True (0-d array) if the two arrays agree elementwise within the tolerances."""
    for a in (a1, a2):
        if not isinstance(a, usm_ndarray):
            raise TypeError(f"Expected dpnp_amd.tensor.usm_ndarray type, got {type(a)}.")
    atol, rtol = float(atol), float(rtol)
    if atol < 0.0 or rtol < 0.0:
        raise ValueError("Absolute and relative tolerances must be non-negative")
    equal_nan = True if equal_nan else False
    shape = _broadcast_shape_impl([a1.shape, a2.shape])
    b1, b2 = a1, a2
    if b1.dtype != b2.dtype:
        res_dt = np.promote_types(b1.dtype, b2.dtype)
        b1, b2 = astype(b1, res_dt), astype(b2, res_dt)
    b1, b2 = broadcast_to(b1, shape), broadcast_to(b2, shape)
    k = b1.dtype.kind
    if k == "c":
        re = _allclose_real_fp(real(b1), real(b2), atol, rtol, equal_nan)
        if not re:
            return re
        return _allclose_real_fp(imag(b1), imag(b2), atol, rtol, equal_nan)
    if k == "f":
        return _allclose_real_fp(b1, b2, atol, rtol, equal_nan)
    return all_(equal(b1, b2))


__all__ = ["allclose"]
