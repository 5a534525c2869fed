"""The `test_<function>_dtype_matrix` and `test_<function>_out_type` cases that every file under
dpnp/tests/tensor/elementwise/ repeats (e.g. test_hypot.py:44-76, test_equal.py:43-75, test_abs.py:43-62): each
function over every pair (or every single) dtype it takes, on contiguous arrays and on the views x[::-1], y[::2];
result dtype and values as NumPy's (int64 with uint64 goes to float64 in both); pairs without a common type
that the function has a loop for raise."""
import warnings

import numpy as np
import pytest

import dpnp_amd.tensor as dpt
from tests.helpers import dev, host

pytestmark = pytest.mark.gpu

ALL = ["?", "i1", "u1", "i2", "u2", "i4", "u4", "i8", "u8", "f2", "f4", "f8", "c8", "c16"]
REAL = ALL[:12]
INTS = ALL[:9]

# name -> (NumPy function, dtypes, fill values of the two operands)
BINARY = {
    "add": (np.add, ALL, 1, 1), "subtract": (np.subtract, ALL[1:], 3, 1), "multiply": (np.multiply, ALL, 3, 2),
    "divide": (np.divide, ALL, 3, 2), "floor_divide": (np.floor_divide, REAL[1:], 7, 2),
    "remainder": (np.remainder, REAL[1:], 7, 3), "pow": (np.power, ALL[1:], 2, 3), "atan2": (np.arctan2, REAL, 1, 1),
    "hypot": (np.hypot, REAL, 3, 4), "copysign": (np.copysign, REAL, 2, 1), "logaddexp": (np.logaddexp, REAL, 1, 1),
    "maximum": (np.maximum, ALL, 1, 2), "minimum": (np.minimum, ALL, 1, 2), "nextafter": (np.nextafter, REAL, 1, 2),
    "equal": (np.equal, ALL, 1, 1), "not_equal": (np.not_equal, ALL, 1, 2), "less": (np.less, ALL, 1, 2),
    "less_equal": (np.less_equal, ALL, 1, 1), "greater": (np.greater, ALL, 2, 1),
    "greater_equal": (np.greater_equal, ALL, 1, 1), "logical_and": (np.logical_and, ALL, 1, 0),
    "logical_or": (np.logical_or, ALL, 0, 1), "logical_xor": (np.logical_xor, ALL, 1, 1),
    "bitwise_and": (np.bitwise_and, INTS, 3, 1), "bitwise_or": (np.bitwise_or, INTS, 2, 1),
    "bitwise_xor": (np.bitwise_xor, INTS, 3, 1), "bitwise_left_shift": (np.left_shift, INTS[1:], 3, 2),
    "bitwise_right_shift": (np.right_shift, INTS[1:], 12, 2),
}
UNARY = {
    "abs": (np.abs, ALL), "negative": (np.negative, ALL[1:]), "positive": (np.positive, ALL[1:]), "square": (np.square, ALL),
    "sign": (np.sign, ["i1", "i2", "i4", "i8", "f2", "f4", "f8"]), "sqrt": (np.sqrt, ALL), "cbrt": (np.cbrt, REAL),
    "exp": (np.exp, ALL), "log": (np.log, ALL), "sin": (np.sin, ALL), "cos": (np.cos, ALL), "tanh": (np.tanh, ALL),
    "floor": (np.floor, REAL), "ceil": (np.ceil, REAL), "trunc": (np.trunc, REAL), "isnan": (np.isnan, ALL),
    "isinf": (np.isinf, ALL), "isfinite": (np.isfinite, ALL), "signbit": (np.signbit, ["f2", "f4", "f8"]),
    "logical_not": (np.logical_not, ALL), "bitwise_invert": (np.invert, INTS), "conj": (np.conj, ALL), "real": (np.real, ALL),
    "imag": (np.imag, ALL), "angle": (np.angle, ["c8", "c16"]), "reciprocal": (np.reciprocal, ["f2", "f4", "f8", "c8", "c16"]),
}


def close(got, want):
    if want.dtype.kind in "fc":
        tol = 4 * float(np.finfo(want.dtype).eps)
        np.testing.assert_allclose(got, want, rtol=tol, atol=tol, equal_nan=True)
    else:
        np.testing.assert_array_equal(got, want)


@pytest.mark.parametrize("name", sorted(BINARY))
def test_binary_dtype_matrix(name):
    np_fn, dts, va, vb = BINARY[name]
    fn = getattr(dpt, name)
    sz = 127
    for d1 in dts:
        for d2 in dts:
            a1, a2 = np.full(sz, va, dtype=d1), np.full(2 * sz, vb, dtype=d2)
            try:
                with np.errstate(all="ignore"), warnings.catch_warnings():
                    warnings.simplefilter("ignore")
                    want = np_fn(a1, a2[:sz])
            except TypeError:
                # no common type that the function has a loop for (int64 with uint64 for the bitwise functions)
                with pytest.raises((ValueError, TypeError)):
                    fn(dev(a1), dev(a2[:sz].copy()))
                continue
            if name in ("floor_divide", "remainder", "pow") and "?" in (d1, d2):
                continue
            r = fn(dev(a1), dev(a2[:sz].copy()))
            assert r.dtype == want.dtype, (name, d1, d2, r.dtype, want.dtype)
            assert r.shape == a1.shape
            close(host(r), want)
            r = fn(dev(a1)[::-1], dev(a2)[::2])
            assert r.dtype == want.dtype
            close(host(r), want)


@pytest.mark.parametrize("name", sorted(UNARY))
def test_unary_out_type(name):
    np_fn, dts = UNARY[name]
    fn = getattr(dpt, name)
    for dt in dts:
        a = np.full(200, 1, dtype=dt)
        with np.errstate(all="ignore"), warnings.catch_warnings():
            warnings.simplefilter("ignore")
            want = np_fn(a)
        r = fn(dev(a))
        assert r.dtype == want.dtype, (name, dt, r.dtype, want.dtype)
        close(host(r), want)
        r = fn(dev(np.full(400, 1, dtype=dt))[::-2])
        assert r.dtype == want.dtype and r.shape == (200,)
        close(host(r), want)
