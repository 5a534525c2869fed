"""Special values, corner cases and error classes of the elementwise functions, exercised like
the reference's per-function tests (dpnp/tests/tensor/elementwise/test_remainder.py,
test_floor_divide.py, test_divide.py, test_maximum_minimum.py, test_round.py, test_sign.py,
test_bitwise_left_shift.py, test_reciprocal.py, test_square.py, test_abs.py, test_pow.py)."""
import itertools

import numpy as np
import pytest

import dpnp_amd.tensor as dpt
from dpnp_amd.tensor import _tensor_elementwise_impl as tei

pytestmark = pytest.mark.gpu

NO_COMPLEX = ["?", "i1", "u1", "i2", "u2", "i4", "u4", "i8", "u8", "f2", "f4", "f8"]
INTEGRAL = NO_COMPLEX[1:9]


@pytest.mark.parametrize("dt", NO_COMPLEX[1:8:2])
def test_remainder_negative_integers(dt):
    # test_remainder.py:80-94
    x, x_np = dpt.arange(-5, -1, 1, dtype=dt), np.arange(-5, -1, 1, dtype=dt)
    assert (dpt.asnumpy(dpt.remainder(x, 3)) == np.remainder(x_np, 3)).all()
    assert (dpt.asnumpy(dpt.remainder(3, x)) == np.remainder(3, x_np)).all()


def test_remainder_and_floor_divide_by_integer_zero():
    # test_remainder.py:97-110, test_floor_divide.py:97-106: x % 0 == 0 and x // 0 == 0 for integers
    for dt in ["i4", "u4"]:
        x = dpt.ones(1, dtype=dt)
        assert (dpt.asnumpy(dpt.remainder(x, dpt.zeros_like(x))) == np.zeros(1, dtype=dt)).all()
    for dt in INTEGRAL:
        x = dpt.arange(10, dtype=dt)
        res = dpt.floor_divide(x, dpt.zeros_like(x))
        np.testing.assert_array_equal(dpt.asnumpy(res), np.zeros(10, dtype=res.dtype))


@pytest.mark.parametrize("dt", ["f2", "f4", "f8"])
def test_remainder_negative_floats_and_special_cases(dt):
    # test_remainder.py:113-153
    x, x_np = dpt.linspace(-5, 5, 20, dtype=dt), np.linspace(-5, 5, 20, dtype=dt)
    tol = 8 * dpt.finfo(dt).resolution
    with np.errstate(invalid="ignore", divide="ignore"):
        assert np.allclose(dpt.asnumpy(dpt.remainder(x, 3)), np.remainder(x_np, 3), rtol=tol, atol=tol, equal_nan=True)
        assert np.allclose(dpt.asnumpy(dpt.remainder(3, x)), np.remainder(3, x_np), rtol=tol, atol=tol, equal_nan=True)
    lhs = [np.nan, np.inf, 0.0, -0.0, -0.0, 1.0, np.inf, -np.inf]
    rhs = [np.nan, np.inf, -0.0, 1.0, 1.0, 0.0, 1.0, -1.0]
    res = dpt.asnumpy(dpt.remainder(dpt.asarray(lhs, dtype=dt), dpt.asarray(rhs, dtype=dt)))
    with np.errstate(invalid="ignore", divide="ignore"):
        want = np.remainder(np.asarray(lhs, dtype=dt), np.asarray(rhs, dtype=dt))
    np.testing.assert_array_equal(res, want)
    np.testing.assert_array_equal(np.signbit(res[~np.isnan(res)]), np.signbit(want[~np.isnan(want)]))


def test_floor_divide_rounding_and_special_cases():
    # test_floor_divide.py:80-148
    np.testing.assert_array_equal(dpt.asnumpy(dpt.floor_divide(dpt.ones(1, dtype="i4"), -2)), [-1])
    np.testing.assert_array_equal(dpt.asnumpy(dpt.floor_divide(dpt.full(1, -1, dtype="i4"), 2)), [-1])
    pairs = [(np.inf, np.inf), (0.0, -1.0), (-1.0, 0.0), (1.0, np.nan), (7.5, -2.0), (-7.5, 2.0), (-0.0, 3.0)]
    a = np.asarray([p[0] for p in pairs], dtype="f4")
    b = np.asarray([p[1] for p in pairs], dtype="f4")
    with np.errstate(all="ignore"):
        want = np.floor_divide(a, b)
    got = dpt.asnumpy(dpt.floor_divide(dpt.asarray(a), dpt.asarray(b)))
    np.testing.assert_array_equal(got, want)
    np.testing.assert_array_equal(np.signbit(got[~np.isnan(got)]), np.signbit(want[~np.isnan(want)]))
    # where the reference's functor (the quotient itself when it is zero, its floor otherwise) and
    # NumPy differ, the reference's tests pin these values (test_floor_divide.py:132-142)
    r = dpt.asnumpy(dpt.floor_divide(dpt.asarray(-1.0, dtype="f4"), dpt.asarray(np.inf, dtype="f4")))
    assert r == 0.0 and np.signbit(r)
    assert dpt.asnumpy(dpt.floor_divide(dpt.asarray(np.inf, dtype="f4"), dpt.asarray(-1.0, dtype="f4"))) == -np.inf


def test_divide_with_python_scalars_and_scalar_overflow():
    # test_divide.py:154-200
    res = dpt.divide(-4, dpt.asarray(1, dtype="u4"))
    assert res.dtype.kind == "f" and dpt.allclose(res, -4 / dpt.asarray(1, dtype="i4"))
    res = dpt.divide(dpt.asarray(3, dtype="u4"), -2)
    assert res.dtype.kind == "f" and dpt.allclose(res, dpt.asarray(3, dtype="i4") / -2)
    for fp_dt in (dpt.float16, dpt.float32):
        x = dpt.ones(10, dtype=fp_dt)
        out = dpt.empty_like(x)
        tei._divide_by_scalar(src=x, scalar=2 ** np.finfo(fp_dt).maxexp, dst=out)
        assert dpt.all(out == 0)
    # in-place true division of an integer array cannot hold the result
    with pytest.raises(ValueError):
        x = dpt.ones(4, dtype="i4")
        x /= 2


@pytest.mark.parametrize("dtype", ["f2", "f4", "f8"])
def test_maximum_minimum_real_special_cases(dtype):
    # test_maximum_minimum.py:148-166
    vals = list(itertools.product([np.nan, np.inf, -np.inf, 5.0, -3.0], repeat=2))
    Xnp = np.array([v[0] for v in vals], dtype=dtype)
    Ynp = np.array([v[1] for v in vals], dtype=dtype)
    X, Y = dpt.asarray(Xnp), dpt.asarray(Ynp)
    np.testing.assert_array_equal(dpt.asnumpy(dpt.maximum(X, Y)), np.maximum(Xnp, Ynp))
    np.testing.assert_array_equal(dpt.asnumpy(dpt.minimum(X, Y)), np.minimum(Xnp, Ynp))


@pytest.mark.parametrize("dtype", ["c8", "c16"])
def test_maximum_minimum_complex_special_cases(dtype):
    # test_maximum_minimum.py:169-192
    parts = [np.nan, -np.inf, -np.inf, +2.0, -1.0]
    zs = [complex(*v) for v in itertools.product(parts, repeat=2)]
    pairs = list(itertools.product(zs, repeat=2))
    Xnp = np.array([p[0] for p in pairs], dtype=dtype)
    Ynp = np.array([p[1] for p in pairs], dtype=dtype)
    X, Y = dpt.asarray(Xnp), dpt.asarray(Ynp)
    for fn, nfn in ((dpt.maximum, np.maximum), (dpt.minimum, np.minimum)):
        R, Rnp = fn(X, Y), nfn(Xnp, Ynp)
        np.testing.assert_array_equal(dpt.asnumpy(dpt.real(R)), np.real(Rnp))
        np.testing.assert_array_equal(dpt.asnumpy(dpt.imag(R)), np.imag(Rnp))


@pytest.mark.parametrize("dtype", ["f2", "f4", "f8"])
def test_round_special_cases_keep_the_sign_of_zero(dtype):
    # test_round.py:109-122: ties to even
    x = [np.nan, np.inf, -np.inf, 1.5, 2.5, -1.5, -2.5, 0.0, -0.0, 0.5, -0.5]
    Y = dpt.asnumpy(dpt.round(dpt.asarray(x, dtype=dtype)))
    Ynp = np.round(np.array(x, dtype=dtype))
    np.testing.assert_array_equal(Y, Ynp)
    np.testing.assert_array_equal(np.signbit(Y), np.signbit(Ynp))
    z = np.array([1.5 - 2.5j, -0.5 + 0.5j, np.inf - 1.5j], dtype="c8")
    np.testing.assert_array_equal(dpt.asnumpy(dpt.round(dpt.asarray(z))), np.round(z))
    assert dpt.round(dpt.ones(3, dtype="i4")).dtype == dpt.dtype("i4")


def test_sign_of_signed_types_and_complex_layouts():
    # test_sign.py:61-101
    for dt in NO_COMPLEX[1:8:2] + NO_COMPLEX[9:]:
        x_np = np.arange(-20, 20, 1, dtype=dt)
        assert (dpt.asnumpy(dpt.sign(dpt.asarray(x_np))) == np.sign(x_np)).all()
    rng = np.random.default_rng(5)
    shape = (4, 5, 6, 3)
    Xnp = (rng.standard_normal(shape) + 1j * rng.standard_normal(shape)).astype("c8")
    X = dpt.asarray(Xnp)
    for order in "CFAK":
        for perms in itertools.permutations(range(4)):
            U = dpt.permute_dims(X[:, ::-1, ::-1, :], perms)
            X_t = np.transpose(Xnp[:, ::-1, ::-1, :], perms)
            tol = dpt.finfo(U.dtype).resolution
            np.testing.assert_allclose(dpt.asnumpy(dpt.sign(U, order=order)), X_t / np.abs(X_t), atol=tol, rtol=tol)


@pytest.mark.parametrize("op_dtype", INTEGRAL)
def test_shifts_by_the_width_or_more_give_zero(op_dtype):
    # test_bitwise_left_shift.py:107-117, test_bitwise_right_shift.py
    x = dpt.ones(255, dtype=op_dtype)
    y = dpt.asarray(64, dtype=op_dtype)
    assert dpt.all(dpt.equal(dpt.bitwise_left_shift(x, y), 0))
    assert dpt.all(dpt.equal(dpt.bitwise_right_shift(x, y), 0))


def test_reciprocal_square_abs_special_cases():
    # test_reciprocal.py:81-110, test_square.py:56-73, test_abs.py:140-184
    x = dpt.asarray([np.nan, 0.0, -0.0, np.inf, -np.inf], dtype="f4")
    expected = dpt.asarray([np.nan, np.inf, -np.inf, 0.0, -0.0], dtype="f4")
    assert dpt.allclose(dpt.reciprocal(x), expected, equal_nan=True)
    assert np.array_equal(np.signbit(dpt.asnumpy(dpt.reciprocal(x))), np.signbit(dpt.asnumpy(expected)))
    finites = [-1.0, -0.0, 0.0, 1.0, 3.5]
    c_ = [complex(*v) for v in itertools.product(finites, repeat=2) if v != (0.0, 0.0) and v != (-0.0, 0.0)
          and v != (0.0, -0.0) and v != (-0.0, -0.0)]
    for dtype in ("c8", "c16"):
        z = dpt.asarray(c_, dtype=dtype)
        tol = dpt.finfo(z.dtype).resolution
        assert dpt.allclose(dpt.reciprocal(z), 1 / z, atol=tol, rtol=tol, equal_nan=True)
    for dtype in ("f2", "f4", "f8"):
        vals = [np.nan, np.inf, -np.inf, 0.0, -0.0]
        X = dpt.asarray(vals, dtype=dtype)
        with np.errstate(all="ignore"):
            np.testing.assert_array_equal(dpt.asnumpy(dpt.square(X)), np.square(dpt.asnumpy(X)))
        np.testing.assert_array_equal(dpt.asnumpy(dpt.abs(X)), np.abs(dpt.asnumpy(X)))
        assert not np.signbit(dpt.asnumpy(dpt.abs(X))[-1])
    z = np.array([complex(np.nan, np.inf), complex(np.inf, np.nan), complex(3, -4), complex(-0.0, 0.0)], dtype="c16")
    np.testing.assert_array_equal(dpt.asnumpy(dpt.abs(dpt.asarray(z))), np.abs(z))


def test_abs_output_overlap_and_errors():
    # test_abs.py:122-137, 201-230
    x = dpt.reshape(dpt.arange(-12, 0, dtype="i4"), (3, 4))
    dpt.abs(x, out=x)                       # the same view: computed in place
    assert dpt.all(x == dpt.reshape(dpt.arange(12, 0, -1, dtype="i4"), (3, 4)))
    a = dpt.arange(-6, 6, dtype="i4")
    dpt.abs(a[:-1], out=a[1:])              # partial overlap: as if computed into a temporary
    assert np.array_equal(dpt.asnumpy(a), np.concatenate([[-6], np.abs(np.arange(-6, 5))]).astype("i4"))
    x = dpt.ones(5, dtype="f4")
    with pytest.raises(TypeError):
        dpt.abs(x, out=np.empty(5, dtype="f4"))
    with pytest.raises(ValueError):
        dpt.abs(x, out=dpt.empty(6, dtype="f4"))
    with pytest.raises(ValueError):
        dpt.abs(x, out=dpt.empty(5, dtype="i4"))
    ro = dpt.empty(5, dtype="f4")
    ro.flags["W"] = False
    with pytest.raises(ValueError):
        dpt.abs(x, out=ro)
    with pytest.raises(TypeError):
        dpt.abs([1.0, -2.0])


@pytest.mark.parametrize("dt1", NO_COMPLEX[1:])
@pytest.mark.parametrize("dt2", ["i1", "u2", "i8", "f4"])
def test_power_dtype_matrix_and_inplace(dt1, dt2):
    # test_pow.py:47-130
    ar1, ar2 = dpt.full(20, 2, dtype=dt1), dpt.full(20, 3, dtype=dt2)
    r = dpt.pow(ar1, ar2)
    want = np.power(np.full(1, 2, dtype=dt1), np.full(1, 3, dtype=dt2))
    assert r.dtype == want.dtype and dpt.all(r == 8)
    if np.can_cast(dt2, dt1, casting="same_kind"):   # the right operand is cast to the left one's dtype
        ar1 **= ar2
        assert dpt.all(ar1 == 8)
    else:
        with pytest.raises(ValueError):
            ar1 **= ar2
