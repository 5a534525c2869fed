"""Special values (NaN, infinities, signed zeros, ones) through every floating elementwise function,
against NumPy: the cases the reference pins function by function in
dpnp/tests/tensor/elementwise/test_{abs,angle,atan2,cbrt,complex,copysign,exp,exp2,expm1,floor_ceil_trunc,
hyperbolic,hypot,isfinite,isinf,isnan,log,log10,log1p,log2,logaddexp,nextafter,reciprocal,rsqrt,signbit,sqrt,
square,trigonometric}.py (the test_*special_cases* and test_*special_values* functions)."""
import itertools
import warnings

import numpy as np
import pytest

import dpnp_amd.tensor as dpt
from tests.helpers import dev, host

pytestmark = pytest.mark.gpu

SPECIAL = [np.nan, np.inf, -np.inf, 0.0, -0.0, 1.0, -1.0, 0.5, -0.5, 2.0, -2.0, 100.0, -100.0]


def check_against_numpy(got, want, tol_eps=8):
    """Same NaN places, same infinities with their signs, same signs of zeros, finite values close."""
    assert got.dtype == want.dtype and got.shape == want.shape
    if got.dtype.kind == "c":
        check_against_numpy(got.real.copy(), want.real.copy(), tol_eps)
        check_against_numpy(got.imag.copy(), want.imag.copy(), tol_eps)
        return
    if got.dtype.kind != "f":
        np.testing.assert_array_equal(got, want)
        return
    np.testing.assert_array_equal(np.isnan(got), np.isnan(want))
    inf = np.isinf(want)
    np.testing.assert_array_equal(got[inf], want[inf])
    zero = want == 0
    np.testing.assert_array_equal(got[zero], want[zero])
    np.testing.assert_array_equal(np.signbit(got[zero]), np.signbit(want[zero]))
    fin = np.isfinite(want) & ~zero
    eps = np.finfo(got.dtype).eps
    assert (np.abs(got[fin].astype("f8") - want[fin].astype("f8")) <= tol_eps * eps * np.abs(want[fin].astype("f8"))).all()


UNARY = ["abs", "negative", "square", "sqrt", "rsqrt", "cbrt", "exp", "exp2", "expm1", "log", "log2", "log10", "log1p",
         "sin", "cos", "tan", "asin", "acos", "atan", "sinh", "cosh", "tanh", "asinh", "acosh", "atanh", "floor", "ceil",
         "trunc", "round", "sign", "reciprocal", "isnan", "isinf", "isfinite", "signbit"]
NP_NAME = {"asin": "arcsin", "acos": "arccos", "atan": "arctan", "asinh": "arcsinh", "acosh": "arccosh",
           "atanh": "arctanh", "rsqrt": None, "round": "rint"}


@pytest.mark.parametrize("dt", ["f2", "f4", "f8"])
@pytest.mark.parametrize("name", UNARY)
def test_unary_real_special_values(name, dt):
    x = np.array(SPECIAL, dtype=dt)
    got = host(getattr(dpt, name)(dev(x)))
    with np.errstate(all="ignore"), warnings.catch_warnings():
        warnings.simplefilter("ignore")
        if name == "rsqrt":
            want = (1 / np.sqrt(x.astype("f8" if dt != "f8" else np.longdouble))).astype(dt)
        else:
            wide = x.astype("f8") if dt == "f2" and name not in ("isnan", "isinf", "isfinite", "signbit") else x
            want = getattr(np, NP_NAME.get(name, name))(wide)
            want = want.astype(dt) if want.dtype.kind == "f" else want
    # strided and reversed views take other kernels
    got_rev = host(getattr(dpt, name)(dev(x)[::-1]))
    check_against_numpy(got, want, 8 if dt != "f2" else 4)
    check_against_numpy(got_rev, want[::-1], 8 if dt != "f2" else 4)


BINARY = ["atan2", "hypot", "copysign", "nextafter", "logaddexp", "maximum", "minimum", "divide", "multiply", "add",
          "subtract", "pow"]


@pytest.mark.parametrize("dt", ["f2", "f4", "f8"])
@pytest.mark.parametrize("name", BINARY)
def test_binary_real_special_value_pairs(name, dt):
    pairs = np.array(list(itertools.product(SPECIAL, repeat=2)), dtype=dt)
    a, b = pairs[:, 0].copy(), pairs[:, 1].copy()
    got = host(getattr(dpt, name)(dev(a), dev(b)))
    with np.errstate(all="ignore"), warnings.catch_warnings():
        warnings.simplefilter("ignore")
        np_name = {"atan2": "arctan2", "pow": "power"}.get(name, name)
        if dt == "f2" and name not in ("nextafter", "copysign", "maximum", "minimum"):
            want = getattr(np, np_name)(a.astype("f4"), b.astype("f4")).astype(dt)
        else:
            want = getattr(np, np_name)(a, b)
    if name == "nextafter":
        # equal operands give the second one, sign of a zero included (test_nextafter.py:93-115); NumPy's float16
        # loop hands back the first
        want = np.where(a == b, b, want)
    if name in ("maximum", "minimum"):
        # NaN from either operand; the sign of a zero result is that of the first operand when both are zeros
        np.testing.assert_array_equal(np.isnan(got), np.isnan(want))
        ok = ~np.isnan(want)
        np.testing.assert_array_equal(got[ok], want[ok])
        return
    check_against_numpy(got, want, 8 if dt != "f2" else 4)


def test_atan2_quadrants_of_zeros_and_infinities():
    # test_atan2.py:88-505, the 26 cases of the array API specification
    pi = np.pi
    cases = [((0.5, 1, 2, np.inf), (0.0,), pi / 2), ((0.5, 1, 2, np.inf), (-0.0,), pi / 2),
             ((0.0,), (0.5, 1, 2, np.inf), 0.0), ((0.0,), (0.0,), 0.0), ((0.0,), (-0.0,), pi),
             ((0.0,), (-0.5, -1, -2, -np.inf), pi), ((-0.0,), (0.5, 1, 2, np.inf), -0.0), ((-0.0,), (0.0,), -0.0),
             ((-0.0,), (-0.0,), -pi), ((-0.0,), (-0.5, -1, -2, -np.inf), -pi), ((-0.5, -1, -2, -np.inf), (0.0,), -pi / 2),
             ((-0.5, -1, -2, -np.inf), (-0.0,), -pi / 2), ((0.5, 1, 100), (np.inf,), 0.0), ((0.5, 1, 100), (-np.inf,), pi),
             ((-0.5, -1, -100), (np.inf,), -0.0), ((-0.5, -1, -100), (-np.inf,), -pi), ((np.inf,), (0.5, -1, 100), pi / 2),
             ((-np.inf,), (0.5, -1, 100), -pi / 2), ((np.inf,), (np.inf,), pi / 4), ((np.inf,), (-np.inf,), 3 * pi / 4),
             ((-np.inf,), (np.inf,), -pi / 4), ((-np.inf,), (-np.inf,), -3 * pi / 4)]
    for dt in ("f2", "f4", "f8"):
        for x1, x2, want in cases:
            got = host(dpt.atan2(dev(np.array(x1, dtype=dt)), dev(np.array(x2, dtype=dt))))
            assert (np.abs(got.astype("f8") - want) <= 8 * np.finfo(dt).eps).all(), (dt, x1, x2, got)
            if want == 0:
                assert (np.signbit(got) == np.signbit(want)).all(), (dt, x1, x2, got)
        nan = host(dpt.atan2(dev(np.array([np.nan, np.nan, 1], dt)), dev(np.array([np.nan, 1, np.nan], dt))))
        assert np.isnan(nan).all()


def test_copysign_nextafter_signs():
    # test_copysign.py:94-110, test_nextafter.py:80-118
    x1 = dev(np.array([1.0, 0.0, np.nan, np.nan], "f4"))
    y1 = dev(np.array([-1.0, -0.0, -np.nan, -1], "f4"))
    x2 = dev(np.array([-1.0, -0.0, -np.nan, -np.nan], "f4"))
    y2 = dev(np.array([0.0, 1.0, np.nan, 1.0], "f4"))
    assert host(dpt.signbit(dpt.copysign(x1, y1))).all() and host(dpt.signbit(dpt.copysign(x2, y1))).all()
    assert not host(dpt.signbit(dpt.copysign(x2, y2))).any() and not host(dpt.signbit(dpt.copysign(x1, y2))).any()
    for dt in ("f2", "f4", "f8"):
        a = dev(np.array([-0.0, 0.0, -0.0, 0.0], dt))
        b = np.array([0.0, -0.0, -0.0, 0.0], dt)
        y = host(dpt.nextafter(a, dev(b)))
        assert (y == 0).all() and (np.signbit(y) == np.signbit(b)).all()
        n = host(dpt.nextafter(dev(np.array([2.0, np.nan, np.nan], dt)), dev(np.array([np.nan, 2.0, np.nan], dt))))
        assert np.isnan(n).all()


CPLX_GRID = [complex(*v) for v in itertools.product([np.nan, np.inf, -np.inf, 0.0, -0.0, 1.0, -1.0], repeat=2)]


@pytest.mark.parametrize("dt", ["c8", "c16"])
@pytest.mark.parametrize("name", ["exp", "sqrt", "conj", "real", "imag", "abs", "negative", "square", "isnan", "isinf",
                                  "isfinite", "proj"])
def test_complex_special_value_grid(name, dt):
    # test_exp.py:191-210, test_sqrt.py:129-160, test_complex.py:187-215, test_abs.py:163-190
    z = np.array(CPLX_GRID, dtype=dt)
    got = host(getattr(dpt, name)(dev(z)))
    with np.errstate(all="ignore"), warnings.catch_warnings():
        warnings.simplefilter("ignore")
        if name == "proj":
            want = np.where(np.isinf(z.real) | np.isinf(z.imag), np.inf + 1j * np.copysign(0.0, z.imag), z).astype(dt)
        else:
            want = getattr(np, {"conj": "conjugate"}.get(name, name))(z)
    if name == "square":
        ok = np.isfinite(want.real) & np.isfinite(want.imag)
        np.testing.assert_allclose(got[ok], want[ok], rtol=8 * np.finfo(dt).eps)
        return
    tol = 8 * np.finfo(dt).resolution
    if got.dtype.kind == "c":
        np.testing.assert_allclose(got.real, want.real, atol=tol, rtol=tol, equal_nan=True)
        np.testing.assert_allclose(got.imag, want.imag, atol=tol, rtol=tol, equal_nan=True)
    elif got.dtype.kind == "f":
        np.testing.assert_allclose(got, want, atol=tol, rtol=tol, equal_nan=True)
    else:
        np.testing.assert_array_equal(got, want)


INF, NAN = np.inf, np.nan
C_NAN = complex(NAN, NAN)
CIS_1 = complex(np.cos(1.0), np.sin(1.0))

# arguments and results of test_expm1.py:97-141, test_exp2.py:97-138, test_log1p.py:102-138; exp shares the case
# tree of exp2 (exp.hpp:75-132), so the same table holds for it
KNOWN_COMPLEX = {
    "expm1": ([complex(0.0, 0.0), complex(-0.0, 0.0), complex(1.0, INF), complex(1.0, NAN), complex(INF, 0.0),
               complex(-INF, 1.0), complex(INF, 1.0), complex(-INF, INF), complex(INF, INF), complex(-INF, NAN),
               complex(INF, NAN), complex(NAN, 0.0), complex(NAN, 1.0), complex(NAN, NAN)],
              [complex(0.0, 0.0), complex(0.0, 0.0), C_NAN, C_NAN, complex(INF, 0.0), 0.0 * CIS_1 - 1.0,
               complex(INF, INF), complex(-1.0, 0.0), complex(INF, NAN), complex(-1.0, 0.0), complex(INF, NAN),
               complex(NAN, 0.0), C_NAN, C_NAN]),
    "exp2": ([complex(0.0, 0.0), complex(1.0, INF), complex(1.0, NAN), complex(INF, 0.0), complex(-INF, 1.0),
              complex(INF, 1.0), complex(-INF, INF), complex(INF, INF), complex(-INF, NAN), complex(INF, NAN),
              complex(NAN, 0.0), complex(NAN, 1.0), complex(NAN, NAN)],
             [complex(1.0, 0.0), C_NAN, C_NAN, complex(INF, 0.0), 0.0, complex(INF, INF), complex(0.0, 0.0),
              complex(INF, NAN), complex(0.0, 0.0), complex(INF, NAN), complex(NAN, 0.0), C_NAN, C_NAN]),
    "exp": ([complex(0.0, 0.0), complex(1.0, INF), complex(1.0, NAN), complex(INF, 0.0), complex(-INF, 1.0),
             complex(INF, 1.0), complex(-INF, INF), complex(INF, INF), complex(-INF, NAN), complex(INF, NAN),
             complex(NAN, 0.0), complex(NAN, 1.0), complex(NAN, NAN)],
            [complex(1.0, 0.0), C_NAN, C_NAN, complex(INF, 0.0), 0.0, complex(INF, INF), complex(0.0, 0.0),
             complex(INF, NAN), complex(0.0, 0.0), complex(INF, NAN), complex(NAN, 0.0), C_NAN, C_NAN]),
    "log1p": ([complex(-1.0, 0.0), complex(2.0, INF), complex(2.0, NAN), complex(-INF, 1.0), complex(INF, 1.0),
               complex(-INF, INF), complex(INF, INF), complex(INF, NAN), complex(NAN, 1.0), complex(NAN, INF),
               complex(NAN, NAN)],
              [complex(-INF, 0.0), complex(INF, np.pi / 2), C_NAN, complex(INF, np.pi), complex(INF, 0.0),
               complex(INF, 3 * np.pi / 4), complex(INF, np.pi / 4), complex(INF, NAN), C_NAN, complex(INF, NAN),
               C_NAN]),
}


@pytest.mark.parametrize("dt", ["c8", "c16"])
@pytest.mark.parametrize("name", sorted(KNOWN_COMPLEX))
def test_complex_known_answers_of_the_reference_tests(name, dt):
    vals, res = KNOWN_COMPLEX[name]
    with np.errstate(all="ignore"):
        want = np.asarray(res, dtype=dt)
    got = host(getattr(dpt, name)(dev(np.asarray(vals, dtype=dt))))
    tol = np.finfo(dt).resolution
    np.testing.assert_allclose(got.real, want.real, atol=tol, rtol=tol)
    np.testing.assert_allclose(got.imag, want.imag, atol=tol, rtol=tol)
    if name == "expm1":  # test_expm1.py:143-146: the real zeros are positive
        assert not np.signbit(got[:2].real).any()


@pytest.mark.parametrize("dt", ["c8", "c16"])
@pytest.mark.parametrize("name", ["sinh", "cosh", "tanh", "sin", "cos", "tan"])
def test_complex_hyperbolic_and_trigonometric_grid_follows_annex_g(name, dt):
    # the case tables of sinh.hpp:75-160, cosh.hpp:75-150, tanh.hpp:75-135 are those of C99 Annex G, which
    # NumPy's complex loops follow too; where the standard leaves a sign open only the magnitude is compared
    z = np.array(CPLX_GRID, dtype=dt)
    got = host(getattr(dpt, name)(dev(z)))
    with np.errstate(all="ignore"), warnings.catch_warnings():
        warnings.simplefilter("ignore")
        want = getattr(np, name)(z)
    tol = 8 * np.finfo(dt).resolution
    for g, w in ((got.real, want.real), (got.imag, want.imag)):
        np.testing.assert_array_equal(np.isnan(g), np.isnan(w))
        ok = ~np.isnan(w)
        np.testing.assert_allclose(np.abs(g[ok]), np.abs(w[ok]), atol=tol, rtol=tol)
    # signs are compared where the argument is finite
    fin = np.isfinite(z.real) & np.isfinite(z.imag)
    np.testing.assert_array_equal(np.signbit(got.real[fin]), np.signbit(want.real[fin]))
    np.testing.assert_array_equal(np.signbit(got.imag[fin]), np.signbit(want.imag[fin]))


@pytest.mark.parametrize("dt", ["c8", "c16"])
@pytest.mark.parametrize("name", ["exp2", "expm1", "log1p", "log2", "log10"])
def test_complex_exponentials_and_logarithms_on_finite_arguments(name, dt):
    # test_exp2.py:56-88, test_expm1.py:56-85, test_log1p.py:56-87, test_log2.py:56-87, test_log10.py:56-87
    rng = np.random.default_rng(11)
    z = (rng.uniform(-3, 3, 4099) + 1j * rng.uniform(-3, 3, 4099)).astype(dt)
    z[:64] *= 0.01  # the small-argument branch of log1p
    got = host(getattr(dpt, name)(dev(z)))
    assert got.dtype == z.dtype
    z16 = z.astype("c16")
    want = {"exp2": lambda v: np.exp(v * np.log(2.0)), "expm1": lambda v: np.exp(v) - 1, "log1p": lambda v: np.log(1 + v),
            "log2": lambda v: np.log(v) / np.log(2.0), "log10": lambda v: np.log(v) / np.log(10.0)}[name](z16)
    if name in ("expm1", "log1p"):
        small = np.abs(z16) < 0.1
        want[small] = getattr(np, name)(z16[small])
    tol = 8 * np.finfo(dt).resolution
    np.testing.assert_allclose(got, want.astype(dt), atol=tol, rtol=tol)


INVERSE = {"asin": "arcsin", "acos": "arccos", "atan": "arctan", "asinh": "arcsinh", "acosh": "arccosh",
           "atanh": "arctanh"}


@pytest.mark.parametrize("dt", ["c8", "c16"])
@pytest.mark.parametrize("name", sorted(INVERSE))
def test_complex_inverse_functions_with_nan_and_infinite_parts(name, dt):
    # complex_math.hpp:57-262 and acosh.hpp:76-105 spell out the Annex G results for NaN and infinite parts; NumPy's
    # loops give the same table.  Signs that the standard leaves open ("opt(+-)") are not compared.
    z = np.array(CPLX_GRID, dtype=dt)
    got = host(getattr(dpt, name)(dev(z)))
    with np.errstate(all="ignore"), warnings.catch_warnings():
        warnings.simplefilter("ignore")
        want = getattr(np, INVERSE[name])(z)
    if name == "acosh":
        # acosh(+-0 + NaN j) = NaN +- pi/2 j in the reference (cacos gives pi/2 + NaN j there, test_hyperbolic.py:207-221);
        # NumPy has NaN in both parts
        at = (z.real == 0) & np.isnan(z.imag)
        want.imag[at] = np.pi / 2
    tol = 8 * np.finfo(dt).resolution
    for g, w in ((got.real, want.real), (got.imag, want.imag)):
        np.testing.assert_array_equal(np.isnan(g), np.isnan(w))
        ok = ~np.isnan(w)
        np.testing.assert_allclose(np.abs(g[ok]), np.abs(w[ok]), atol=tol, rtol=tol)
    signed = ~(np.isnan(z.real) | np.isnan(z.imag))
    if name in ("atan", "atanh"):
        # beyond 1/eps the reference returns 0 + i copysign(pi/2, y) for atanh whatever the sign of x
        # (complex_math.hpp:222-227), and the mirrored value for atan
        big = np.isinf(z.real) | np.isinf(z.imag)
        zero_part = got.real if name == "atanh" else got.imag
        assert not np.signbit(zero_part[signed & big]).any() and (zero_part[signed & big] == 0).all()
        signed &= ~big
    np.testing.assert_array_equal(np.signbit(got.real[signed]), np.signbit(want.real[signed]))
    np.testing.assert_array_equal(np.signbit(got.imag[signed]), np.signbit(want.imag[signed]))


@pytest.mark.parametrize("dt", ["c8", "c16"])
def test_acosh_of_zero_plus_nan(dt):
    # test_hyperbolic.py:207-221: acosh(+-0 + NaN j) = NaN +- pi/2 j
    y = host(dpt.acosh(dev(np.array([complex(+0.0, np.nan), complex(-0.0, np.nan)], dtype=dt))))
    assert np.isnan(y.real).all()
    np.testing.assert_allclose(np.abs(y.imag), np.pi / 2, atol=1e-6)


@pytest.mark.parametrize("dt", ["c8", "c16"])
@pytest.mark.parametrize("name", sorted(INVERSE))
def test_complex_inverse_functions_of_large_arguments(name, dt):
    # test_hyperbolic.py:222-305, test_trigonometric.py:240-320: arguments around the switch to the logarithmic form,
    # in all four quadrants
    thr1 = 1 / np.finfo(dt).eps
    thr2 = np.sqrt(thr1) / 2
    base = [complex(4e7, 1.0), complex(9e7, 1.0), complex(1e8, 1.0), complex(4.45712982e8, 1.0), complex(thr1, 1.0),
            complex(thr2, 1.0), complex(np.nextafter(thr1, np.inf), 1.0), complex(np.nextafter(thr2, np.inf), 1.0),
            complex(1.0, 4e7), complex(1.0, thr2 * 1.01), complex(3e4, 4e4), complex(2e30, 1e30)]
    x = np.array([complex(sr * v.real, si * v.imag) for v in base for sr in (1, -1) for si in (1, -1)], dtype=dt)
    got = host(getattr(dpt, name)(dev(x)))
    want = getattr(np, INVERSE[name])(x)
    tol = 8 * np.finfo(dt).resolution
    assert not np.isinf(got.real).any() and not np.isinf(got.imag).any()
    np.testing.assert_allclose(got, want, atol=tol, rtol=tol)


def test_comparisons_with_python_ints_beyond_the_dtype():
    # test_greater.py:172-200, test_less.py:172-200 (and _equal forms)
    x = dpt.zeros(10, dtype="i4")
    big = 2**40
    for fn, pos, neg in ((dpt.greater, False, True), (dpt.greater_equal, False, True), (dpt.less, True, False),
                         (dpt.less_equal, True, False)):
        assert (host(fn(x, big)) == pos).all() and (host(fn(x, -big)) == neg).all()
        assert (host(fn(big, x)) == (not pos)).all() and (host(fn(-big, x)) == (not neg)).all()
    assert not host(dpt.equal(x, big)).any() and host(dpt.not_equal(x, big)).all()
    b = dpt.asarray(np.full(2**16 + 3, True))
    assert not host(dpt.bitwise_invert(b)).any() and host(dpt.logical_not(dpt.bitwise_invert(b))).all()
