"""Pins the CPU oracle: reference known answers, closed forms, brute force, mpmath.
Runs without a GPU.

Oracle function -> what pins it here (none of the pins calls NumPy for the rule under test):
  binary add/subtract/multiply/bitwise_*  test_integer_ops_wrap_like_python_ints, test_add_ones_is_two
  binary floor_divide, remainder (ints)   test_integer_functors_brute_force_int8 (scalar C-semantics
                                          transcription of floor_divide.hpp:69-86, remainder.hpp:66-83)
  binary floor_divide, remainder (floats) test_float_floor_divide_and_remainder_rules (Fractions; the
                                          special cases of test_floor_divide.py:109-147, test_remainder.py:138-152)
  binary bitwise_left/right_shift         test_integer_functors_brute_force_int8 (+ uint8),
                                          test_shift_range_known_answer (test_bitwise_*_shift.py:107-117)
  binary pow (ints)                       test_integer_functors_brute_force_int8 (pow.hpp:72-92)
  binary fmod (ints)                      test_integer_functors_brute_force_int8 (fmod.hpp:52-62)
  unary sign                              test_sign_rules (sign.hpp:73-110, test_sign.py:61-101)
  unary round                             test_round_conj_parts_proj_rules (test_round.py:107-122)
  comparisons (incl. int64/uint64)        test_mixed_int64_uint64_comparisons_are_exact
  maximum / minimum                       test_maximum_minimum_nan_rule
  promote_binary                          test_promotion_matches_numpy_result_type,
                                          test_promotion_with_acceptance_hooks
  black_scholes                           test_black_scholes_against_the_textbook_formula_in_40_digits (mpmath ncdf)
  fmax / fmin / <= / >= of complex        test_complex_fmax_fmin_ordering_brute_force (scalar transcription of
                                          math_utils.hpp:73-95 and fmax.hpp:57-70 on a grid with NaN parts)
  binary pow (floats)                     test_float_pow_special_values (C99 F.10.4.4 written out; the reference's
                                          list, test_binary_ufuncs.py:972-994)
  var_around_mean                         test_var_around_mean_identities_and_docstring_values (exact
                                          rational arithmetic, var(z) = var(Re z) + var(Im z), the shift
                                          identity, dpnp_iface_statistics.py:1815-1826,1625-1634)
  cast, where, reductions, collapse       the tests of those names below
"""
from fractions import Fraction
import itertools
import json
import math
import os
import warnings

import numpy as np
import pytest

from oracle import oracle as orc
from oracle.oracle_c import OracleC

GOLD = json.load(open(os.path.join(os.path.dirname(__file__), "golden", "reference_known_answers.json")))
ALL = [d.str[1:] if d.kind != "b" else "?" for d in orc.ALL_DTYPES]


def _f(v):
    return float(v) if isinstance(v, str) else v


# ---- elementwise -----------------------------------------------------------------------------
@pytest.mark.parametrize("dt", ALL)
def test_add_ones_is_two(dt):
    # dpnp/tests/tensor/elementwise/test_add.py:49-88: ones + ones == 2 (bool: True)
    a = np.ones(7, dtype=dt)
    r = orc.binary("add", a, a)
    assert r.dtype == a.dtype
    assert (r == np.full(7, 2, dtype=dt)).all() if dt != "?" else r.all()


@pytest.mark.parametrize("dt", ["i1", "u1", "i2", "u2"])
@pytest.mark.parametrize("op", ["add", "subtract", "multiply", "bitwise_and", "bitwise_or", "bitwise_xor"])
def test_integer_ops_wrap_like_python_ints(dt, op):
    info = np.iinfo(dt)
    vals = np.array([info.min, info.min + 1, -1 if info.min < 0 else 1, 0, 1, 2, 3, 7, info.max - 1, info.max],
                    dtype=dt)
    a, b = np.meshgrid(vals, vals)
    r = orc.binary(op, a, b)
    py = {"add": int.__add__, "subtract": int.__sub__, "multiply": int.__mul__, "bitwise_and": int.__and__,
          "bitwise_or": int.__or__, "bitwise_xor": int.__xor__}[op]
    bits = 8 * np.dtype(dt).itemsize
    for x, y, z in zip(a.ravel(), b.ravel(), r.ravel()):
        want = py(int(x), int(y)) & ((1 << bits) - 1)
        if info.min < 0 and want >= (1 << (bits - 1)):
            want -= 1 << bits
        assert int(z) == want


def test_floor_divide_and_remainder_integer_rules():
    # floor_divide.hpp:69-86, remainder.hpp: x // 0 == 0, x % 0 == 0, Python floor semantics otherwise
    vals = np.array([-7, -3, -1, 0, 1, 3, 7], dtype="i4")
    a, b = np.meshgrid(vals, vals)
    q, r = orc.binary("floor_divide", a, b), orc.binary("remainder", a, b)
    for x, y, qq, rr in zip(a.ravel(), b.ravel(), q.ravel(), r.ravel()):
        if y == 0:
            assert qq == 0 and rr == 0
        else:
            assert qq == int(x) // int(y) and rr == int(x) % int(y)


# Scalar transcriptions of the reference's integer functors in C semantics (division truncates
# towards zero, `%` takes the dividend's sign, results wrap to the operand width).  They are
# written from the functor text, branch by branch, and share no code with the oracle.
def _wrap(v, bits, signed):
    v &= (1 << bits) - 1
    return v - (1 << bits) if signed and v >= (1 << (bits - 1)) else v


def _c_div(a, b):
    q = abs(a) // abs(b)
    return q if (a < 0) == (b < 0) else -q


def _c_mod(a, b):
    return a - _c_div(a, b) * b


def _functor_right_shift(a, b, bits, signed):  # bitwise_right_shift.hpp:88-105
    if not signed:
        return (a >> b) if b < bits else 0
    return 0 if b < 0 else ((a >> b) if b < bits else (-1 if a < 0 else 0))


def _functor_left_shift(a, b, bits, signed):   # bitwise_left_shift.hpp:88-103
    if not signed:
        return _wrap(a << b, bits, False) if b < bits else 0
    return 0 if b < 0 else (_wrap(a << b, bits, True) if b < bits else 0)


def _functor_pow(a, b, bits, signed):          # pow.hpp:72-92
    if signed and b < 0:
        return 0
    res = 1
    if a == 1 or b == 0:
        return res
    while b > 0:
        if b & 1:
            res = _wrap(res * a, bits, signed)
        b >>= 1
        a = _wrap(a * a, bits, signed)
    return res


def _functor_floor_divide(a, b, bits, signed):  # floor_divide.hpp:69-86
    if b == 0:
        return 0
    if not signed:
        return a // b
    div, mod = _c_div(a, b), _c_mod(a, b)
    return _wrap(div - int(mod != 0 and ((mod < 0) != (b < 0))), bits, True)


def _functor_remainder(a, b, bits, signed):     # remainder.hpp:66-83
    if b == 0:
        return 0
    out = _c_mod(a, b)
    if signed and out != 0 and ((a < 0) != (b < 0)):
        out += b
    return _wrap(out, bits, signed)


def _functor_fmod(a, b, bits, signed):          # dpnp/backend/kernels/elementwise_functions/fmod.hpp:52-62
    return 0 if b == 0 else _c_mod(a, b)


@pytest.mark.parametrize("dt", ["i1", "u1"])
def test_integer_functors_brute_force_int8(dt):
    info = np.iinfo(dt)
    signed = info.min < 0
    vals = np.arange(info.min, info.max + 1).astype(dt)
    a, b = np.meshgrid(vals, vals, indexing="ij")
    for op, fn in (("bitwise_right_shift", _functor_right_shift), ("bitwise_left_shift", _functor_left_shift),
                   ("pow", _functor_pow), ("floor_divide", _functor_floor_divide),
                   ("remainder", _functor_remainder), ("fmod", _functor_fmod)):
        got = orc.binary(op, a, b)
        assert got.dtype == np.dtype(dt)
        want = np.array([[fn(int(x), int(y), 8, signed) for y in vals] for x in vals], dtype=dt)
        bad = np.argwhere(got != want)
        assert bad.size == 0, (op, dt, [(int(vals[i]), int(vals[j]), int(got[i, j]), int(want[i, j])) for i, j in bad[:5]])


def test_integer_functors_wider_types_spot_checks():
    # the same rules at 16, 32 and 64 bits on the values where width matters
    for dt in ("i2", "u2", "i4", "u4", "i8", "u8"):
        info = np.iinfo(dt)
        bits, signed = 8 * np.dtype(dt).itemsize, info.min < 0
        vals = [info.min, info.min + 1, -3 if signed else 3, -1 if signed else 1, 0, 1, 2, 3, 7, bits - 1, bits,
                bits + 1, info.max - 1, info.max]
        a, b = np.meshgrid(np.array(vals, dtype=dt), np.array(vals, dtype=dt), indexing="ij")
        for op, fn in (("bitwise_right_shift", _functor_right_shift), ("bitwise_left_shift", _functor_left_shift),
                       ("pow", _functor_pow), ("floor_divide", _functor_floor_divide),
                       ("remainder", _functor_remainder), ("fmod", _functor_fmod)):
            got = orc.binary(op, a, b)
            for i, x in enumerate(vals):
                for j, y in enumerate(vals):
                    if signed and y == -1 and x == info.min and op in ("floor_divide", "remainder", "fmod"):
                        continue  # INT_MIN / -1 overflows in C: undefined in the reference
                    assert int(got[i, j]) == fn(x, y, bits, signed), (op, dt, x, y)


@pytest.mark.parametrize("dt", ["i1", "u1", "i2", "u2", "i4", "u4", "i8", "u8"])
def test_shift_range_known_answer(dt):
    # test_bitwise_right_shift.py:107-117, test_bitwise_left_shift.py:107-117: ones shifted by 64 are 0
    x, y = np.ones(255, dtype=dt), np.asarray(64, dtype=dt)
    assert not orc.binary("bitwise_right_shift", x, y).any()
    assert not orc.binary("bitwise_left_shift", x, y).any()


def test_float_floor_divide_and_remainder_rules():
    # floor_divide.hpp:84-86: floor of the ROUNDED quotient (1.0 // 0.1 is 10, where Python's and
    # NumPy's divmod-based rule give 9); remainder.hpp:84-96: fmod, `+= y` on a sign mismatch, a
    # zero remainder takes y's sign.  Exact rational arithmetic is the independent evaluation.
    rng = np.random.default_rng(21)
    for dt in ("f4", "f8"):
        a = rng.uniform(-50, 50, 400).astype(dt)
        b = rng.uniform(-7, 7, 400).astype(dt)
        a[:6] = [1.0, -1.0, 7.5, -7.5, 6.0, -6.0]
        b[:6] = [0.1, 0.1, 2.5, 2.5, -3.0, 3.0]
        q, r = orc.binary("floor_divide", a, b), orc.binary("remainder", a, b)
        for x, y, qq, rr in zip(a, b, q, r):
            assert float(qq) == float(math.floor(np.dtype(dt).type(x) / np.dtype(dt).type(y)))
            fx, fy = Fraction(float(x)), Fraction(float(y))
            t = fx - fy * int(fx / fy)              # C fmod: exact, truncated quotient
            if t != 0 and ((fy < 0) != (t < 0)):
                want = np.dtype(dt).type(float(t)) + np.dtype(dt).type(y)  # one rounded addition
            else:
                want = np.dtype(dt).type(float(t))
            assert float(rr) == float(want), (x, y, rr, want)
            if t == 0:
                assert np.signbit(rr) == np.signbit(y)
    assert orc.binary("floor_divide", np.array([1.0]), np.array([0.1]))[0] == 10.0
    # special cases, test_floor_divide.py:109-147 and test_remainder.py:138-152
    inf, nan = np.inf, np.nan
    x = np.array([inf, 0.0, -1.0, -1.0, inf, 1.0], dtype="f4")
    y = np.array([inf, -1.0, 0.0, inf, -1.0, nan], dtype="f4")
    q = orc.binary("floor_divide", x, y)
    assert np.isnan(q[0]) and q[1] == 0 and np.signbit(q[1]) and q[2] == -inf
    assert q[3] == 0 and np.signbit(q[3]) and q[4] == -inf and np.isnan(q[5])
    lhs = np.array([nan, inf, 0.0, -0.0, -0.0, 1.0, inf, -inf, 5.0, -5.0], dtype="f4")
    rhs = np.array([nan, inf, -0.0, 1.0, -1.0, 0.0, 1.0, -1.0, inf, inf], dtype="f4")
    r = orc.binary("remainder", lhs, rhs)
    assert np.isnan(r[[0, 1, 2, 5, 6, 7]]).all()
    assert r[3] == 0 and not np.signbit(r[3]) and r[4] == 0 and np.signbit(r[4])
    assert r[8] == 5.0 and r[9] == inf  # fmod(-5, inf) = -5, sign differs from y: -5 + inf


def test_sign_rules():
    # sign.hpp:73-110; known answers of test_sign.py:61-101
    for dt in ("i1", "i2", "i4", "i8", "f2", "f4", "f8"):
        x = np.arange(-20, 20, 1).astype(dt)
        want = [(0 < int(v)) - (int(v) < 0) for v in x]
        assert orc.unary("sign", x).tolist() == want and orc.unary("sign", x).dtype == np.dtype(dt)
    assert orc.unary("sign", np.array([0, 1, 200], dtype="u1")).tolist() == [0, 1, 1]
    f = orc.unary("sign", np.array([np.nan, -np.inf, np.inf, -0.0, 0.0], dtype="f4"))
    assert np.isnan(f[0]) and f[1:].tolist() == [-1, 1, 0, 0] and not np.signbit(f[3])
    z = np.array([3 + 4j, -5j, 0], dtype="c16")
    got = orc.unary("sign", z)
    assert got[0] == complex(0.6, 0.8) and got[1] == -1j and got[2] == 0


def test_promotion_with_acceptance_hooks():
    # dpnp/tests/tensor/elementwise/test_divide.py dtype matrix: the result dtype of divide is
    # NumPy's for every pair (int8 / uint8 is float64, not float16)
    fp_only = lambda a, b: a if (a == b and a.kind in "fc") else None  # noqa: E731
    for d1 in orc.ALL_DTYPES:
        for d2 in orc.ALL_DTYPES:
            _b1, _b2, r = orc.promote_binary(fp_only, d1, d2, accept=orc.accept_divide)
            want = np.true_divide(np.ones(1, d1), np.ones(1, d2)).dtype
            assert r == want, (d1, d2, r, want)


def test_mixed_int64_uint64_comparisons_are_exact():
    a = np.array([-1, 0, 2**62, -2**63, 2**63 - 1], dtype="i8")
    b = np.array([2**64 - 1, 0, 2**62, 2**63, 2**63 - 1], dtype="u8")
    for op, f in (("less", int.__lt__), ("greater", int.__gt__), ("equal", int.__eq__),
                  ("less_equal", int.__le__), ("greater_equal", int.__ge__), ("not_equal", int.__ne__)):
        for x, y in ((a, b), (b, a)):
            r = orc.binary(op, x, y)
            assert [bool(v) for v in r] == [f(int(p), int(q)) for p, q in zip(x, y)]


def test_bool_arithmetic_is_logical():
    t = np.array([True, True, False, False])
    u = np.array([True, False, True, False])
    assert (orc.binary("add", t, u) == (t | u)).all()
    assert (orc.binary("multiply", t, u) == (t & u)).all()
    assert (orc.binary("bitwise_and", t, u) == (t & u)).all()


def test_maximum_minimum_nan_rule():
    a = np.array([np.nan, 1.0, 2.0, np.nan], dtype="f4")
    b = np.array([1.0, np.nan, 3.0, np.nan], dtype="f4")
    assert np.isnan(orc.binary("maximum", a, b)[[0, 1, 3]]).all() and orc.binary("maximum", a, b)[2] == 3
    assert np.isnan(orc.binary("minimum", a, b)[[0, 1, 3]]).all() and orc.binary("minimum", a, b)[2] == 2


def test_exp_known_answers():
    g = GOLD["exp_powers_of_two"]
    for dt in ("f2", "f4", "f8"):
        x = (np.array(g["k"], dtype=dt) * np.dtype(dt).type(g["log2"])).astype(dt)
        tol = 8 * np.finfo(dt).resolution
        np.testing.assert_allclose(orc.unary("exp", x).astype("f8"), np.exp(x.astype("f8")), rtol=tol, atol=tol)
    s = GOLD["exp_special"]
    x = np.array([_f(v) for v in s["x"]], dtype="f8")
    want = np.array([_f(v) for v in s["expected"]], dtype="f8")
    np.testing.assert_array_equal(orc.unary("exp", x), want)


@pytest.mark.parametrize("op", ["exp", "log", "erf"])
def test_high_precision_evaluation_against_mpmath(op):
    import mpmath

    mpmath.mp.dps = 60
    rng = np.random.default_rng(5)
    x = {"exp": rng.uniform(-80, 80, 200), "log": rng.uniform(1e-30, 1e30, 200), "erf": rng.uniform(-4, 4, 200)}[op]
    f = {"exp": mpmath.exp, "log": mpmath.log, "erf": mpmath.erf}[op]
    for dt in ("f4", "f8"):
        xs = x.astype(dt)
        got = orc.unary(op, xs)
        exact = np.array([np.longdouble(mpmath.nstr(f(mpmath.mpf(float(v))), 40)) for v in xs])
        assert orc.ulp_error(got, exact).max() <= 0.5 + 1e-3  # the oracle rounds the exact value


def test_cast_rules():
    # type_utils.hpp:64-117
    assert (orc.cast(np.array([0.0, -0.0, 0.5, np.nan]), "?") == [False, False, True, True]).all()
    assert (orc.cast(np.array([-1.0, -3.7, 5.2], dtype="f4"), "u1") == [255, 253, 5]).all()
    assert (orc.cast(np.array([-1.0, 2.0**31], dtype="f8"), "u4") == [2**32 - 1, 2**31]).all()
    assert orc.cast(np.array([3 + 4j]), "f8")[0] == 3.0
    assert orc.cast(np.array([0 + 1j]), "?")[0]


def test_where_known_answer():
    g = GOLD["where_basic"]
    cond = np.array(g["cond"], dtype=bool)
    r = orc.where(cond, np.full(cond.shape, g["x1"]), np.full(cond.shape, g["x2"]))
    assert (r == np.array(g["expected"])).all()
    # truthiness of non-bool conditions: any set bit except -0.0
    assert (orc.where(np.array([0.0, -0.0, np.nan, 2.0]), np.ones(4), np.zeros(4)) == [0, 0, 1, 1]).all()


def test_black_scholes_against_the_textbook_formula_in_40_digits():
    """The oracle restates the reference example's expression tree (erf of w1, w2).  Pinned against the textbook
    form written independently of it: call = S0 Phi(d1) - K exp(-rT) Phi(d2), put = K exp(-rT) Phi(-d2) -
    S0 Phi(-d1), d1 = (ln(S0/K) + (r + sigma^2/2) T) / (sigma sqrt(T)), d2 = d1 - sigma sqrt(T), with Phi the
    normal distribution function of mpmath (ncdf) at 40 digits.  A dropped term, a wrong sign of r or a swapped
    price and strike changes the prices by far more than the bound."""
    import mpmath

    rng = np.random.default_rng(4)
    n = 200
    p, s, t = rng.uniform(10, 50, n), rng.uniform(10, 50, n), rng.uniform(1, 2, n)
    r, sigma = 0.1, 0.2
    call, put = orc.black_scholes(p, s, t, r, sigma)
    with mpmath.workdps(40):
        rr, sg = mpmath.mpf(r), mpmath.mpf(sigma)
        for i in range(n):
            s0, k, tt = mpmath.mpf(float(p[i])), mpmath.mpf(float(s[i])), mpmath.mpf(float(t[i]))
            d1 = (mpmath.log(s0 / k) + (rr + sg * sg / 2) * tt) / (sg * mpmath.sqrt(tt))
            d2 = d1 - sg * mpmath.sqrt(tt)
            disc = k * mpmath.exp(-rr * tt)
            c = s0 * mpmath.ncdf(d1) - disc * mpmath.ncdf(d2)
            q = disc * mpmath.ncdf(-d2) - s0 * mpmath.ncdf(-d1)
            scale = max(float(s0), float(k))
            assert abs(float(call[i]) - float(c)) <= 1e-13 * scale, (i, float(call[i]), float(c))
            assert abs(float(put[i]) - float(q)) <= 1e-13 * scale, (i, float(put[i]), float(q))
    # deep in and out of the money, where one of the two products dominates
    p2, s2, t2 = np.array([1.0, 1000.0, 50.0]), np.array([1000.0, 1.0, 50.0]), np.array([0.25, 0.25, 30.0])
    c2, q2 = orc.black_scholes(p2, s2, t2, r, sigma)
    assert c2[0] < 1e-100 and abs(q2[0] - (1000 * math.exp(-0.025) - 1)) < 1e-9
    assert q2[1] < 1e-100 and abs(c2[1] - (1000 - math.exp(-0.025))) < 1e-9


def test_complex_fmax_fmin_ordering_brute_force():
    """fmax / fmin of complex operands (dpnp/backend/kernels/elementwise_functions/fmax.hpp:57-70, fmin.hpp): the
    first operand is kept when the second holds a NaN or when first >= second (<=) in the order of
    math_utils.hpp:73-95.  Checked against a scalar transcription written with Python floats, on every pair of
    a grid with signed zeros, infinities and NaN parts."""
    vals = [0.0, -0.0, 1.0, -1.0, 2.5, np.inf, -np.inf, np.nan]
    grid = np.array([complex(re, im) for re in vals for im in vals], dtype="c16")

    def ge(x, y):  # greater_equal_complex
        return (x.imag >= y.imag) if x.real == y.real else (x.real > y.real and not math.isnan(x.imag) and not math.isnan(y.imag))

    def le(x, y):  # less_equal_complex
        return (x.imag <= y.imag) if x.real == y.real else (x.real < y.real and not math.isnan(x.imag) and not math.isnan(y.imag))

    a, b = np.meshgrid(grid, grid, indexing="ij")
    a, b = a.ravel(), b.ravel()
    for name, cmp in (("fmax", ge), ("fmin", le)):
        got = orc.binary(name, a, b)
        for x, y, g in zip(a, b, got):
            x, y = complex(x), complex(y)
            want = x if (math.isnan(y.real) or math.isnan(y.imag) or cmp(x, y)) else y
            same = (g.real == want.real or (math.isnan(g.real) and math.isnan(want.real))) and \
                   (g.imag == want.imag or (math.isnan(g.imag) and math.isnan(want.imag)))
            assert same and math.copysign(1, g.real) == math.copysign(1, want.real) \
                and math.copysign(1, g.imag) == math.copysign(1, want.imag), (name, x, y, g, want)
    # the ordering functions themselves, on the same grid (less_equal / greater_equal of complex arrays)
    for name, cmp in (("greater_equal", ge), ("less_equal", le)):
        got = orc.binary(name, a, b)
        assert [bool(g) for g in got] == [cmp(complex(x), complex(y)) for x, y in zip(a, b)], name


def test_float_pow_special_values():
    """Real pow is the C library's (pow.hpp:93-95: sycl::pow): the special values of C99 F.10.4.4, written out here,
    and the reference's own list (dpnp/tests/test_binary_ufuncs.py:972-994: finite and infinite bases to
    infinite exponents)."""
    inf, nan = np.inf, np.nan
    cases = [  # (x, y, pow(x, y))
        (1.0, inf, 1.0), (1.0, -inf, 1.0), (2.0, inf, inf), (2.0, -inf, 0.0), (-2.0, inf, inf), (-2.0, -inf, 0.0),
        (inf, inf, inf), (-inf, -inf, 0.0),  # the reference's list
        (0.5, inf, 0.0), (0.5, -inf, inf), (-0.5, inf, 0.0), (-1.0, inf, 1.0), (-1.0, -inf, 1.0),
        (nan, 0.0, 1.0), (nan, -0.0, 1.0), (1.0, nan, 1.0), (inf, 0.0, 1.0), (0.0, 0.0, 1.0),
        (0.0, 3.0, 0.0), (-0.0, 3.0, -0.0), (-0.0, 2.0, 0.0), (0.0, -3.0, inf), (-0.0, -3.0, -inf), (-0.0, -2.0, inf),
        (0.0, -inf, inf), (0.0, inf, 0.0),
        (-inf, 3.0, -inf), (-inf, 2.0, inf), (-inf, -3.0, -0.0), (-inf, -2.0, 0.0), (inf, -1.0, 0.0), (inf, 0.5, inf),
        (-8.0, 1.0 / 3, nan), (-2.0, 0.5, nan), (nan, 2.0, nan), (2.0, nan, nan),
        (-2.0, 3.0, -8.0), (-2.0, -2.0, 0.25), (4.0, 0.5, 2.0), (10.0, -2.0, 0.01),
    ]
    for dt in ("f4", "f8"):
        x = np.array([c[0] for c in cases], dtype=dt)
        y = np.array([c[1] for c in cases], dtype=dt)
        want = np.array([c[2] for c in cases], dtype=dt)
        with np.errstate(all="ignore"):
            got = orc.binary("pow", x, y)
        assert got.dtype == np.dtype(dt)
        for c, g, w in zip(cases, got, want):
            if math.isnan(w):
                assert math.isnan(g), c
            else:
                assert g == w and math.copysign(1, g) == math.copysign(1, w), (c, g)


# ---- reductions ----------------------------------------------------------------------------------
@pytest.mark.parametrize("dt", ALL)
def test_sum_of_ones(dt):
    for n in GOLD["sum_ones"]["n"]:
        r = orc.reduce("sum", np.ones(n, dtype=dt), 1)
        assert r == n
        assert r.dtype == orc.default_accumulation_dtype(np.dtype(dt))
    g = GOLD["sum_strided_ones"]
    assert orc.reduce("sum", np.ones(g["base_n"], dtype=dt)[slice(*g["slice"])], 1) == g["expected"]


def test_sum_known_answers():
    g = GOLD["sum_gh1391"]
    a = np.arange(g["arange"], dtype="i4").reshape(g["shape"]).transpose(g["permute"])
    assert (orc.reduce("sum", a, 1) == np.array(g["expected"])).all()
    g = GOLD["sum_axis0_3x4x5"]
    x = np.arange(g["arange"], dtype="f4").reshape(g["shape"])
    assert (orc.reduce("sum", np.moveaxis(x, 0, -1), 1) == np.array(g["expected"], dtype="f4")).all()
    g = GOLD["sum_flip_axis2_3x4x5"]
    assert (orc.reduce("sum", np.flip(x, 2), 1) == np.array(g["expected"], dtype="f4")).all()
    g = GOLD["sum_bool_dtype_gh1944"]
    for dt in g["dtypes"]:
        assert bool(orc.reduce("sum", np.array(g["input"], dtype=dt), 1, out_dtype="?")) is True
    assert orc.reduce("sum", np.empty(0, dtype="u1"), 1) == 0
    assert orc.reduce("prod", np.empty(0, dtype="f4"), 1) == 1


def test_integer_sum_wraps():
    x = np.full(300, 127, dtype="i1")
    assert orc.reduce("sum", x, 1, out_dtype="i1") == np.int8((300 * 127) % 256 - 256 if (300 * 127) % 256 > 127 else (300 * 127) % 256)
    assert orc.reduce("sum", x, 1) == 300 * 127


def test_float_sum_is_exact_sum_rounded():
    rng = np.random.default_rng(0)
    x = rng.uniform(-1, 1, 4097).astype("f4")
    assert orc.reduce("sum", x, 1) == np.float32(math.fsum(x.astype("f8")))


def test_max_min_known_answers():
    g = GOLD["max_axis0_arange"]
    x = np.arange(g["arange"]).reshape(g["shape"])
    assert (orc.reduce("max", np.moveaxis(x, 0, -1), 1) == x[-1]).all()
    for c in GOLD["max_min_nan"]["cases"]:
        v = np.array([_f(e) for e in c["values"]], dtype=c["dtype"])
        assert np.isnan(orc.reduce("max", v, 1)) and np.isnan(orc.reduce("min", v, 1))
    z = np.arange(4, dtype="c8")
    z[0] = complex(np.nan, 0)
    assert np.isnan(orc.reduce("max", z, 1)) and np.isnan(orc.reduce("min", z, 1))
    with pytest.raises(ValueError):
        orc.reduce("max", np.empty((3, 0)), 1)


def test_argmax_known_answers():
    g = GOLD["argmax_2x3"]
    x = np.array(g["input"], dtype=g["dtype"])
    assert orc.argreduce("argmax", x, 2) == g["argmax_flat"]
    assert (orc.argreduce("argmax", x.T, 1) == g["argmax_axis0"]).all()
    assert (orc.argreduce("argmax", x, 1) == g["argmax_axis1"]).all()
    assert orc.argreduce("argmax", np.full(3, np.iinfo("i4").min, dtype="i4"), 1) == 0
    assert orc.argreduce("argmin", np.full(3, np.iinfo("i4").max, dtype="i4"), 1) == 0
    for idx in range(4):
        for dt in ("f4", "c8"):
            x = np.arange(4, dtype=dt)
            x[idx] = np.nan
            assert orc.argreduce("argmax", x, 1) == idx and orc.argreduce("argmin", x, 1) == idx
    x = np.arange(4, dtype="c8")
    x[2] = complex(0, np.nan)
    assert orc.argreduce("argmax", x, 1) == 2 and orc.argreduce("argmin", x, 1) == 2


def test_argmax_brute_force_all_patterns():
    vals = [0.0, 1.0, -1.0, np.nan, np.inf, -np.inf]
    for n in (1, 2, 3, 4):
        for combo in itertools.product(vals, repeat=n):
            x = np.array(combo, dtype="f4")
            nan = [i for i, v in enumerate(combo) if v != v]
            want_max = nan[0] if nan else max(range(n), key=lambda i: (combo[i], -i))
            want_min = nan[0] if nan else min(range(n), key=lambda i: (combo[i], i))
            assert orc.argreduce("argmax", x, 1) == want_max
            assert orc.argreduce("argmin", x, 1) == want_min
            assert orc.argreduce("argmax", x, 1) == np.argmax(x)  # NumPy: first NaN, first maximum


def test_mean_var_known_answers():
    g = GOLD["mean_3x3"]
    x = np.arange(g["arange"], dtype=g["dtype"]).reshape(g["shape"])
    assert orc.mean(x, 2) == g["mean"]
    assert (orc.mean(x.T, 1) == g["mean_axis0"]).all() and (orc.mean(x, 1) == g["mean_axis1"]).all()
    g = GOLD["var_3x3"]
    np.testing.assert_allclose(orc.var(x, 2), g["var"], rtol=1e-6)
    np.testing.assert_allclose(orc.var(x, 2, correction=3), g["var_corr3"], rtol=1e-6)
    np.testing.assert_allclose(orc.var(x.T, 1), g["var_axis0"], rtol=1e-6)
    np.testing.assert_allclose(orc.var(x.T, 1, correction=1), g["var_axis0_corr1"], rtol=1e-6)
    np.testing.assert_allclose(orc.var(x, 1), g["var_axis1"], rtol=1e-6)
    np.testing.assert_allclose(orc.var(x, 1, correction=1), g["var_axis1_corr1"], rtol=1e-6)
    # test_tensor_statistical_functions.py:229-241: N - correction <= 0 gives NaN
    assert np.isnan(orc.var(x, 2, correction=9)) and np.isnan(orc.var(x, 1, correction=3)).all()
    assert orc.mean(np.arange(4, dtype="i4"), 1).dtype == np.dtype("f8")


# ---- stride collapsing ----------------------------------------------------------------------------------
def random_view_strides(rng, shape):
    """Element strides of a random view with `shape`: permuted base layout, steps of +-1/+-2,
    some dims broadcast (stride 0)."""
    nd = len(shape)
    perm = rng.permutation(nd)
    big = [2 * s + 1 for s in shape]
    base = np.arange(int(np.prod(big))).reshape([big[p] for p in perm])
    v = np.transpose(base, np.argsort(perm))
    v = v[tuple(slice(None, None, int(st)) for st in rng.choice([1, 2, -1, -2], nd))]
    v = v[tuple(slice(0, s) for s in shape)]
    for d in range(nd):
        if rng.random() < 0.2:
            one = v[tuple(slice(0, 1) if i == d else slice(None) for i in range(nd))]
            v = np.broadcast_to(one, shape)
    assert v.shape == tuple(shape)
    return [st // base.itemsize for st in v.strides]


def test_collapse_keeps_the_address_set():
    rng = np.random.default_rng(11)
    for _ in range(300):
        nd = int(rng.integers(1, 5))
        shape = [int(s) for s in rng.integers(1, 5, nd)]
        strides = [random_view_strides(rng, shape) for _k in range(int(rng.integers(1, 4)))]
        for keep in (False, True):
            sh, st, off = orc.collapse(shape, strides, keep_order=keep)
            assert orc.address_tuples(sh, st, off) == orc.address_tuples(shape, strides)
            assert len(sh) <= nd


def test_collapse_merges_contiguous_and_reversed():
    assert orc.collapse([3, 4, 5], [[20, 5, 1], [20, 5, 1]])[0] == [60]
    sh, st, off = orc.collapse([3, 4], [[-4, -1]])
    assert sh == [12] and st == [[1]] and off == [-11]
    sh, st, off = orc.collapse([8192, 4096], [[8192, 2], [0, 1], [4096, 1]])
    assert sh == [8192, 4096] and st == [[8192, 2], [0, 1], [4096, 1]]
    # keep_order: only neighbours merge, nothing is reordered or reversed
    sh, st, off = orc.collapse([3, 4], [[1, 3]], keep_order=True)
    assert sh == [3, 4] and st == [[1, 3]]


# ---- promotion --------------------------------------------------------------------------------------------
def test_promotion_matches_numpy_result_type():
    # dpnp/tests/tensor/elementwise/test_add.py:62-65: result dtype of add == numpy.result_type
    same = lambda a, b: a if a == b else None  # noqa: E731  (add has all 14 same-dtype pairs)
    for d1 in orc.ALL_DTYPES:
        for d2 in orc.ALL_DTYPES:
            b1, b2, r = orc.promote_binary(same, d1, d2)
            assert r == np.result_type(d1, d2), (d1, d2, r)


# ---- C restatement vs NumPy restatement ----------------------------------------------------------------------
@pytest.fixture(scope="module")
def oc():
    return OracleC()


@pytest.mark.parametrize("n", [1, 100, 255, 256, 257, 2048, 16384, 16385, 100003, 1 << 20])
def test_c_port_matches_numpy_oracle(oc, n):
    rng = np.random.default_rng(n)
    a = rng.uniform(-1, 1, n).astype("f4")
    b = rng.uniform(-1, 1, n).astype("f4")
    assert np.array_equal(oc.add(a, b), orc.binary("add", a, b))
    exact = orc.reduce("sum", a, 1)
    assert abs(float(oc.sum(a)) - float(exact)) <= 1e-5 * max(abs(float(exact)), float(np.abs(a).sum()) * 1e-2)
    x = rng.standard_normal(n).astype("f4")
    x[rng.integers(0, n, max(n // 100, 1))] = x.max()
    assert oc.argmax(x) == orc.argreduce("argmax", x, 1)
    assert oc.argmin(x) == orc.argreduce("argmin", x, 1)
    x[int(rng.integers(0, n))] = np.nan  # a single NaN is pinned by the reference's tests
    assert oc.argmax(x) == orc.argreduce("argmax", x, 1) == oc.argmin(x)


def test_round_conj_parts_proj_rules():
    # round.hpp:74-96 (rint: ties to even), conj.hpp / real.hpp / imag.hpp / proj.hpp type maps
    assert (orc.unary("round", np.array([0.5, 1.5, 2.5, -0.5, -1.5], dtype="f4")) == [0, 2, 2, -0.0, -2]).all()
    assert (orc.unary("round", np.array([3, -4], dtype="i2")) == [3, -4]).all()
    for dt in ("f2", "f4", "f8"):  # test_round.py:107-122 (values spelled out: ties go to even)
        x = np.array([np.nan, np.inf, -np.inf, 1.5, 2.5, -1.5, -2.5, 0.0, -0.0], dtype=dt)
        y = orc.unary("round", x)
        assert np.isnan(y[0]) and y[1:].tolist() == [np.inf, -np.inf, 2, 2, -2, -2, 0, 0]
        assert np.signbit(y).tolist() == [False, False, True, False, False, True, True, False, True]
        h = np.arange(-9, 10).astype(dt) + np.dtype(dt).type(0.5)
        assert orc.unary("round", h).tolist() == [float(round(float(v))) for v in h]  # Python: half to even
    assert orc.unary("conj", np.array([True])).dtype == np.dtype("i1")
    assert orc.unary("conj", np.array([1 + 2j], dtype="c8"))[0] == 1 - 2j
    assert orc.unary("real", np.array([1 + 2j], dtype="c16")).dtype == np.dtype("f8")
    assert orc.unary("imag", np.array([5], dtype="i4"))[0] == 0
    p = orc.unary("proj", np.array([complex(-np.inf, -2.0), 1 + 1j]))
    assert p[0].real == np.inf and np.signbit(p[0].imag) and p[1] == 1 + 1j
    # logaddexp closed forms: log(e^x + e^x) = x + log 2; one operand at -inf leaves the other
    assert orc.binary("logaddexp", np.array([3.0]), np.array([3.0]))[0] == 3.0 + np.log(2.0)
    assert orc.binary("logaddexp", np.array([-np.inf]), np.array([7.0]))[0] == 7.0


# ---- NaN-ignoring reductions: the restated composition against NumPy's nan-functions ----------
@pytest.mark.parametrize("dt", ["f4", "f8"])
def test_oracle_nan_functions_match_numpy(dt):
    rng = np.random.default_rng(5)
    a = rng.uniform(-5, 5, (6, 9, 4)).astype(dt)
    a[rng.random(a.shape) < 0.3] = np.nan
    a[1, :, 2] = np.nan
    for trailing, axis in ((1, -1), (2, (1, 2)), (3, None)):
        for name in ("nansum", "nanprod", "nanmax", "nanmin"):
            with warnings.catch_warnings():
                warnings.simplefilter("ignore", RuntimeWarning)
                want = getattr(np, name)(a.astype("f8"), axis=axis)
            got, _ = orc.nan_reduce(name, a, trailing)
            np.testing.assert_allclose(got, want, rtol=2e-6 if dt == "f4" else 1e-13, equal_nan=True)
        with warnings.catch_warnings():
            warnings.simplefilter("ignore", RuntimeWarning)
            np.testing.assert_allclose(orc.nanmean(a, trailing), np.nanmean(a.astype("f8"), axis=axis),
                                       rtol=2e-6 if dt == "f4" else 1e-13, equal_nan=True)
            np.testing.assert_allclose(orc.nanvar(a, trailing, 1), np.nanvar(a.astype("f8"), axis=axis, ddof=1),
                                       rtol=2e-5 if dt == "f4" else 1e-12, equal_nan=True)
    b = a.copy()
    b[..., 0] = rng.uniform(-5, 5, b.shape[:-1]).astype(dt)  # no run of NaNs only
    assert_equal = np.testing.assert_array_equal
    assert_equal(orc.nan_argreduce("nanargmax", b, 1), np.nanargmax(b, axis=-1))
    assert_equal(orc.nan_argreduce("nanargmin", b, 1), np.nanargmin(b, axis=-1))
    with pytest.raises(ValueError):
        orc.nan_argreduce("nanargmax", a, 1)
    # reference docstring values (dpnp/dpnp_iface_nanfunctions.py:583-590,1301-1306)
    c = np.array([[1, np.nan], [3, 4]])
    assert orc.nanmean(c, 2) == pytest.approx(2.6666666666666665)
    np.testing.assert_allclose(orc.nanvar(c.T, 1), [1.0, 0.0])
    assert orc.nanvar(c, 2) == pytest.approx(1.5555555555555556)


# ---- functions of the ufunc extension: the oracle's entries against independent evaluations ----
def test_oracle_extension_functions_known_values():
    import mpmath

    mpmath.mp.dps = 40
    x = np.array([-2.5, -0.3, 0.0, 0.7, 3.0], dtype="f8")
    for name, ref in (("erfc", mpmath.erfc), ("i0", lambda v: mpmath.besseli(0, v)),
                      ("erfcx", lambda v: mpmath.exp(v * v) * mpmath.erfc(v))):
        want = np.array([float(ref(mpmath.mpf(float(v)))) for v in x])
        np.testing.assert_allclose(orc.unary(name, x), want, rtol=1e-14)
    p = np.array([-0.9, -0.2, 0.0, 0.5, 0.99], dtype="f8")
    np.testing.assert_allclose([math.erf(v) for v in orc.unary("erfinv", p)], p, rtol=1e-14, atol=1e-16)
    q = np.array([0.01, 0.5, 1.0, 1.7], dtype="f8")
    np.testing.assert_allclose([math.erfc(v) for v in orc.unary("erfcinv", q)], q, rtol=1e-13)
    # closed forms
    assert orc.unary("sinc", np.array([0.0, 0.5, 1.0], dtype="f8")).tolist() == pytest.approx([1.0, 2 / math.pi, 0.0],
                                                                                           abs=1e-16)
    assert orc.unary("degrees", np.array([math.pi], dtype="f8"))[0] == 180.0
    assert orc.unary("bitwise_count", np.array([0, 1, -1, 127, -128], dtype="i1")).tolist() == [0, 1, 1, 7, 1]
    assert orc.unary("spacing", np.array([1.0], dtype="f4"))[0] == np.finfo("f4").eps
    assert orc.unary("spacing", np.array([-1.0], dtype="f2"))[0] == np.float16(2.0 ** -11)  # towards +inf
    assert orc.binary("fmod", np.array([-7, 7, 5], dtype="i4"), np.array([3, -3, 0], dtype="i4")).tolist() == [-1, 1, 0]
    assert orc.binary("gcd", np.array([12, -12, 0], dtype="i4"), np.array([18, 18, 0], dtype="i4")).tolist() == [6, 6, 0]
    assert orc.binary("lcm", np.array([4, -4, 0], dtype="i4"), np.array([6, 6, 5], dtype="i4")).tolist() == [12, 12, 0]
    nan = np.nan
    assert np.array_equal(orc.binary("fmax", np.array([1.0, nan, nan]), np.array([nan, 2.0, nan])),
                          np.array([1.0, 2.0, nan]), equal_nan=True)
    assert orc.binary("heaviside", np.array([-1.0, 0.0, 2.0]), np.array([0.5, 0.5, 0.5])).tolist() == [0.0, 0.5, 1.0]
    assert orc.binary("logaddexp2", np.array([3.0]), np.array([3.0]))[0] == 4.0


def test_clip_matches_numpy_and_the_reference_special_cases():
    # pins oracle.clip: np.clip wherever lo <= hi and nothing is NaN; hi wins when lo > hi
    # (dpnp/tests/tensor/test_tensor_clip.py:638-644); a NaN bound gives NaN, a NaN element stays
    # (test_tensor_clip.py:178-187); bool: (x or lo) and hi by truth table
    rng = np.random.default_rng(3)
    for dt in ("i1", "u2", "i4", "i8", "f2", "f4", "f8"):
        x = (rng.uniform(-100, 100, 500)).astype(dt)
        lo = (rng.uniform(-100, 0, 500)).astype(dt)
        hi = (rng.uniform(0, 100, 500)).astype(dt)
        np.testing.assert_array_equal(orc.clip(x, lo, hi), np.clip(x, lo, hi))
        got = orc.clip(x, hi, lo)  # lo > hi: the upper bound is applied last
        np.testing.assert_array_equal(got[hi > lo], lo[hi > lo])
    x = np.arange(10, dtype="f4")
    assert np.isnan(orc.clip(x, np.float32(np.nan), np.float32(np.inf))).all()
    assert np.isnan(orc.clip(x, np.float32(-np.inf), np.float32(np.nan))).all()
    xn = np.array([np.nan, 1.0, 5.0], "f8")
    np.testing.assert_array_equal(orc.clip(xn, np.float64(2), np.float64(3)), np.array([np.nan, 2.0, 3.0]))
    for xv in (False, True):
        for lv in (False, True):
            for hv in (False, True):
                assert bool(orc.clip(np.array(xv), np.array(lv), np.array(hv))) == ((xv or lv) and hv)
    # complex: lexicographic order on (real, imag)
    z = np.array([1 + 1j, 1 + 5j, 3 + 0j, 0 + 9j], "c8")
    got = orc.clip(z, np.complex64(1 + 2j), np.complex64(2 + 0j))
    np.testing.assert_array_equal(got, np.array([1 + 2j, 1 + 5j, 2 + 0j, 1 + 2j], "c8"))


def test_var_around_mean_identities_and_docstring_values():
    # the reference's documented values (dpnp_iface_statistics.py:1821-1826 and 1629-1634)
    a = np.array([[14, 8, 11, 10], [7, 9, 10, 11], [10, 15, 5, 10]])
    m = a.mean(axis=1)
    v = orc.var_around_mean(a, 1, mean=m)
    assert v.dtype == np.dtype("f8")
    assert np.array_equal(v, [4.6875, 2.1875, 12.5])
    np.testing.assert_allclose(np.sqrt(v), [2.16506351, 1.47901995, 3.53553391], rtol=1e-8)
    # exact rational arithmetic on small integer data, real and complex, with and without a given mean
    rng = np.random.default_rng(5)
    re, im = rng.integers(-9, 10, (4, 7)), rng.integers(-9, 10, (4, 7))
    z = (re + 1j * im).astype("c16")
    for ddof in (0, 1, 2.5, 7, 9):
        for r in range(4):
            mr, mi = Fraction(int(re[r].sum()), 7), Fraction(int(im[r].sum()), 7)
            tot = sum((Fraction(int(p)) - mr) ** 2 + (Fraction(int(q)) - mi) ** 2 for p, q in zip(re[r], im[r]))
            got = orc.var_around_mean(z, 1, ddof=ddof)[r]
            div = Fraction(7) - Fraction(ddof)
            if div == 0:
                assert np.isnan(got)
            else:  # (a negative divisor is kept: the reference does not clamp it)
                assert got == pytest.approx(float(tot / div), rel=1e-14)
    given = np.array([1.5 - 2j, 0, 3j, -1])
    for r in range(4):
        tot = sum((Fraction(int(p)) - Fraction(given[r].real)) ** 2 + (Fraction(int(q)) - Fraction(given[r].imag)) ** 2
                  for p, q in zip(re[r], im[r]))
        assert orc.var_around_mean(z, 1, mean=given, ddof=1)[r] == pytest.approx(float(tot / 6), rel=1e-14)
    # var(z) = var(Re z) + var(Im z); var(x, mean=m) = var(x) + (mean(x) - m)^2
    x = rng.normal(3, 2, (5, 64))
    w = (x + 1j * rng.normal(-1, 0.5, (5, 64))).astype("c16")
    np.testing.assert_allclose(orc.var_around_mean(w, 1), orc.var(w.real.copy(), 1) + orc.var(w.imag.copy(), 1),
                               rtol=1e-13)
    shift = rng.normal(0, 1, 5)
    np.testing.assert_allclose(orc.var_around_mean(x, 1, mean=x.mean(axis=1) + shift),
                               orc.var(x, 1) + shift ** 2, rtol=1e-13)
    # dtypes: complex64 -> float32, integers -> float64, float32 data with a float32 mean stays float32
    assert orc.var_around_mean(w.astype("c8"), 1).dtype == np.dtype("f4")
    assert orc.var_around_mean(re.astype("i2"), 1, mean=np.zeros(4, "f4")).dtype == np.dtype("f8")
    assert orc.var_around_mean(x.astype("f4"), 1, mean=np.zeros(5, "f4")).dtype == np.dtype("f4")
    assert np.isnan(orc.var_around_mean(np.zeros((2, 0)), 1)).all()
