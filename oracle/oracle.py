"""NumPy restatement of what the reference computes on the elementwise + reduction path.

TEST INFRASTRUCTURE ONLY (see oracle/__init__.py).  Every function cites the reference code
it restates (paths relative to the reference tree; libtensor = dpnp/tensor/libtensor).

How each part is pinned (tests/test_oracle.py):
  * add/subtract/multiply/divide/sqrt on floats: IEEE-754 correctly rounded, so NumPy's
    same-dtype result is the bit-exact answer; known answers of
    dpnp/tests/tensor/elementwise/test_add.py:49-88.
  * integer and bool arithmetic, bitwise ops, comparisons, where: brute force over small
    ranges against Python integer arithmetic; fixtures of test_bitwise_and.py:43-94 and
    test_usm_ndarray_search_functions.py:69-110.
  * exp/log/erf: checked against mpmath at 60 digits (ulp_error below).
  * sum/prod: closed forms (all-ones, arange) of test_tensor_sum.py:56-101,184-257; max/min
    NaN propagation test_usm_ndarray_reductions.py:150-173.
  * argmax/argmin: fixtures test_usm_ndarray_reductions.py:94-106,254-299 and brute force on
    every tie/NaN pattern of short arrays.  With SEVERAL NaNs the reference's answer depends
    on the device's work-group size (reductions.hpp:1916-1972,2219-2320); this oracle returns
    the first NaN (NumPy): parity unpinned for that case only.
  * mean/var: closed forms of test_tensor_statistical_functions.py:159-241.
  * collapse: pointer-set invariance (strided_iters.hpp:340-361) by brute-force enumeration.
  * promotion: numpy.result_type as in test_add.py:62-65 and the cases of
    dpnp/tests/tensor/test_type_utils.py:87-240.
"""
import itertools
import math

import numpy as np

ALL_DTYPES = [np.dtype(c) for c in ("?", "i1", "u1", "i2", "u2", "i4", "u4", "i8", "u8",
                                    "f2", "f4", "f8", "c8", "c16")]


# ---------------------------------------------------------------------------------------------
# conversions: convert_impl, libtensor/include/utils/type_utils.hpp:64-117
# ---------------------------------------------------------------------------------------------
def cast(a, dtype):
    a = np.asarray(a)
    dtype = np.dtype(dtype)
    if a.dtype == dtype:
        return a.copy()
    if dtype.kind == "b":
        return a != 0
    if a.dtype.kind == "c" and dtype.kind != "c":
        a = a.real  # real_t(complex) == real_t(complex.real())
    if a.dtype.kind == "f" and dtype.kind == "u":
        # negative values wrap like two's complement: through a signed type first
        mid = np.int32 if dtype.itemsize < 4 else np.int64
        with np.errstate(invalid="ignore", over="ignore"):
            neg = a < 0
            out = np.where(neg, 0, a).astype(dtype)
            out[neg] = a[neg].astype(mid).astype(dtype)
        return out
    with np.errstate(invalid="ignore", over="ignore"):
        return a.astype(dtype)


# ---------------------------------------------------------------------------------------------
# elementwise functors: libtensor/include/kernels/elementwise_functions/<op>.hpp
# ---------------------------------------------------------------------------------------------
def _same(a, b):
    a, b = np.asarray(a), np.asarray(b)
    assert a.dtype == b.dtype, "binary kernels exist for same-dtype pairs"
    return a, b


def _floor_divide(a, b):
    # floor_divide.hpp:69-86: x // 0 == 0 for ints, floor(x / y) for floats
    if a.dtype.kind in "iu":
        out = np.zeros(np.broadcast(a, b).shape, dtype=a.dtype)
        nz = np.broadcast_to(b != 0, out.shape)
        with np.errstate(all="ignore"):
            q = np.floor_divide(a, np.where(b == 0, 1, b))
        out[nz] = np.broadcast_to(q, out.shape)[nz]
        return out
    with np.errstate(all="ignore"):
        d = a / b
        return np.where(d == 0, d, np.floor(d)).astype(a.dtype)


def _remainder(a, b):
    # remainder.hpp:66-97.  ints: x % 0 == 0; C remainder (sign of the dividend), then `+= y` when
    # it is non-zero and the operands' signs differ.  floats: fmod, then `+= y` when the
    # remainder is non-zero and its sign differs from y's; a zero remainder takes y's sign.
    if a.dtype.kind in "iu":
        shape = np.broadcast(a, b).shape
        a, b = np.broadcast_to(a, shape), np.broadcast_to(b, shape)
        zero = b == 0
        with np.errstate(all="ignore"):
            r = np.fmod(a, np.where(zero, 1, b)).astype(a.dtype)      # C `%`, pinned by brute force
            if a.dtype.kind == "i":
                fix = (r != 0) & ((a < 0) != (b < 0))
                r = np.where(fix, r + b, r).astype(a.dtype)
        return np.where(zero, 0, r).astype(a.dtype)
    with np.errstate(all="ignore"):
        r = np.fmod(a, b)
        fix = (r != 0) & ((b < 0) != (r < 0))
        r = np.where(fix, r + b, r)
        r = np.where(r == 0, np.copysign(0, b), r)  # NaN != 0: NaNs pass through
        return r.astype(a.dtype)


def _shift(a, b, left):
    # bitwise_left_shift.hpp:88-103, bitwise_right_shift.hpp:88-105: a negative count gives 0 in
    # both directions; a count >= the width gives 0, except -1 for a right shift of a negative value
    bits = a.dtype.itemsize * 8
    shape = np.broadcast(a, b).shape
    a, b = np.broadcast_to(a, shape), np.broadcast_to(b, shape)
    signed = a.dtype.kind == "i"
    neg = (b < 0) if signed else np.zeros(shape, dtype=bool)
    wide = (b >= bits) & ~neg
    sb = np.where(neg | wide, 0, b).astype(a.dtype)
    if left:
        val = np.left_shift(a, sb)
        over = np.zeros(shape, dtype=a.dtype)
    else:
        val = np.right_shift(a, sb)
        over = np.where(a < 0, -1, 0).astype(a.dtype) if signed else np.zeros(shape, dtype=a.dtype)
    return np.where(neg, 0, np.where(wide, over, val)).astype(a.dtype)


def _int_pow(a, b):
    # pow.hpp:72-92: a negative exponent gives 0 for every base; otherwise repeated squaring in
    # the operand type (wraps), with 1 for base 1 or exponent 0
    shape = np.broadcast(a, b).shape
    dt = a.dtype
    base = np.broadcast_to(a, shape).copy()
    e = np.broadcast_to(b, shape).copy()
    neg = (e < 0) if dt.kind == "i" else np.zeros(shape, dtype=bool)
    e = np.where(neg, 0, e).astype(dt)
    res = np.ones(shape, dtype=dt)
    with np.errstate(over="ignore"):
        while (e > 0).any():
            odd = (e & 1).astype(bool)
            res = np.where(odd, res * base, res).astype(dt)
            e = (e >> 1).astype(dt)
            base = (base * base).astype(dt)
    return np.where(neg, 0, res).astype(dt)


def _sign(a):
    # sign.hpp:73-110: unsigned 0 < x; signed and floats (0 < x) - (x < 0), NaN stays NaN;
    # complex z / |z| with sign(0) = 0
    k = a.dtype.kind
    if k == "b":
        return a.copy()
    if k == "u":
        return (a > 0).astype(a.dtype)
    if k == "c":
        mag = np.where(a == 0, 1, np.abs(a))
        with np.errstate(all="ignore"):
            out = np.empty(a.shape, dtype=a.dtype)   # complex / real: each part divided once
            out.real, out.imag = a.real / mag, a.imag / mag
        return np.where(a == 0, 0, out).astype(a.dtype)
    out = ((a > 0).astype(np.int8) - (a < 0).astype(np.int8)).astype(a.dtype)
    if k == "f":
        out[np.isnan(a)] = np.nan
    return out


def _maximum(a, b):
    # maximum.hpp:74-90: (isnan(x) || x > y) ? x : y
    if a.dtype.kind == "c":
        return np.where(_cplx_pick(a, b, True), a, b)
    if a.dtype.kind == "f":
        with np.errstate(invalid="ignore"):
            return np.where(np.isnan(a) | (a > b), a, b)
    return np.maximum(a, b)


def _minimum(a, b):
    if a.dtype.kind == "c":
        return np.where(_cplx_pick(a, b, False), a, b)
    if a.dtype.kind == "f":
        with np.errstate(invalid="ignore"):
            return np.where(np.isnan(a) | (a < b), a, b)
    return np.minimum(a, b)


def _cplx_cmp(a, b, op):
    # libtensor/include/utils/math_utils.hpp:43-95
    with np.errstate(invalid="ignore"):
        same_re = a.real == b.real
        ok = ~np.isnan(a.imag) & ~np.isnan(b.imag)
        im = {"<": a.imag < b.imag, "<=": a.imag <= b.imag, ">": a.imag > b.imag, ">=": a.imag >= b.imag}[op]
        re = (a.real < b.real) if op in ("<", "<=") else (a.real > b.real)
        return np.where(same_re, im, re & ok)


def _cplx_pick(a, b, is_max):
    # max_complex / min_complex, math_utils.hpp:97-127: true where the first operand wins
    return np.isnan(a.real) | np.isnan(a.imag) | _cplx_cmp(a, b, ">" if is_max else "<")


def _compare(a, b, op):
    if a.dtype.kind == "c" and op not in ("==", "!="):
        return _cplx_cmp(a, b, op)
    with np.errstate(invalid="ignore"):
        return {"==": a == b, "!=": a != b, "<": a < b, "<=": a <= b, ">": a > b, ">=": a >= b}[op]


def binary(op, a, b):
    """out = op(a, b) for same-dtype operands, as the reference's functors compute it."""
    a, b = np.asarray(a), np.asarray(b)
    if op in ("equal", "not_equal", "less", "less_equal", "greater", "greater_equal") and \
            {a.dtype.str[1:], b.dtype.str[1:]} == {"i8", "u8"}:
        # mixed int64/uint64 comparisons are exact (greater.hpp:62-146): Python ints
        sym = {"equal": "==", "not_equal": "!=", "less": "<", "less_equal": "<=", "greater": ">",
               "greater_equal": ">="}[op]
        ai, bi = np.broadcast_arrays(a, b)
        f = {"==": int.__eq__, "!=": int.__ne__, "<": int.__lt__, "<=": int.__le__, ">": int.__gt__,
             ">=": int.__ge__}[sym]
        return np.array([f(int(x), int(y)) for x, y in zip(ai.ravel(), bi.ravel())], dtype=bool).reshape(ai.shape)
    a, b = _same(a, b)
    k = a.dtype.kind
    with np.errstate(all="ignore"):
        if op == "add":
            return (a | b) if k == "b" else a + b      # add.hpp:63-114; bool + bool is logical or
        if op == "subtract":
            assert k != "b"
            return a - b
        if op == "multiply":
            return (a & b) if k == "b" else a * b
        if op == "divide":
            assert k in "fc"
            return a / b
        if op in ("bitwise_and", "bitwise_or", "bitwise_xor"):
            assert k in "biu"
            return {"bitwise_and": np.bitwise_and, "bitwise_or": np.bitwise_or, "bitwise_xor": np.bitwise_xor}[op](a, b)
        if op in ("equal", "not_equal", "less", "less_equal", "greater", "greater_equal"):
            sym = {"equal": "==", "not_equal": "!=", "less": "<", "less_equal": "<=", "greater": ">",
                   "greater_equal": ">="}[op]
            return _compare(a, b, sym)
        if op == "maximum":
            return _maximum(a, b).astype(a.dtype)
        if op == "minimum":
            return _minimum(a, b).astype(a.dtype)
        if op in ("logical_and", "logical_or", "logical_xor"):
            x, y = cast(a, "?"), cast(b, "?")
            return {"logical_and": x & y, "logical_or": x | y, "logical_xor": x ^ y}[op]
        if op == "floor_divide":
            return _floor_divide(a, b)
        if op == "remainder":
            return _remainder(a, b)
        if op == "pow":
            return _int_pow(a, b) if k in "iu" else np.power(a, b)
        if op == "atan2":
            return np.arctan2(a, b)
        if op == "hypot":
            return np.hypot(a, b)
        if op == "copysign":
            return np.copysign(a, b)
        if op == "bitwise_left_shift":
            return _shift(a, b, True)
        if op == "bitwise_right_shift":
            return _shift(a, b, False)
        if op == "logaddexp":           # math_utils.hpp:129-150
            return np.logaddexp(a.astype(np.longdouble), b.astype(np.longdouble)).astype(a.dtype)
        if op == "nextafter":
            return np.nextafter(a, b)
        # ---- dpnp/backend/kernels/elementwise_functions/*.hpp (the ufunc extension) ----
        if op in ("fmax", "fmin"):      # fmax.hpp / fmin.hpp: a NaN operand loses
            if k == "c":                # keep a when b holds a NaN or a >= b (a <= b) lexicographically
                bn = np.isnan(b.real) | np.isnan(b.imag)
                keep = bn | _cplx_cmp(a, b, ">=" if op == "fmax" else "<=")
                return np.where(keep, a, b)
            if k == "b":
                return (a | b) if op == "fmax" else (a & b)
            return (np.fmax if op == "fmax" else np.fmin)(a, b)
        if op == "fmod":                # fmod.hpp: C remainder; integer x fmod 0 == 0; bool -> int8
            if k == "b":
                return np.zeros(a.shape, dtype="i1")
            if k in "iu":
                safe = np.where(b == 0, 1, b)
                return np.where(b == 0, 0, np.fmod(a, safe)).astype(a.dtype)
            return np.fmod(a, b)
        if op == "logaddexp2":          # logaddexp2.hpp
            return np.logaddexp2(a.astype(np.longdouble), b.astype(np.longdouble)).astype(a.dtype)
        if op == "heaviside":           # heaviside.hpp
            return np.heaviside(a, b)
        if op == "gcd":                 # gcd.hpp: std::gcd
            return np.gcd(a, b)
        if op == "lcm":                 # lcm.hpp: std::lcm
            return np.lcm(a, b)
    raise KeyError(op)


def unary_result_dtype(op, dt):
    dt = np.dtype(dt)
    if op in ("isnan", "isinf", "isfinite", "logical_not", "signbit"):
        return np.dtype("?")
    if op in ("abs", "real", "imag", "angle"):
        return np.dtype({"c8": "f4", "c16": "f8"}.get(dt.str[1:], dt))
    if op in ("square", "conj") and dt.kind == "b":
        return np.dtype("i1")           # square.hpp / conj.hpp type maps: bool -> int8
    if op in ("erf", "erfc", "erfcx", "erfinv", "erfcinv") and dt == np.dtype("f2"):
        return np.dtype("f4")           # dpnp/backend/extensions/ufunc/elementwise_functions/erf_funcs.cpp:74-84
    if op == "bitwise_count":
        return np.dtype("u1")           # bitwise_count.cpp:72-82
    return dt


def unary(op, a):
    """out = op(a).  Transcendentals are evaluated in float64 (float32/16 input) or long
    double (float64 input) and rounded once: a high-precision stand-in to measure ULPs against."""
    a = np.asarray(a)
    k = a.dtype.kind
    out_dt = unary_result_dtype(op, a.dtype)
    with np.errstate(all="ignore"):
        if op == "abs":
            return np.abs(a).astype(out_dt)
        if op == "negative":
            return np.negative(a)
        if op == "positive":
            return a.copy()
        if op == "square":
            return a.astype(out_dt) * a.astype(out_dt)
        if op == "sqrt":
            return np.sqrt(a)            # IEEE: correctly rounded
        if op in _HI:
            return hi_precision(op, a).astype(out_dt)
        if op == "rsqrt":
            return (1 / np.sqrt(a)).astype(a.dtype)
        if op == "reciprocal":
            return (1 / a).astype(a.dtype)
        if op in ("floor", "ceil", "trunc"):
            return getattr(np, op)(a).astype(a.dtype) if k == "f" else a.copy()
        if op == "sign":
            return _sign(a)
        if op == "isnan":
            return np.isnan(a)
        if op == "isinf":
            return np.isinf(a)
        if op == "isfinite":
            return np.isfinite(a)
        if op == "logical_not":
            return ~cast(a, "?")
        if op == "bitwise_invert":
            return ~a
        if op == "signbit":
            return np.signbit(a)
        if op == "round":               # round.hpp:74-96: rint, ties to even; ints unchanged
            return np.rint(a).astype(a.dtype) if k in "fc" else a.copy()
        if op == "conj":
            return np.conj(a).astype(out_dt)
        if op == "real":
            return np.real(a).astype(out_dt)
        if op == "imag":
            return np.imag(a).astype(out_dt)
        if op == "angle":
            return np.angle(a).astype(out_dt)
        # ---- dpnp/backend/kernels/elementwise_functions/*.hpp (the ufunc extension) ----
        if op == "fabs":
            return np.fabs(a)
        if op in ("degrees", "radians"):
            return getattr(np, op)(a.astype(np.longdouble)).astype(a.dtype)
        if op == "sinc":                # sinc.hpp:52-72
            wide = np.clongdouble if k == "c" else np.longdouble
            return np.sinc(a.astype(wide)).astype(a.dtype)
        if op == "spacing":             # spacing.hpp: float16 always steps towards +inf
            if a.dtype == np.dtype("f2"):
                out = (np.nextafter(a, np.float16(np.inf)) - a).astype("f2")
                out[np.isinf(a)] = np.nan
                return out
            # nextafter(x, copysign(inf, x)) - x: equals numpy.spacing except at -0.0, where the
            # step is taken downwards (numpy gives +tiny there)
            out = np.nextafter(a, np.copysign(np.inf, a).astype(a.dtype)) - a
            out[np.isinf(a)] = np.nan
            return out.astype(a.dtype)
        if op == "bitwise_count":       # bitwise_count.hpp: popcount(|x|)
            mag = np.abs(a.astype(object)) if k == "i" else a.astype(object)
            return np.array([bin(int(v)).count("1") for v in mag.ravel()], dtype="u1").reshape(a.shape)
        if op in ("erfc", "erfcx", "erfinv", "erfcinv", "i0"):
            import scipy.special as sp

            x = a.astype(np.float64)
            return getattr(sp, op)(x).astype(out_dt)
        if op == "proj":                # proj.hpp: infinities collapse to (inf, copysign(0, im))
            inf = np.isinf(a.real) | np.isinf(a.imag)
            out = a.copy()
            out.real[inf] = np.inf
            out.imag[inf] = np.copysign(0.0, a.imag[inf])
            return out
    raise KeyError(op)


_HI = {"exp": np.exp, "log": np.log, "sin": np.sin, "cos": np.cos, "tan": np.tan, "tanh": np.tanh,
       "exp2": np.exp2, "expm1": np.expm1, "log2": np.log2, "log10": np.log10, "log1p": np.log1p,
       "cbrt": np.cbrt, "erf": None, "asin": np.arcsin, "acos": np.arccos, "atan": np.arctan,
       "sinh": np.sinh, "cosh": np.cosh, "asinh": np.arcsinh, "acosh": np.arccosh, "atanh": np.arctanh}


def hi_precision(op, a):
    """op(a) in a precision well above a.dtype's (float64 for <= float32 input, long double
    for float64 input; erf through mpmath-free math.erf in float64 / mpmath for float64)."""
    a = np.asarray(a)
    if a.dtype.kind == "c":
        wide = np.complex128 if a.dtype.itemsize <= 8 else np.clongdouble
    else:
        wide = np.float64 if a.dtype.itemsize <= 4 else np.longdouble
    x = a.astype(wide)
    with np.errstate(all="ignore"):
        if op == "erf":
            if wide is np.float64:
                return np.vectorize(math.erf, otypes=[np.float64])(x)
            import mpmath

            mpmath.mp.dps = 40
            return np.array([np.longdouble(str(mpmath.erf(mpmath.mpf(float(v))))) if np.isfinite(v)
                             else np.longdouble(math.erf(float(v))) for v in x.ravel()],
                            dtype=np.longdouble).reshape(x.shape)
        return _HI[op](x)


def ulp_error(result, exact_hi):
    """|result - exact| in units of the spacing of result's dtype at `exact`; 0 where both are
    the same non-finite value."""
    result = np.asarray(result)
    dt = result.dtype
    exact_hi = np.asarray(exact_hi)
    with np.errstate(all="ignore"):
        rounded = exact_hi.astype(dt)
        both_nan = np.isnan(result) & np.isnan(rounded)
        same_inf = np.isinf(result) & (result == rounded)
        ulp = np.spacing(np.abs(rounded)).astype(exact_hi.dtype)
        err = np.abs(result.astype(exact_hi.dtype) - exact_hi) / ulp
        err = np.where(both_nan | same_inf, 0, err)
        err = np.where(np.isnan(err), np.inf, err)
    return err


def clip(x, lo, hi):
    """libtensor/include/kernels/clip.hpp:66-86: max(x, lo) then min(.., hi).  Floats: a NaN in x
    stays, a NaN bound wins; bool: (x or lo) and hi; complex through max_complex / min_complex
    (math_utils.hpp:99-129), i.e. the first operand unless the second is lexicographically beyond
    it, NaN first operands kept."""
    x, lo, hi = np.broadcast_arrays(np.asarray(x), np.asarray(lo), np.asarray(hi))
    dt = x.dtype
    assert lo.dtype == dt and hi.dtype == dt
    if dt.kind == "b":
        return (x | lo) & hi
    if dt.kind == "c":
        t = np.where(_cplx_pick(x, lo, True), x, lo)
        return np.where(_cplx_pick(t, hi, False), t, hi).astype(dt)
    if dt.kind == "f":
        with np.errstate(invalid="ignore"):
            t = np.where(np.isnan(x) | (x > lo), x, lo)
            return np.where(np.isnan(t) | (t < hi), t, hi).astype(dt)
    t = np.where(x > lo, x, lo)
    return np.where(t < hi, t, hi).astype(dt)


def where(cond, x1, x2):
    """where.hpp:72-161: cond is true when non-zero (any dtype); x1, x2 of one dtype."""
    x1, x2 = _same(x1, x2)
    return np.where(cast(cond, "?"), x1, x2)


def black_scholes(price, strike, t, rate, vol):
    """examples/example_bs.py:50-78, every operation rounded to the arrays' dtype."""
    dt = price.dtype
    erf = np.vectorize(math.erf, otypes=[np.float64])
    mr = dt.type(-rate)
    sig_sig_two = dt.type(vol * vol * 2)
    a = np.log(price / strike)
    b = t * mr
    z = t * sig_sig_two
    c = dt.type(0.25) * z
    y = dt.type(1.0) / np.sqrt(z)
    w1 = (a - b + c) * y
    w2 = (a - b - c) * y
    d1 = dt.type(0.5) + dt.type(0.5) * erf(w1).astype(dt)
    d2 = dt.type(0.5) + dt.type(0.5) * erf(w2).astype(dt)
    se = np.exp(b) * strike
    call = price * d1 - se * d2
    put = call - price + se
    return call, put


# ---------------------------------------------------------------------------------------------
# reductions: libtensor/include/kernels/reductions.hpp, libtensor/source/reductions/*.cpp
# ---------------------------------------------------------------------------------------------
def default_accumulation_dtype(dt):
    """dpnp/tensor/_type_utils.py:932-952 on a device with fp64."""
    dt = np.dtype(dt)
    if dt.kind in "bi":
        return np.dtype("i8")
    if dt.kind == "u":
        return np.dtype("u8")
    return dt


def _split(a, trailing):
    a = np.asarray(a)
    lead = a.shape[: a.ndim - trailing]
    n = int(np.prod(a.shape[a.ndim - trailing:], dtype=np.int64)) if trailing else 1
    return a.reshape(lead + (n,)), lead, n


def reduce(op, a, trailing, out_dtype=None):
    """Reduce the last `trailing` axes.  sum/prod convert every element to the result dtype
    first (reductions.hpp:482-491) and integer results wrap; bool results are logical or/and
    (sum.cpp:268-270).  Float sums are returned as the correctly rounded exact sum (the
    reference's summation order is unspecified; compare with a tolerance)."""
    a2, lead, n = _split(a, trailing)
    in_dt = a2.dtype
    if op in ("max", "min"):
        if n == 0:
            raise ValueError("reduction cannot be performed over zero-size axes")
        if in_dt.kind in "fc":
            f = _maximum if op == "max" else _minimum
            out = a2[..., 0].copy()
            for j in range(1, n):
                out = f(out, a2[..., j]).astype(in_dt)
            # NaN anywhere wins regardless of the order of the combine
            nan_any = np.isnan(a2).any(axis=-1)
            if in_dt.kind == "f":
                out = np.where(nan_any, np.nan, out).astype(in_dt)
            return out
        if in_dt.kind == "b":
            return a2.any(axis=-1) if op == "max" else a2.all(axis=-1)
        return (a2.max(axis=-1) if op == "max" else a2.min(axis=-1)).astype(in_dt)
    out_dt = np.dtype(out_dtype) if out_dtype is not None else default_accumulation_dtype(in_dt)
    conv = cast(a2, out_dt)
    if out_dt.kind == "b":
        return conv.any(axis=-1) if op == "sum" else conv.all(axis=-1)
    if out_dt.kind in "iu":
        with np.errstate(over="ignore"):
            return (conv.sum(axis=-1, dtype=out_dt) if op == "sum" else conv.prod(axis=-1, dtype=out_dt))
    if op == "sum":
        if out_dt.kind == "c":
            return (_fsum(conv.real, lead) + 1j * _fsum(conv.imag, lead)).astype(out_dt)
        return _fsum(conv, lead).astype(out_dt)
    wide = np.longdouble if out_dt.kind == "f" else np.clongdouble
    with np.errstate(all="ignore"):
        return conv.astype(wide).prod(axis=-1).astype(out_dt)


def _fsum(conv, lead):
    flat = conv.reshape(-1, conv.shape[-1]).astype(np.float64)
    out = np.empty(flat.shape[0], dtype=np.float64)
    for i in range(flat.shape[0]):
        row = flat[i]
        if not np.isfinite(row).all():
            with np.errstate(all="ignore"):
                out[i] = row.sum()
        else:
            out[i] = math.fsum(row)
    return out.reshape(lead)


def argreduce(op, a, trailing):
    """Flat C-order index of the extremum over the last `trailing` axes -> int64: ties take
    the smallest index (argmax.cpp:137-160), a NaN is the extremum for both argmax and argmin
    (reductions.hpp:1958-1963); several NaNs: the first (NumPy; see module docstring)."""
    a2, lead, n = _split(a, trailing)
    if n == 0:
        raise ValueError("reduction cannot be performed over zero-size axes")
    flat = a2.reshape(-1, n)
    out = np.empty(flat.shape[0], dtype=np.int64)
    is_max = op == "argmax"
    for i in range(flat.shape[0]):
        row = flat[i]
        if row.dtype.kind == "c":
            nan = np.isnan(row.real) | np.isnan(row.imag)
            if nan.any():
                out[i] = int(np.argmax(nan))
                continue
            best = 0
            for j in range(1, n):
                if _cplx_cmp(row[j:j + 1], row[best:best + 1], ">" if is_max else "<")[0]:
                    best = j
            out[i] = best
        elif row.dtype.kind == "f":
            nan = np.isnan(row)
            out[i] = int(np.argmax(nan)) if nan.any() else int(np.argmax(row) if is_max else np.argmin(row))
        else:
            out[i] = int(np.argmax(row) if is_max else np.argmin(row))
    return out.reshape(lead)


def mean(a, trailing, out_dtype=None):
    """dpnp/tensor/_statistical_functions.py:166-270: sum / N in the floating dtype of the input
    (float64 for integer and bool input).  Evaluated exactly, rounded once."""
    a2, lead, n = _split(a, trailing)
    dt = np.dtype(out_dtype) if out_dtype else (a2.dtype if a2.dtype.kind in "fc" else np.dtype("f8"))
    if n == 0:
        return np.full(lead, np.nan, dtype=dt)
    s = _fsum(a2.astype(np.float64), lead)
    return (s / n).astype(dt)


def var(a, trailing, correction=0.0, out_dtype=None):
    """dpnp/tensor/_statistical_functions.py:38-163: sum((x - mean)^2) / (N - correction),
    NaN when N - correction <= 0.  Evaluated in float64/long double, rounded once."""
    a2, lead, n = _split(a, trailing)
    dt = np.dtype(out_dtype) if out_dtype else (a2.dtype if a2.dtype.kind == "f" else np.dtype("f8"))
    div = max(n - correction, 0)
    if n == 0 or not div:
        return np.full(lead, np.nan, dtype=dt)
    x = a2.astype(np.longdouble)
    with np.errstate(all="ignore"):
        mu = x.mean(axis=-1, keepdims=True)
        return (((x - mu) ** 2).sum(axis=-1) / div).astype(dt)


def var_around_mean(a, trailing, mean=None, ddof=0, out_dtype=None):
    """dpnp/dpnp_iface_statistics.py:1832-1869, the branch dpnp.var takes for complex input or a
    caller's `mean`: x = a - mean (mean of the run when none is given), |x|^2 (x * conj(x), real part,
    for complex x; x^2 otherwise), summed over the last `trailing` axes, divided by N - ddof.
    `mean` has the leading shape of `a` (one value per run), or broadcasts to it.
    The divisor is N - ddof as it comes (line 1864 writes numpy.max(cnt - ddof, 0): the 0 is an axis
    argument, not a lower bound) and NaN when it is zero.  Result dtype: `out_dtype`, else the real type
    of what `a - mean` promotes to (float64 for integer and bool input).  Evaluated in long double, rounded once."""
    a = np.asarray(a)
    a2, lead, n = _split(a, trailing)
    wide = np.clongdouble if (a2.dtype.kind == "c" or (mean is not None and np.asarray(mean).dtype.kind == "c")) \
        else np.longdouble
    x = a2.astype(wide)
    if mean is None:
        mdt = a2.dtype
        with np.errstate(all="ignore"):
            mu = x.mean(axis=-1, keepdims=True) if n else np.full(lead + (1,), np.nan, dtype=wide)
    else:
        m = np.asarray(mean)
        mdt = m.dtype
        mu = np.broadcast_to(m, lead).astype(wide)[..., None]
    if out_dtype is not None:
        dt = np.dtype(out_dtype)
    else:
        base = a2.dtype if a2.dtype.kind in "fc" else np.dtype("f8")
        dt = np.result_type(base, mdt)
        dt = np.dtype({"c8": "f4", "c16": "f8"}.get(dt.str[1:], dt.str[1:]))
    div = n - ddof
    with np.errstate(all="ignore"):
        d = x - mu
        sq = (d.real * d.real + d.imag * d.imag) if wide is np.clongdouble else d * d
        return (sq.sum(axis=-1) / (np.longdouble(div) if div else np.nan)).astype(dt)


# ---------------------------------------------------------------------------------------------
# NaN-ignoring reductions: dpnp/dpnp_iface_nanfunctions.py
# ---------------------------------------------------------------------------------------------
def _replace_nan(a, val):
    """dpnp/dpnp_iface_nanfunctions.py:78-116: (copy of `a` with NaNs overwritten by val, mask of
    the NaNs) for inexact input, (a, None) otherwise or when there is no NaN."""
    a = np.asarray(a)
    if a.dtype.kind not in "fc":
        return a, None
    mask = np.isnan(a)
    if not mask.any():
        return a, None
    b = a.copy()
    b[mask] = val
    return b, mask


def nan_reduce(op, a, trailing, out_dtype=None):
    """nansum / nanprod / nanmax / nanmin over the last `trailing` axes.
    nansum, nanprod (dpnp_iface_nanfunctions.py:922,1026): NaN -> 1 / 0, then the plain reduction.
    nanmax, nanmin (:509-518, :825-834): NaN -> -inf / +inf, plain reduction, NaN written where the
    whole run was NaN.  Returns (result, all_nan_seen)."""
    a = np.asarray(a)
    if op in ("nansum", "nanprod"):
        b, _ = _replace_nan(a, 0.0 if op == "nansum" else 1.0)
        return reduce(op[3:], b, trailing, out_dtype), False
    b, mask = _replace_nan(a, -np.inf if op == "nanmax" else np.inf)
    res = reduce(op[3:], b, trailing)
    if mask is None:
        return res, False
    m2, _, _ = _split(mask, trailing)
    bad = m2.all(axis=-1)
    res = np.where(bad, np.nan, res).astype(res.dtype)
    return res, bool(bad.any())


def nan_argreduce(op, a, trailing):
    """nanargmax / nanargmin (dpnp_iface_nanfunctions.py:195-200, 279-284): NaN -> -inf / +inf, then
    argmax / argmin; a run of NaNs only raises ValueError."""
    b, mask = _replace_nan(a, -np.inf if op == "nanargmax" else np.inf)
    if mask is not None:
        m2, _, _ = _split(mask, trailing)
        if m2.all(axis=-1).any():
            raise ValueError("All-NaN slice encountered")
    return argreduce(op[3:], b, trailing)


def nanmean(a, trailing, out_dtype=None):
    """dpnp_iface_nanfunctions.py:600-636: sum of the non-NaN elements / their number."""
    a = np.asarray(a)
    b, mask = _replace_nan(a, 0)
    if mask is None:
        return mean(a, trailing, out_dtype)
    dt = np.dtype(out_dtype) if out_dtype else a.dtype
    m2, lead, n = _split(mask, trailing)
    cnt = (~m2).sum(axis=-1)
    b2, _, _ = _split(b, trailing)
    if dt.kind == "c":
        s = _fsum(b2.real, lead) + 1j * _fsum(b2.imag, lead)
    else:
        s = _fsum(b2, lead)
    with np.errstate(all="ignore"):
        return (s / cnt).astype(dt)


def nanvar(a, trailing, ddof=0, out_dtype=None):
    """dpnp_iface_nanfunctions.py:1318-1391 for real input: mean of the non-NaN elements, squared
    deviations with the NaN positions zeroed, divided by (count - ddof); NaN where that is <= 0."""
    a = np.asarray(a)
    b, mask = _replace_nan(a, 0)
    if mask is None:
        return var(a, trailing, ddof, out_dtype)
    dt = np.dtype(out_dtype) if out_dtype else a.dtype
    m2, lead, n = _split(mask, trailing)
    b2 = _split(b, trailing)[0].astype(np.longdouble)
    cnt = (~m2).sum(axis=-1, keepdims=True)
    with np.errstate(all="ignore"):
        avg = b2.sum(axis=-1, keepdims=True) / cnt
        dev = np.where(m2, 0, b2 - avg)
        dof = cnt[..., 0] - ddof
        res = (dev * dev).sum(axis=-1) / dof
    res = np.where(dof <= 0, np.nan, res)
    return res.astype(dt)


# ---------------------------------------------------------------------------------------------
# stride collapsing: libtensor/include/utils/strided_iters.hpp:364-899,946-983
# ---------------------------------------------------------------------------------------------
def address_tuples(shape, strides_list, offsets=None):
    """Set of per-operand element offsets visited by iterating `shape` (brute force)."""
    offsets = offsets or [0] * len(strides_list)
    out = set()
    for idx in itertools.product(*[range(s) for s in shape]):
        out.add(tuple(o + sum(i * s for i, s in zip(idx, st)) for o, st in zip(offsets, strides_list)))
    return out


def collapse(shape, strides_list, keep_order=False):
    """Plain restatement of the contract: drop extent-1 dims, (optionally) sort dims by
    |stride| of the last operand then the ones before it then the extent, reverse dims no
    operand walks forwards, merge neighbours with stride[i] == shape[i+1]*stride[i+1] for all
    operands.  Returns (shape, strides_list, offsets)."""
    nops = len(strides_list)
    dims = [d for d in range(len(shape)) if shape[d] != 1]
    if not keep_order:
        dims.sort(key=lambda d: tuple(abs(strides_list[k][d]) for k in range(nops - 1, -1, -1)) + (shape[d],),
                  reverse=True)
    sh = [shape[d] for d in dims]
    st = [[s[d] for d in dims] for s in strides_list]
    off = [0] * nops
    if not keep_order:
        for i in range(len(sh)):
            if all(s[i] <= 0 for s in st) and any(s[i] < 0 for s in st):
                for k in range(nops):
                    off[k] += st[k][i] * (sh[i] - 1)
                    st[k][i] = -st[k][i]
    changed = True
    while changed:
        changed = False
        for i in range(len(sh) - 1):
            if all(s[i] == sh[i + 1] * s[i + 1] for s in st):
                sh[i] *= sh[i + 1]
                del sh[i + 1]
                for s in st:
                    del s[i]
                changed = True
                break
    return sh, st, off


# ---------------------------------------------------------------------------------------------
# type promotion: dpnp/tensor/_type_utils.py:197-251 (a device with fp16 and fp64)
# ---------------------------------------------------------------------------------------------
def accept_divide(dt1, dt2, c1, c2, r):
    """_acceptance_fn_divide, _type_utils.py:89-107: when BOTH operands change kind, only the
    default dtype of the result's kind is taken (int8 / uint8 is float64, not float16)."""
    if c1.kind != dt1.kind and c2.kind != dt2.kind:
        return r == np.dtype({"f": "f8", "c": "c16"}.get(r.kind, r))
    return True


def promote_binary(supported, dt1, dt2, accept=None):
    """(cast1 or None, cast2 or None, result) where supported(d1, d2) -> result dtype or None:
    first pair, in the fixed dtype order, that both inputs cast to safely and that the op's
    acceptance hook `accept(dt1, dt2, cast1, cast2, result)` takes (_find_buf_dtype2,
    _type_utils.py:219-251)."""
    dt1, dt2 = np.dtype(dt1), np.dtype(dt2)
    r = supported(dt1, dt2)
    if r is not None:
        return None, None, r
    for c1 in ALL_DTYPES:
        for c2 in ALL_DTYPES:
            if np.can_cast(dt1, c1) and np.can_cast(dt2, c2):
                r = supported(c1, c2)
                if r is not None and (accept is None or accept(dt1, dt2, c1, c2, r)):
                    return (None if c1 == dt1 else c1), (None if c2 == dt2 else c2), r
    return None, None, None
