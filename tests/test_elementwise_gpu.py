"""Elementwise kernels against the oracle, through the Python layer and the C ABI.
Bar: bit-exact for integer/bool results and IEEE basic ops; <= 4 ULP for transcendentals."""
import zlib

import numpy as np
import pytest

import dpnp_amd.tensor as dpt
from oracle import oracle as orc
from tests.helpers import ALL, FLOATS, INTS, assert_same, assert_ulp, dev, dev_view_like, host, random_array, strided_views

pytestmark = pytest.mark.gpu

SIZES = [1, 3, 255, 1023, 1024, 1025, 4099, 70001]
EXACT_BINARY = ["add", "subtract", "multiply", "divide", "bitwise_and", "bitwise_or", "bitwise_xor", "equal",
                "not_equal", "less", "less_equal", "greater", "greater_equal", "maximum", "minimum",
                "logical_and", "logical_or", "logical_xor", "floor_divide", "remainder", "copysign",
                "bitwise_left_shift", "bitwise_right_shift"]
ULP_BINARY = ["pow", "atan2", "hypot"]
EXACT_UNARY = ["abs", "negative", "positive", "square", "sqrt", "floor", "ceil", "trunc", "sign", "isnan",
               "isinf", "isfinite", "logical_not", "bitwise_invert", "signbit", "reciprocal", "round", "conj",
               "real", "imag", "proj"]
ULP_UNARY = ["exp", "log", "erf", "sin", "cos", "tan", "tanh", "exp2", "expm1", "log2", "log10", "log1p", "cbrt",
             "rsqrt", "asin", "acos", "atan", "sinh", "cosh", "asinh", "acosh", "atanh"]


def assert_close_complex(got, want, a, b=None):
    """|got - want| within 8 eps of the magnitude of the operands' product (or of the result)."""
    assert got.dtype == want.dtype and got.shape == want.shape
    ok = np.isfinite(want)
    with np.errstate(all="ignore"):
        scale = np.maximum(np.abs(a) * np.abs(a if b is None else b), np.abs(np.where(ok, want, 0)))
    err = np.abs(got[ok] - want[ok])
    assert (err <= 8 * np.finfo(got.dtype).eps * np.maximum(scale[ok], 1e-30)).all()
    assert (np.isnan(got[~ok]) == np.isnan(want[~ok])).all()


def supported_binary(op, dt):
    from dpnp_amd.tensor import _tensor_elementwise_impl as tei

    return getattr(tei, f"_{op}_result_type")(dt, dt) is not None


def supported_unary(op, dt):
    from dpnp_amd.tensor import _tensor_elementwise_impl as tei

    return getattr(tei, f"_{op}_result_type")(dt) is not None


@pytest.mark.parametrize("d1", ALL, ids=str)
def test_add_dtype_matrix(d1):
    # dpnp/tests/tensor/elementwise/test_add.py:49-88
    for d2 in ALL:
        a, b = dpt.ones(33, dtype=d1), dpt.ones(33, dtype=d2)
        r = dpt.add(a, b)
        want_dt = np.result_type(d1, d2)
        assert r.dtype == want_dt
        want = np.ones(33, d1) + np.ones(33, d2)
        assert_same(host(r), want.astype(want_dt))
        r2 = dpt.add(a[::-1], b[::-1])
        assert_same(host(r2), want.astype(want_dt))


@pytest.mark.parametrize("op", EXACT_BINARY)
def test_binary_exact_all_dtypes_and_sizes(op):
    rng = np.random.default_rng(zlib.crc32(op.encode()))  # fixed per op: a failure can be replayed
    for dt in ALL:
        if not supported_binary(op, dt):
            continue
        for n in SIZES:
            a, b = random_array(rng, n, dt, -9, 9), random_array(rng, n, dt, -9, 9)
            if dt.kind == "f":
                a[rng.integers(0, n)] = np.nan
                b[rng.integers(0, n)] = np.inf
                if n > 3:
                    b[rng.integers(0, n)] = 0.0
            if "shift" in op and n > 8:
                # counts on both sides of every boundary: negative, 0, width - 1, width, beyond
                bits = 8 * dt.itemsize
                edge = [0, 1, bits - 1, bits, bits + 1, 127] + ([-1, -bits, -128] if dt.kind == "i" else [])
                b[: len(edge)] = np.array(edge).astype(dt)
                a[: len(edge)] = np.array([-8, 8] * 5)[: len(edge)].astype(dt) if dt.kind == "i" else 200
            got = host(getattr(dpt, op)(dev(a), dev(b)))
            want = orc.binary(op, a, b)
            if op in ("divide", "multiply") and dt.kind == "c":
                # complex products are sums of two rounded products: the last bit depends on
                # whether the compiler fuses them, so compare to a few ULP of the magnitude
                assert_close_complex(got, want, a, b)
            else:
                assert_same(got, want)


@pytest.mark.parametrize("op", ULP_BINARY)
def test_binary_ulp(op):
    rng = np.random.default_rng(7)
    for dt in FLOATS:
        a = random_array(rng, 5000, dt, 0.1, 6)
        b = random_array(rng, 5000, dt, -4, 4)
        got = host(getattr(dpt, op)(dev(a), dev(b)))
        wide = np.float64 if dt.itemsize <= 4 else np.longdouble
        f = {"pow": np.power, "atan2": np.arctan2, "hypot": np.hypot}[op]
        assert_ulp(got, f(a.astype(wide), b.astype(wide)), 4.0)
    for dt in INTS:
        # negative exponents give 0 for every base, 1 and -1 included (pow.hpp:72-78)
        a = random_array(rng, 500, dt, -5, 5)
        b = random_array(rng, 500, dt, -4, 7)
        if op == "pow":
            assert_same(host(dpt.pow(dev(a), dev(b))), orc.binary("pow", a, b))
            nonneg = b >= 0
            with np.errstate(over="ignore"):
                assert_same(host(dpt.pow(dev(a[nonneg]), dev(b[nonneg]))), np.power(a[nonneg], b[nonneg]))


@pytest.mark.parametrize("op", ["floor_divide", "remainder"])
def test_narrow_integer_division_every_pair(op):
    """floor_divide and remainder of 1- and 2-byte integers go through the float reciprocal: every
    (dividend, divisor) pair of int8 and uint8, and 16-bit operands over their whole range with the
    divisors that sit next to zero and at the ends."""
    for dt in ("i1", "u1"):
        info = np.iinfo(dt)
        v = np.arange(info.min, info.max + 1).astype(dt)
        a, b = [m.ravel() for m in np.meshgrid(v, v)]
        assert_same(host(getattr(dpt, op)(dev(a), dev(b))), orc.binary(op, a, b))
    rng = np.random.default_rng(5)
    for dt in ("i2", "u2"):
        info = np.iinfo(dt)
        n = 400000
        a = rng.integers(info.min, info.max + 1, n).astype(dt)
        b = rng.integers(info.min, info.max + 1, n).astype(dt)
        b[: n // 4] = rng.integers(max(info.min, -40), 41, n // 4).astype(dt)
        edge = np.array([info.min, info.max, 0, 1, 2, 3, info.max - 1] + ([-1, -2, info.min + 1] if info.min < 0 else []), dtype=dt)
        ea, eb = [m.ravel() for m in np.meshgrid(edge, edge)]
        a, b = np.concatenate([a, ea]), np.concatenate([b, eb])
        # exact multiples, where the reciprocal product must not fall below the integer
        k = rng.integers(1, 180, 20000)
        d = rng.integers(1, 180, 20000)
        a, b = np.concatenate([a, (k * d).astype(dt)]), np.concatenate([b, d.astype(dt)])
        assert_same(host(getattr(dpt, op)(dev(a), dev(b))), orc.binary(op, a, b))


def test_float32_hyperbolic_functions_over_the_whole_range():
    """float32 sinh / cosh, asinh / acosh / atanh and log1p are the library's own routines (the argument of the
    logarithm formed in double, hardware log2 / reciprocal / rsqrt seeds).  Against a float64 evaluation: magnitudes
    spread over every binade the function is finite on, both signs, the places where the routines change form
    (2^-12, 1, 88, 2^30), arguments next to the ends of the domain, and the special values."""
    rng = np.random.default_rng(31)
    n = 400000
    def spread(lo, hi):  # log-uniform magnitudes
        return np.exp(rng.uniform(np.log(lo), np.log(hi), n)).astype("f4")
    def around(c, rel=1e-3):
        return (c * (1 + rng.uniform(-rel, rel, n // 10))).astype("f4")
    sign = rng.choice(np.array([-1, 1], dtype="f4"), n)
    cases = {
        "sinh": np.concatenate([spread(1e-30, 89.4) * sign, around(1.0), around(88.0), around(2.0 ** -12)]),
        "cosh": np.concatenate([spread(1e-30, 89.4) * sign, around(88.0), rng.uniform(-2, 2, n).astype("f4")]),
        "asinh": np.concatenate([spread(1e-30, 3e38) * sign, spread(1e-5, 100) * sign, around(2.0 ** -12), around(2.0 ** 30)]),
        "acosh": np.concatenate([spread(1.0, 3e38), 1 + spread(1e-7, 1.0), around(2.0 ** 30),
                                 np.nextafter(np.float32(1), np.float32(2)) * np.ones(1, "f4")]),
        "atanh": np.concatenate([spread(1e-30, 1.0) * sign, 1 - spread(6e-8, 0.1), around(2.0 ** -12), around(0.5)]),
        "log1p": np.concatenate([spread(1e-30, 3e38), -spread(1e-30, 1.0), -1 + spread(6e-8, 0.1), around(2.0 ** -12),
                                 -around(2.0 ** -12)]),
    }
    ref = {"sinh": np.sinh, "cosh": np.cosh, "asinh": np.arcsinh, "acosh": np.arccosh, "atanh": np.arctanh,
           "log1p": np.log1p}
    worst = {}
    for name, x in cases.items():
        x = x[np.isfinite(x)]
        if name == "atanh":
            x = x[np.abs(x) < 1]
        if name == "acosh":
            x = x[x >= 1]
        if name == "log1p":
            x = x[x > -1]
        got = host(getattr(dpt, name)(dev(x)))
        assert got.dtype == np.float32
        with np.errstate(all="ignore"):
            exact = ref[name](x.astype("f8"))
        fin = np.isfinite(exact.astype("f4"))
        assert fin.sum() > 0.99 * x.size
        worst[name] = float(np.max(orc.ulp_error(got[fin], exact[fin])))
        assert_same(got[~fin], exact[~fin].astype("f4"))  # overflow to infinity at the same arguments
    assert max(worst.values()) <= 3.0, worst
    # special values and signed zeros
    sp = np.array([0.0, -0.0, np.inf, -np.inf, np.nan, 1.0, -1.0, 1e-45, -1e-45, 1.2e-38, 3.4028235e38, -3.4028235e38,
                   2.0, -2.0, 0.5, -0.5, 89.0, -89.0, 90.0, -90.0, 1e10, -1e10], dtype="f4")
    for name in cases:
        got = host(getattr(dpt, name)(dev(sp)))
        with np.errstate(all="ignore"):
            want = ref[name](sp.astype("f8")).astype("f4")
        assert (np.isnan(got) == np.isnan(want)).all(), name
        ok = ~np.isnan(want)
        assert (np.signbit(got[ok]) == np.signbit(want[ok])).all(), name
        inf = np.isinf(want) | (want == 0)
        assert_same(got[inf], want[inf])
        fin = ok & ~inf
        assert_ulp(got[fin], ref[name](sp.astype("f8"))[fin], 3.0)
    # float16 goes through the same routines
    xh = rng.uniform(-8, 8, 50000).astype("f2")
    for name in ("sinh", "cosh", "asinh"):
        assert_ulp(host(getattr(dpt, name)(dev(xh))), ref[name](xh.astype("f8")), 1.0)


def test_float64_inverse_hyperbolic_functions_over_the_whole_range():
    """float64 asinh / acosh / atanh carry the argument of their logarithm as a sum of two doubles into the library's
    table logarithm.  Against long double: every binade, both signs, arguments next to 0 and next to 1, the switch
    to the series below 2^-13 and to log(2a) above 2^500, the special values."""
    rng = np.random.default_rng(41)
    n = 300000
    def spread(lo, hi):
        return np.exp(rng.uniform(np.log(lo), np.log(hi), n))
    sign = rng.choice([-1.0, 1.0], n)
    cases = {
        "asinh": np.concatenate([spread(1e-300, 1e300) * sign, rng.uniform(-4, 4, n), 2.0 ** -13 * (1 + rng.uniform(-0.5, 1, n)),
                                 2.0 ** 500 * (1 + rng.uniform(-0.5, 1, n)), rng.uniform(-1e-3, 1e-3, n)]),
        "acosh": np.concatenate([spread(1.0, 1e300), 1 + spread(1e-16, 1.0), 1 + rng.uniform(0, 3, n),
                                 2.0 ** 500 * (1 + rng.uniform(-0.5, 1, n)), np.array([1.0, np.nextafter(1.0, 2.0)])]),
        "atanh": np.concatenate([spread(1e-300, 1.0) * sign, 1 - spread(1.2e-16, 0.5), rng.uniform(-1, 1, n),
                                 2.0 ** -13 * (1 + rng.uniform(-0.5, 1, n))]),
    }
    ref = {"asinh": np.arcsinh, "acosh": np.arccosh, "atanh": np.arctanh}
    worst = {}
    for name, x in cases.items():
        if name == "atanh":
            x = x[np.abs(x) < 1]
        got = host(getattr(dpt, name)(dev(x)))
        with np.errstate(all="ignore"):
            exact = ref[name](x.astype(np.longdouble))
        worst[name] = float(np.max(orc.ulp_error(got, exact)))
    assert max(worst.values()) <= 1.5, worst  # host check of the routines: 0.98, 1.01, 0.90 ULP
    sp = np.array([0.0, -0.0, np.inf, -np.inf, np.nan, 1.0, -1.0, 5e-324, -5e-324, 2.2e-308, 1.7e308, -1.7e308, 2.0, -2.0,
                   0.5, -0.5, 1e200, -1e200, 1e-200], dtype="f8")
    for name in cases:
        got = host(getattr(dpt, name)(dev(sp)))
        with np.errstate(all="ignore"):
            want = ref[name](sp)
        assert (np.isnan(got) == np.isnan(want)).all(), name
        ok = ~np.isnan(want)
        assert (np.signbit(got[ok]) == np.signbit(want[ok])).all(), name
        inf = np.isinf(want) | (want == 0)
        assert_same(got[inf], want[inf])
        with np.errstate(all="ignore"):
            assert_ulp(got[ok & ~inf], ref[name](sp.astype(np.longdouble))[ok & ~inf], 1.5)
    # strided and float32-from-float64 paths evaluate the same routine
    x = rng.uniform(-3, 3, 5000)
    assert_same(host(dpt.asinh(dev(x)[::2])), host(dpt.asinh(dev(x)))[::2])


_HALF_TABLE_OPS = ["sin", "cos", "tan", "tanh", "expm1", "log1p", "sinh", "asinh", "acosh", "atanh", "sinc", "exp"]


@pytest.mark.parametrize("name", _HALF_TABLE_OPS)
def test_float16_functions_through_their_table(name):
    """Large contiguous float16 arrays go through a table of the function's 65536 results, staged in LDS; smaller
    and strided ones, and those of cheap functions (exp here), through the plain kernel.  Every bit pattern (NaNs with their payloads, subnormals, both
    zeros, infinities) must give the same bits both ways, whatever the alignment and the tail."""
    fn = getattr(dpt, name)
    every = np.arange(65536, dtype="u2")
    small = host(fn(dev(every.view("f2")))).view("u2")   # the plain kernel: 65536 elements
    # against the host for the numbers (the plain kernel's own accuracy tests are elsewhere: a loose bound here)
    x = every.view("f2")
    with np.errstate(all="ignore"):
        ref = {"rsqrt": lambda v: 1 / np.sqrt(v), "asin": np.arcsin, "acos": np.arccos, "asinh": np.arcsinh,
               "acosh": np.arccosh, "atanh": np.arctanh}.get(name, getattr(np, name, None))(x.astype("f8"))
    got = small.view("f2")
    fin = np.isfinite(ref) & np.isfinite(ref.astype("f2")) & (np.abs(ref) > 6.2e-5)
    assert_ulp(got[fin], ref[fin], 2.0)
    rng = np.random.default_rng(5)
    n = (1 << 23) + 13
    bits = np.concatenate([np.tile(every, 8), rng.integers(0, 65536, n - 8 * 65536).astype("u2")])
    rng.shuffle(bits)
    d = dev(bits.view("f2"))
    for view, hv in ((d, bits), (d[1:], bits[1:]), (d[3:-2], bits[3:-2])):
        assert view.size >= 1 << 23
        got = host(fn(view)).view("u2")
        assert np.array_equal(got, small[hv]), name
    out = dpt.empty(n - 1, dtype="f2")
    fn(d[:-1], out=out)  # into a given array
    assert np.array_equal(host(out).view("u2"), small[bits[:-1]])
    got = host(fn(d[::2])).view("u2")  # strided: the plain kernel
    assert np.array_equal(got, small[bits[::2]])
    fn(d, out=d)  # in place
    assert np.array_equal(host(d).view("u2"), small[bits])


def test_float64_pow_over_the_whole_range():
    """pow of doubles takes the library's own routine (two-term logarithm from a 128-interval table, pow_f64_fast)
    for a positive normal base with a finite exponent and |y log x| < 700, the device library's otherwise.  Against
    an 80-bit evaluation: ordinary arguments, results up to the ends of that range, bases next to 1 with huge
    exponents (where the logarithm's relative error is multiplied by up to 2^10), every binade of the base, the
    edges of the table's intervals, integer exponents; then what the routine leaves to the device library."""
    rng = np.random.default_rng(29)
    n = 120000
    parts = []
    parts.append((rng.uniform(0.1, 10, n), rng.uniform(-3, 3, n)))
    x = np.exp(rng.uniform(-700, 700, n))
    parts.append((x, rng.uniform(-1, 1, n) * 690 / np.maximum(np.abs(np.log(x)), 1e-3)))
    x = 1 + rng.uniform(-0.015, 0.015, n)
    parts.append((x, rng.uniform(-1, 1, n) * 600 / np.maximum(np.abs(np.log(x)), 1e-300)))
    x = (np.float64(1).view("i8") + rng.integers(-2000, 2000, n)).view("f8")  # a few thousand ULP around 1
    lg = np.log1p(x - 1)
    y = np.where(lg != 0, rng.uniform(-1, 1, n) * 690 / np.where(lg != 0, lg, 1), rng.uniform(-1e18, 1e18, n))
    parts.append((x, y))
    parts.append((np.ldexp(rng.uniform(0.5, 1.5, n), rng.integers(-1020, 1020, n)), rng.uniform(-0.65, 0.65, n)))
    edge = 0.705078125 * (1 + rng.uniform(-5e-7, 5e-7, n)) * rng.choice([1.0, 2.0], n)
    parts.append((edge, rng.uniform(-50, 50, n)))
    parts.append((rng.uniform(1, 2, n), rng.integers(-100, 100, n).astype("f8")))
    x = np.concatenate([p[0] for p in parts])
    y = np.concatenate([p[1] for p in parts])
    got = host(dpt.pow(dev(x), dev(y)))
    with np.errstate(all="ignore"):
        exact = np.power(x.astype(np.longdouble), y.astype(np.longdouble))
        t = y * np.log(x)
    own = np.abs(t) < 699
    assert own.sum() > 0.95 * x.size
    assert_ulp(got[own], exact[own], 2.0)   # measured on the host: mean 0.26, worst 1.71 ULP
    rest = ~own & np.isfinite(exact.astype("f8")) & (np.abs(exact) > 1e-300)
    assert_ulp(got[rest], exact[rest], 2.0)  # the device library's pow
    assert float(dpt.pow(dev(np.array([1.0])), dev(np.array([5.0])))[0]) == 1.0
    assert_same(host(dpt.pow(dev(np.array([2.0, 4.0, 10.0, 7.0])), dev(np.array([3.0, 0.5, -2.0, 0.0])))),
                np.array([8.0, 2.0, 0.01, 1.0]))
    # the special values of C's pow, negative bases, subnormals, overflow and underflow: what the routine declines
    sp = [0.0, -0.0, 1.0, -1.0, 2.0, -2.0, 0.5, -0.5, np.inf, -np.inf, np.nan, 5e-324, -5e-324, 1e-310, 1e308, -8.0, 3.0]
    sx, sy = (g.ravel() for g in np.meshgrid(np.array(sp), np.array(sp + [1 / 3, 1e3, -1e3, 2.0 ** 60]), indexing="ij"))
    with np.errstate(all="ignore"):
        want = np.power(sx, sy)
    g = host(dpt.pow(dev(sx), dev(sy)))
    fin = np.isfinite(want) & (want != 0)
    assert np.array_equal(np.isnan(g), np.isnan(want)) and np.array_equal(g[~fin & ~np.isnan(want)], want[~fin & ~np.isnan(want)])
    assert np.array_equal(np.signbit(g[~np.isnan(want)]), np.signbit(want[~np.isnan(want)]))
    assert_ulp(g[fin], np.power(sx[fin].astype(np.longdouble), sy[fin].astype(np.longdouble)), 2.0)
    # the strided and the transposing kernels evaluate element by element: the same values
    assert_same(host(dpt.pow(dev(x)[::2], dev(y)[::2])), got[::2])
    xm, ym = x[:160000].reshape(400, 400), y[:160000].reshape(400, 400)
    assert_same(host(dpt.pow(dev(xm).T, dev(ym).T, order="C")), got[:160000].reshape(400, 400).T)
    # a scalar exponent (broadcast operand)
    assert_same(host(dpt.pow(dev(x[:5000]), 1.75)), host(dpt.pow(dev(x[:5000]), dev(np.full(5000, 1.75)))))


def test_float32_pow_over_the_whole_range():
    """pow of floats takes the library's own routine (float arithmetic, the logarithm in two floats from a small table)
    for a positive normal base with a finite exponent and a normal result, the device library's otherwise: every binade of the base, exponents that overflow,
    underflow and hit the subnormal range, and the special-value table of C's pow."""
    rng = np.random.default_rng(23)
    n = 200000
    x = np.exp(rng.uniform(np.log(1e-37), np.log(1e37), n)).astype("f4")
    y = rng.uniform(-40, 40, n).astype("f4")
    y[: n // 4] = rng.uniform(-2, 2, n // 4).astype("f4")
    y[n // 4: n // 2] = np.round(y[n // 4: n // 2])          # integer exponents
    x[n // 2: n // 2 + 5000] = 1.0 + rng.uniform(-1e-3, 1e-3, 5000).astype("f4")   # bases next to 1
    y[n // 2: n // 2 + 5000] = rng.uniform(-3e4, 3e4, 5000).astype("f4")
    got = host(dpt.pow(dev(x), dev(y)))
    with np.errstate(all="ignore"):
        exact = np.power(x.astype("f8"), y.astype("f8"))
    own = np.abs(y.astype("f8") * np.log2(x.astype("f8"))) < 125.4   # the library's routine: normal results
    assert own.sum() > n // 4 and (~own).sum() > n // 10
    assert_ulp(got[own], exact[own], 1.0)                            # (host check: mean 0.26, worst 0.97 ULP)
    assert_ulp(got[~own], exact[~own], 2.0)                          # the device library's powf
    # the strided and the transposing kernels evaluate element by element: the same values
    assert_same(host(dpt.pow(dev(x)[::2], dev(y)[::2])), got[::2])
    xm, ym = x[:160000].reshape(400, 400), y[:160000].reshape(400, 400)
    assert_same(host(dpt.pow(dev(xm).T, dev(ym).T, order="C")), got[:160000].reshape(400, 400).T)
    # x ** 2 is the rounded product, for every float type, array or scalar exponent, special values included
    for dt in ("f2", "f4", "f8"):
        b = np.concatenate([random_array(rng, 4000, dt, -300, 300), np.array([0.0, -0.0, np.inf, -np.inf, np.nan], dtype=dt)])
        with np.errstate(all="ignore"):
            want = b * b
        assert_same(host(dpt.pow(dev(b), dev(np.full(b.shape, 2, dtype=dt)))), want)
        assert_same(host(dpt.pow(dev(b), 2)), want)
        assert_same(host(dpt.pow(dev(b)[::-1], 2.0)), want[::-1])
    for dt in ("f2",):
        xh, yh = rng.uniform(0.1, 8, 5000).astype(dt), rng.uniform(-4, 4, 5000).astype(dt)
        with np.errstate(all="ignore"):
            assert_ulp(host(dpt.pow(dev(xh), dev(yh))), np.power(xh.astype("f8"), yh.astype("f8")), 1.0)
    sp = np.array([0.0, -0.0, 1.0, -1.0, 0.5, -0.5, 2.0, -2.0, 3.0, -3.0, np.inf, -np.inf, np.nan, 1e-45, -1e-45,
                   3.4e38, 1.1754944e-38], dtype="f4")
    X, Y = [v.ravel() for v in np.meshgrid(sp, sp)]
    got = host(dpt.pow(dev(X), dev(Y)))
    with np.errstate(all="ignore"):
        want = np.power(X, Y)
        exact = np.power(X.astype("f8"), Y.astype("f8"))
    np.testing.assert_array_equal(np.isnan(got), np.isnan(want))
    ok = ~np.isnan(want)
    np.testing.assert_array_equal(np.signbit(got[ok]), np.signbit(want[ok]))
    assert_ulp(got[ok], exact[ok], 1.0)


def test_float16_pow_over_the_whole_range():
    """float16 pow of contiguous operands: 2^(y log2 x) on the hardware's float log2 / exp2 for a positive finite
    base and a finite exponent, the general routine otherwise.  Every positive base against a spread of exponents
    (results that overflow, underflow and land in the subnormal range included), exact cases, the special values."""
    rng = np.random.default_rng(37)
    xs = np.arange(1, 0x7c00, dtype="u2").view("f2")              # every positive finite float16
    x = np.tile(xs, 16)
    y = np.concatenate([rng.uniform(-4, 4, xs.size), rng.uniform(-40, 40, xs.size), np.round(rng.uniform(-9, 9, xs.size)),
                        rng.uniform(-1, 1, xs.size) * 24 / np.maximum(np.abs(np.log2(xs.astype("f8"))), 1e-3)]
                       * 4).astype("f2")
    got = host(dpt.pow(dev(x), dev(y)))
    with np.errstate(all="ignore"):
        exact = np.power(x.astype("f8"), y.astype("f8"))
        want = exact.astype("f2")
    fin = np.isfinite(want) & (want != 0)
    assert fin.sum() > 0.5 * x.size
    assert_ulp(got[fin], exact[fin], 0.51)
    # overflow to infinity and underflow to zero happen at the same arguments, up to a result that sits within
    # 1/100 ULP of the border
    rest = ~fin
    near = np.isfinite(exact) & ((np.abs(np.abs(exact) / 65520.0 - 1) < 1e-5) | (np.abs(np.abs(exact) / 2.0 ** -25 - 1) < 1e-5))
    assert_same(got[rest & ~near], want[rest & ~near])
    assert_same(host(dpt.pow(dev(np.array([2, 4, 9, 10, 0.5, 7], dtype="f2")), dev(np.array([3, 0.5, 0.5, -2, -3, 0], dtype="f2")))),
                np.array([8, 2, 3, 0.01, 8, 1], dtype="f2"))
    sp = np.array([0.0, -0.0, 1.0, -1.0, 0.5, -0.5, 2.0, -2.0, 3.0, -3.0, np.inf, -np.inf, np.nan, 6e-8, -6e-8, 65504.0,
                   6.1e-5, 0.333, 1000.0], dtype="f2")
    X, Y = [v.ravel() for v in np.meshgrid(sp, sp)]
    got = host(dpt.pow(dev(X), dev(Y)))
    with np.errstate(all="ignore"):
        exact = np.power(X.astype("f8"), Y.astype("f8"))
        want = exact.astype("f2")
    np.testing.assert_array_equal(np.isnan(got), np.isnan(want))
    ok = ~np.isnan(want)
    np.testing.assert_array_equal(np.signbit(got[ok]), np.signbit(want[ok]))
    assert_ulp(got[ok], exact[ok], 1.0)
    # the strided kernel evaluates element by element with the general routine: within an ULP of it
    a, b = rng.uniform(0.1, 8, 4000).astype("f2"), rng.uniform(-4, 4, 4000).astype("f2")
    with np.errstate(all="ignore"):
        assert_ulp(host(dpt.pow(dev(a)[::2], dev(b)[::2])), np.power(a[::2].astype("f8"), b[::2].astype("f8")), 1.0)


@pytest.mark.parametrize("op", EXACT_UNARY)
def test_unary_exact(op):
    rng = np.random.default_rng(11)
    for dt in ALL:
        if not supported_unary(op, dt):
            continue
        for n in (1, 1025, 4099):
            a = random_array(rng, n, dt, -50, 50)
            if dt.kind == "f" and n > 4:
                a[:4] = [np.nan, np.inf, -np.inf, -0.0]
            if op in ("sqrt",) and dt.kind != "c":
                a = np.abs(a)
            if op == "proj" and n > 4:
                a[:2] = [complex(np.inf, -1.0), complex(2.0, -np.inf)]
            got = host(getattr(dpt, op)(dev(a)))
            want = orc.unary(op, a)
            if dt.kind == "c" and op in ("abs", "sign", "sqrt", "reciprocal"):
                if op == "sqrt":
                    want = np.sqrt(a.astype("c16")).astype(dt)
                np.testing.assert_allclose(got, want, rtol=8 * np.finfo(got.dtype).eps)
            elif dt.kind == "c" and op == "square":
                assert_close_complex(got, want, a)
            elif op == "proj":
                assert_same(got, want)
                assert_same(np.signbit(got.imag), np.signbit(want.imag))
            elif dt == np.dtype("f2") and op in ("reciprocal",):
                assert_ulp(got, 1 / a.astype("f8"), 1.0)
            else:
                assert_same(got, want)


@pytest.mark.parametrize("op", ULP_UNARY)
def test_unary_transcendentals_within_4_ulp(op):
    rng = np.random.default_rng(13)
    rng_by_op = {"exp": (-80, 80), "exp2": (-100, 100), "expm1": (-30, 30), "log": (1e-30, 1e30),
                 "log2": (1e-30, 1e30), "log10": (1e-30, 1e30), "log1p": (-0.99, 1e10), "erf": (-6, 6),
                 "sin": (-50, 50), "cos": (-50, 50), "tan": (-1.5, 1.5), "tanh": (-20, 20), "cbrt": (-1e10, 1e10),
                 "rsqrt": (1e-10, 1e10), "asin": (-1, 1), "acos": (-1, 1), "atan": (-1e3, 1e3), "sinh": (-20, 20),
                 "cosh": (-20, 20), "asinh": (-1e6, 1e6), "acosh": (1, 1e6), "atanh": (-0.999, 0.999)}
    lo, hi = rng_by_op[op]
    for dt in FLOATS:
        if dt == np.dtype("f2"):
            lo2, hi2 = max(lo, -10), min(hi, 10)
            if op == "acosh":
                lo2, hi2 = 1, 1000
            if op in ("log", "log2", "log10", "rsqrt"):
                lo2, hi2 = 1e-3, 6e4
        else:
            lo2, hi2 = (max(lo, -80), min(hi, 80)) if (dt == np.dtype("f4") and op in ("exp", "exp2")) else (lo, hi)
        n = 3000 if (dt.itemsize == 8 and op == "erf") else 20000
        a = rng.uniform(lo2, hi2, n).astype(dt)
        if op.startswith("log") or op == "rsqrt":
            a = np.exp(rng.uniform(np.log(max(lo2, 1e-30)), np.log(hi2), n)).astype(dt)
        got = host(getattr(dpt, op)(dev(a)))
        if op == "rsqrt":
            wide = np.float64 if dt.itemsize <= 4 else np.longdouble
            exact = 1 / np.sqrt(a.astype(wide))
        else:
            exact = orc.hi_precision(op, a)
        assert got.dtype == orc.unary_result_dtype(op, dt)
        assert_ulp(got, exact, 4.0)
    # special values, dpnp/tests/tensor/elementwise/test_exp.py:124-137, test_log.py:88, test_sqrt.py:94-129
    x = np.array([np.nan, np.inf, -np.inf, 0.0, -0.0], dtype="f4")
    with np.errstate(all="ignore"):
        want = {"exp": np.exp, "log": np.log, "erf": None}.get(op)
        if want is not None:
            got = host(getattr(dpt, op)(dev(x)))
            np.testing.assert_array_equal(got, want(x))
            np.testing.assert_array_equal(np.signbit(got), np.signbit(want(x)))


def test_float64_trigonometric_functions_on_hard_arguments():
    """asin, acos and, below 1e6 in magnitude, sin, cos and tan of doubles are the library's own routines, the
    rest the device library's: against an 80-bit evaluation on every binade, next to multiples of pi/2 and
    pi/4 (where the reduced argument cancels, and where tan's half-angle form has its quotient's extremes),
    across the hand-over at 1e6, next to +-1 and +-1/2."""
    if np.finfo(np.longdouble).nmant < 63:
        pytest.skip("needs an extended-precision long double")
    rng = np.random.default_rng(31)
    tiny = float(np.finfo("f8").tiny)
    mag = np.exp(rng.uniform(np.log(tiny * 4), np.log(1e15), 60000))
    k = rng.integers(1, 636000, 40000).astype("f8")
    near = k * (np.pi / 2) + rng.choice([0.0, 1e-9, -1e-9, 1e-4, -3e-13], k.size)
    edge = 1e6 + rng.uniform(-50, 50, 2000)
    a = np.concatenate([mag * rng.choice([-1.0, 1.0], mag.size), near, -near[:5000], edge, -edge,
                        rng.uniform(-50, 50, 40000)])
    for op, bound in (("sin", 2.0), ("cos", 2.0), ("tan", 2.0)):
        got = host(getattr(dpt, op)(dev(a)))
        assert_ulp(got, orc.hi_precision(op, a), bound)
    # tan below the hand-over: the own routine stays within an ULP, also on the doubles next to multiples of pi/4
    k4 = rng.integers(1, 1272000, 60000).astype("f8")
    m4 = k4 * (np.pi / 4)
    near4 = np.concatenate([m4, np.nextafter(m4, 0), np.nextafter(m4, 2e6), m4 + rng.choice([1e-9, -1e-9, 3e-13, -1e-5], m4.size)])
    t = np.concatenate([a[np.abs(a) < 999900.0], near4[near4 < 999900.0], -near4[:20000][near4[:20000] < 999900.0],
                        rng.uniform(-1.6, 1.6, 40000)])
    assert_ulp(host(dpt.tan(dev(t))), orc.hi_precision("tan", t), 1.0)
    m1 = np.exp(rng.uniform(np.log(tiny * 4), 0.0, 40000))
    b = np.concatenate([m1, 1.0 - m1[m1 < 0.5], 0.5 + rng.uniform(-1e-3, 1e-3, 5000), rng.uniform(0, 1, 40000),
                        np.array([0.0, 0.5, 1.0, np.nextafter(1.0, 0), np.nextafter(0.5, 0), np.nextafter(0.5, 1)])])
    b = np.concatenate([b, -b])
    for op in ("asin", "acos"):
        got = host(getattr(dpt, op)(dev(b)))
        assert_ulp(got, orc.hi_precision(op, b), 1.5)
    special = np.array([0.0, -0.0, np.inf, -np.inf, np.nan, 1.0 + 2.0 ** -52, -1.5, 1e300])
    with np.errstate(all="ignore"):
        for op, f in (("sin", np.sin), ("cos", np.cos), ("tan", np.tan), ("asin", np.arcsin), ("acos", np.arccos)):
            got, want = host(getattr(dpt, op)(dev(special))), f(special)
            np.testing.assert_array_equal(np.isnan(got), np.isnan(want))
            ok = ~np.isnan(want)
            if op in ("asin", "acos"):
                np.testing.assert_array_equal(got[ok], want[ok])
                np.testing.assert_array_equal(np.signbit(got[ok]), np.signbit(want[ok]))
            else:
                assert_ulp(got[ok], f(special[ok].astype(np.longdouble)), 2.0)
                np.testing.assert_array_equal(np.signbit(got[:2]), np.signbit(want[:2]))


@pytest.mark.parametrize("op", ["log1p", "expm1", "sinh", "tanh", "asinh", "atanh", "acosh", "erf", "cosh", "log2", "log10"])
def test_own_math_routines_keep_relative_accuracy_at_every_magnitude(op):
    """The library's own fp32 / fp64 routines (log2, log10, log1p, erf, sinh, cosh, tanh, asinh, acosh, atanh) against
    the high-precision evaluation on arguments spread over every binade: near zero the result is as small as the
    argument and the error bound is relative to it.  Signed zeros, infinities and NaN as NumPy has them."""
    rng = np.random.default_rng(29)
    for dt in (np.dtype("f4"), np.dtype("f8")):
        fi = np.finfo(dt)
        lo, hi = float(fi.tiny) * 4, {"log1p": 1e30, "expm1": 80.0, "sinh": 80.0, "cosh": 80.0, "tanh": 30.0, "asinh": 1e30,
                                      "atanh": 0.9999, "acosh": 1e30, "erf": 6.0, "log2": 1e30, "log10": 1e30}[op]
        mag = np.exp(rng.uniform(np.log(lo), np.log(hi), 40000))
        if op == "acosh":
            a = 1.0 + mag
        elif op in ("log2", "log10"):
            a = np.concatenate([mag, 1.0 / mag[:20000], rng.uniform(0.5, 2.0, 20000)])
        elif op == "log1p":
            a = np.concatenate([mag, -mag[mag < 0.999]])
        else:
            a = mag * rng.choice([-1.0, 1.0], mag.size)
        a = a.astype(dt)
        got = host(getattr(dpt, op)(dev(a)))
        assert_ulp(got, orc.hi_precision(op, a), 4.0)
        special = np.array([0.0, -0.0, np.inf, -np.inf, np.nan, 1.0, -1.0, 0.5, -2.0], dtype=dt)
        with np.errstate(all="ignore"):
            want = getattr(np, {"asinh": "arcsinh", "acosh": "arccosh", "atanh": "arctanh"}.get(op, op), None)
            want = want(special) if want is not None else np.array([0.0, -0.0, 1.0, -1.0, np.nan] + [np.nan] * 4, dtype=dt)
        got = host(getattr(dpt, op)(dev(special)))
        n = 5 if op == "erf" else special.size
        np.testing.assert_array_equal(np.isnan(got[:n]), np.isnan(want[:n]))
        np.testing.assert_array_equal(np.isinf(got[:n]), np.isinf(want[:n]))
        sel = np.isinf(want[:n]) | (want[:n] == 0)
        np.testing.assert_array_equal(got[:n][sel], want[:n][sel])
        np.testing.assert_array_equal(np.signbit(got[:n][sel]), np.signbit(want[:n][sel]))
        if op == "log2":  # powers of two are exact
            k = np.arange(-100, 101)
            np.testing.assert_array_equal(host(dpt.log2(dev((2.0 ** k).astype(dt)))), k.astype(dt))


def test_log_float64_every_binade_within_1_ulp():
    # log of a double is evaluated by the library's own routine (argument reduction + polynomial):
    # dense check against an 80-bit evaluation, all binades including subnormals, and around 1
    if np.finfo(np.longdouble).nmant < 63:
        pytest.skip("needs an extended-precision long double")
    rng = np.random.default_rng(17)
    n = 1 << 20
    mant = rng.uniform(0.5, 1.0, n)
    a = np.concatenate([
        np.ldexp(mant, rng.integers(-1073, 1025, n)),          # every binade
        1.0 + rng.uniform(-1e-3, 1e-3, n),                      # cancellation around 1
        1.0 + np.ldexp(rng.uniform(-1, 1, n), rng.integers(-52, -8, n)),
        rng.uniform(0.5, 2.0, n),                               # both sides of the sqrt(1/2) split
        np.array([np.finfo("f8").max, np.finfo("f8").tiny, 5e-324, 1.0, 0.70710678118654746, 0.70710678118654757]),
    ])
    a = a[a > 0]
    got = host(dpt.log(dev(a)))
    assert_ulp(got, np.log(a.astype(np.longdouble)), 1.0)
    x = np.array([np.nan, np.inf, -np.inf, 0.0, -0.0, -1.0, -5e-324])
    with np.errstate(all="ignore"):
        want = np.log(x)
    got = host(dpt.log(dev(x)))
    np.testing.assert_array_equal(got, want)
    # the same routine behind logaddexp, the complex logarithm and logsumexp
    b = rng.uniform(-700, 700, 4096)
    c = rng.uniform(-700, 700, 4096)
    assert_ulp(host(dpt.logaddexp(dev(b), dev(c))), np.logaddexp(b.astype(np.longdouble), c.astype(np.longdouble)), 2.0)


def test_exp_known_answers():
    # dpnp/tests/tensor/elementwise/test_exp.py:111-120
    for dt in ("f2", "f4", "f8"):
        x = (np.arange(11, dtype=dt) * np.dtype(dt).type(0.69314718055994530943)).astype(dt)
        tol = 8 * np.finfo(dt).resolution
        np.testing.assert_allclose(host(dpt.exp(dev(x))).astype("f8"), np.exp(x.astype("f8")), rtol=tol, atol=tol)


@pytest.mark.parametrize("dt", ["f4", "i4", "?", "f8", "i1", "c8"])
def test_strided_and_broadcast_views(dt):
    rng = np.random.default_rng(17)
    base_a = random_array(rng, (37, 130), dt, -9, 9)
    base_b = random_array(rng, (37, 130), dt, -9, 9)
    for (na, va), (nb, vb) in zip(strided_views(base_a), strided_views(base_b)):
        a, b = dev_view_like(va, base_a), dev_view_like(vb, base_b)
        assert a.strides == tuple(s // va.itemsize for s in va.strides)
        if dt == "c8":
            assert_close_complex(host(dpt.multiply(a, b)), orc.binary("multiply", va, vb), va, vb)
        else:
            assert_same(host(dpt.multiply(a, b)), orc.binary("multiply", va, vb))
        assert_same(host(dpt.greater(a, b)), orc.binary("greater", va, vb))
    # row vector and column vector broadcast, scalar operand
    row, col = random_array(rng, (1, 130), dt, -9, 9), random_array(rng, (37, 1), dt, -9, 9)
    assert_same(host(dpt.add(dev(base_a), dev(row))), orc.binary("add", base_a, np.broadcast_to(row, base_a.shape)))
    assert_same(host(dpt.add(dev(col), dev(base_a))), orc.binary("add", np.broadcast_to(col, base_a.shape), base_a))
    assert_same(host(dpt.add(dev(row), dev(col))),
                orc.binary("add", np.broadcast_to(row, (37, 130)), np.broadcast_to(col, (37, 130))))
    if dt != "?":
        two = np.dtype(dt).type(2)
        assert_same(host(dpt.multiply(dev(base_a), 2)), orc.binary("multiply", base_a, np.full_like(base_a, two)))
        assert_same(host(dpt.multiply(2, dev(base_a)[:, ::3])),
                    orc.binary("multiply", np.full_like(base_a[:, ::3], two), base_a[:, ::3]))


def test_nd_views_random():
    rng = np.random.default_rng(19)
    for _ in range(25):
        nd = int(rng.integers(1, 6))
        shape = tuple(int(s) for s in rng.integers(1, 9, nd))
        big = tuple(2 * s + 1 for s in shape)
        base_a, base_b = random_array(rng, big, "i4"), random_array(rng, big, "i4")

        def rv(base):
            perm = rng.permutation(nd)
            v = np.transpose(base, perm)
            v = v[tuple(slice(None, None, int(st)) for st in rng.choice([1, 2, -1, -2], nd))]
            inv = np.argsort(perm)
            v = np.transpose(v, inv)
            return v[tuple(slice(0, s) for s in shape)] if all(
                v.shape[d] >= shape[d] for d in range(nd)) else np.broadcast_to(base.ravel()[:1].reshape((1,) * nd), shape)

        va, vb = rv(base_a), rv(base_b)
        if va.shape != shape or vb.shape != shape:
            continue
        a = dev_view_like(va, base_a) if va.base is not None and va.strides != (0,) * nd else dev(np.ascontiguousarray(va))
        b = dev_view_like(vb, base_b) if vb.base is not None and vb.strides != (0,) * nd else dev(np.ascontiguousarray(vb))
        assert_same(host(dpt.subtract(a, b)), va - vb)
        cond = random_array(rng, shape, "?")
        assert_same(host(dpt.where(dev(cond), a, b)), np.where(cond, va, vb))


@pytest.mark.parametrize("order", ["K", "C", "F", "A"])
def test_result_layout(order):
    rng = np.random.default_rng(23)
    a = random_array(rng, (12, 20), "f4")
    for v in (dev(a), dev(a).T, dev(a)[:, ::2], dpt.permute_dims(dev(random_array(rng, (3, 4, 5), "f4")), (1, 2, 0))):
        r = dpt.exp(v, order=order)
        want = np.exp(host(v))
        assert_ulp(host(r), np.exp(host(v).astype("f8")), 4.0)
        if order == "C":
            assert r.flags.c_contiguous
        elif order == "F":
            assert r.flags.f_contiguous
        elif order == "K" and v.flags.f_contiguous and not v.flags.c_contiguous:
            assert r.flags.f_contiguous
        assert r.shape == want.shape
        r2 = dpt.add(v, v, order=order)
        assert_same(host(r2), host(v) + host(v))


def test_out_and_overlap():
    rng = np.random.default_rng(29)
    a, b = random_array(rng, 1000, "f4"), random_array(rng, 1000, "f4")
    da, db = dev(a), dev(b)
    out = dpt.empty(1000, dtype="f4")
    r = dpt.add(da, db, out=out)
    assert r is out
    assert_same(host(out), a + b)
    # out is an input: computed in place
    dc = dev(a)
    assert dpt.add(dc, db, out=dc) is dc
    assert_same(host(dc), a + b)
    dc = dev(b)
    assert dpt.subtract(da, dc, out=dc) is dc
    assert_same(host(dc), a - b)
    # partial overlap: a temporary is used, result lands in out
    buf = dev(np.concatenate([a, a]))
    x, o = buf[:1000], buf[1:1001]
    dpt.multiply(x, db, out=o)
    assert_same(host(buf)[1:1001], a * b)
    assert host(buf)[0] == a[0]
    # out in a strided slice of a larger zero array leaves the neighbours untouched
    big = dpt.zeros((1000, 2), dtype="f4")
    dpt.exp(da, out=big[:, 1])
    hb = host(big)
    assert (hb[:, 0] == 0).all()
    assert_ulp(hb[:, 1], np.exp(a.astype("f8")))
    # in-place operators
    dc = dev(a)
    dc += db
    dc *= 2
    assert_same(host(dc), (a + b) * 2)
    di = dev(np.arange(10, dtype="i4"))
    with pytest.raises(ValueError):
        di += 1.5
    ro = dev(a)
    ro.flags.writable = False
    with pytest.raises(ValueError):
        ro += db


def test_python_scalars_follow_weak_promotion():
    a = dev(np.arange(5, dtype="i1"))
    assert dpt.add(a, 1).dtype == np.dtype("i1")
    assert dpt.add(a, 1.5).dtype == np.dtype("f8")
    f = dev(np.arange(5, dtype="f4"))
    assert dpt.multiply(f, 2.5).dtype == np.dtype("f4")
    assert dpt.multiply(f, 1j).dtype == np.dtype("c8")
    assert_same(host(dpt.greater(dev(np.array([1, 200], dtype="u1")), -1)), np.array([True, True]))
    assert_same(host(dpt.divide(dev(np.arange(4, dtype="i4")), 2)), np.arange(4) / 2)
    with pytest.raises(OverflowError):
        dpt.add(a, 1000)


@pytest.mark.parametrize("src", ALL, ids=str)
def test_astype_matrix(src):
    rng = np.random.default_rng(31)
    a = random_array(rng, 2051, src, -120, 120)
    if src.kind == "f":
        a[:3] = [-0.0, 0.25, -3.75]
    for dst in ALL:
        got = host(dpt.astype(dev(a), dst))
        want = orc.cast(a, dst)
        assert_same(got, want)
    v = dev(a)[::-2]
    assert_same(host(dpt.astype(v, "f8")), orc.cast(a[::-2], "f8"))
    assert_same(host(dpt.copy(v)), a[::-2])


def test_empty_and_zero_d():
    z = dpt.empty((0, 5), dtype="f4")
    assert dpt.add(z, z).shape == (0, 5)
    assert dpt.exp(z).shape == (0, 5)
    s = dev(np.float32(3.0))
    assert host(dpt.add(s, s)).shape == () and float(dpt.add(s, s)) == 6.0
    assert float(dpt.sqrt(dev(np.float64(16)))) == 4.0


def test_unaligned_base_pointer():
    # kernels must not assume 16-byte alignment (views such as x[1:])
    rng = np.random.default_rng(37)
    for dt in ("i1", "f2", "f4", "f8"):
        a, b = random_array(rng, 5003, dt), random_array(rng, 5003, dt)
        for k in (1, 2, 3, 5):
            assert_same(host(dpt.add(dev(a)[k:], dev(b)[k:])), (a + b)[k:])
            o = dpt.empty(5003, dtype=dt)
            dpt.add(dev(a)[k:], dev(b)[:-k], out=o[k:])
            assert_same(host(o)[k:], a[k:] + b[:-k])


@pytest.mark.parametrize("op", ["exp", "log", "sqrt", "sin", "cos", "tan", "tanh", "sinh", "cosh"])
def test_complex_elementary_functions(op):
    rng = np.random.default_rng(97)
    for dt, rtol in (("c8", 4e-6), ("c16", 8e-15)):
        a = (rng.uniform(-3, 3, 4000) + 1j * rng.uniform(-3, 3, 4000)).astype(dt)
        got = host(getattr(dpt, op)(dev(a)))
        want = getattr(np, op)(a.astype("c16" if dt == "c8" else np.clongdouble))
        assert got.dtype == np.dtype(dt)
        # log: the real part log|z| vanishes on the unit circle, measure against |z|-scale there
        scale = np.maximum(np.abs(want), 1.0 if op == "log" else 1e-3)
        err = np.abs(got - want) / scale
        assert float(err.max()) <= rtol, float(err.max())
    z = np.array([0j, 1 + 0j, -1 + 0j, 1j, -4 + 0j], dtype="c16")
    np.testing.assert_allclose(host(dpt.sqrt(dev(z))), np.sqrt(z), rtol=1e-15, atol=0)
    np.testing.assert_allclose(host(dpt.exp(dev(z))), np.exp(z), rtol=1e-15, atol=1e-16)
    np.testing.assert_allclose(host(dpt.pow(dev(z[1:]), dev(np.full(4, 2 + 0j)))), z[1:] ** 2, rtol=1e-14, atol=1e-15)


@pytest.mark.parametrize("op", ["asin", "acos", "atan", "asinh", "acosh", "atanh"])
def test_complex_inverse_functions(op):
    rng = np.random.default_rng(131)
    npf = getattr(np, "arc" + op[1:])
    for dt, rtol in (("c8", 4e-6), ("c16", 2e-14)):
        a = (rng.uniform(-3, 3, 4000) + 1j * rng.uniform(-3, 3, 4000)).astype(dt)
        a[:6] = [0.5 + 0j, 2 + 0j, -2 + 0j, 0.25j, 3j, -3j]
        got = host(getattr(dpt, op)(dev(a)))
        want = npf(a.astype("c16" if dt == "c8" else np.clongdouble))
        assert got.dtype == np.dtype(dt)
        err = np.abs(got - want) / np.maximum(np.abs(want), 1e-2)
        assert float(err.max()) <= rtol, (float(err.max()), a[int(np.argmax(err))])
    # the side of a branch cut is chosen by the sign of the zero part, as in NumPy
    cuts = np.array([complex(2, 0.0), complex(2, -0.0), complex(-2, 0.0), complex(-2, -0.0),
                     complex(0.0, 2), complex(-0.0, 2), complex(0.0, -2), complex(-0.0, -2), complex(0.5, -0.0)],
                    dtype="c16")
    got, want = host(getattr(dpt, op)(dev(cuts))), npf(cuts)
    np.testing.assert_allclose(got, want, rtol=1e-14, atol=1e-15)
    assert np.array_equal(np.signbit(got.real), np.signbit(want.real))
    assert np.array_equal(np.signbit(got.imag), np.signbit(want.imag))
    big = np.array([1e200 + 1e200j, -1e200 + 3j, 5 - 1e300j], dtype="c16")
    np.testing.assert_allclose(host(getattr(dpt, op)(dev(big))), npf(big), rtol=1e-13)


def test_angle_logaddexp_nextafter():
    rng = np.random.default_rng(101)
    z = (rng.standard_normal(3000) + 1j * rng.standard_normal(3000)).astype("c8")
    got = host(dpt.angle(dev(z)))
    assert got.dtype == np.dtype("f4")
    assert_ulp(got, np.angle(z.astype("c16")), 4.0)
    for dt in FLOATS:
        a, b = random_array(rng, 5000, dt, -30, 30), random_array(rng, 5000, dt, -30, 30)
        a[:4] = [np.inf, -np.inf, np.nan, 1.0]
        b[:4] = [np.inf, -np.inf, 1.0, 1.0]
        got = host(dpt.logaddexp(dev(a), dev(b)))
        wide = np.float64 if dt.itemsize <= 4 else np.longdouble
        with np.errstate(all="ignore"):
            want = np.logaddexp(a.astype(wide), b.astype(wide))
            # max(x, y) + log1p(exp(-|x - y|)) (the reference's formula) cancels when the result is
            # near zero: the error is a few ULPs of the operands, not of the result
            scale = np.maximum(np.maximum(np.abs(a), np.abs(b)).astype(wide), np.abs(want))
            fin = np.isfinite(want)
            assert (np.abs(got[fin].astype(wide) - want[fin]) <= 4 * np.finfo(dt).eps * scale[fin]).all()
            assert_same(got[~fin], want[~fin].astype(dt))
        x, y = random_array(rng, 3000, dt, -5, 5), random_array(rng, 3000, dt, -5, 5)
        x[:6] = [0.0, 0.0, -0.0, 1.0, np.inf, np.nan]
        y[:6] = [1.0, -1.0, 0.0, 1.0, 0.0, 0.0]
        want = np.nextafter(x, y)
        # C's rule for equal operands (the second one comes back, so -0.0 -> +0.0 gives +0.0), which NumPy
        # follows for float32/64 but not for float16, where it hands back the first operand
        want = np.where(x == y, y, want).astype(dt)
        assert_same(host(dpt.nextafter(dev(x), dev(y))), want)


# ---- transposed operands (LDS tile kernel) ----------------------------------------------------
def _plan_path(fn_name, *arrays):
    """Kernel the library would use for these operands (last one is the output)."""
    import dpnp_amd._lib as L

    p = L.Plan()
    views = [dpt.broadcast_to(a, arrays[-1].shape)._as_view() for a in arrays]
    if len(arrays) == 2:
        L.check(L.lib.dpx_unary_plan(L.UNARY_ID[fn_name], views[0], views[1], p))
    else:
        L.check(L.lib.dpx_binary_plan(L.BINARY_ID[fn_name], views[0], views[1], views[2], p))
    return L.PATH_NAMES[p.path]


@pytest.mark.parametrize("dt", ["?", "i1", "u2", "f2", "i4", "f4", "i8", "f8", "c8", "c16"])
@pytest.mark.parametrize("shape", [(64, 128), (200, 333), (17, 1000), (1000, 19), (129, 513), (256, 1024), (300, 1100)])
def test_transposed_input_all_widths(dt, shape):
    """out (C-contiguous) = op(A.T): full tiles, ragged edges, lengths that are not a multiple of
    the 16-byte pack (element-wise staging), every item size."""
    rng = np.random.default_rng(101)
    a = random_array(rng, shape[::-1], dt, -50, 50)
    d = dev(a)
    out = dpt.empty(shape, dtype=dt)
    if dt == "?":
        dpt.logical_not(d.T, out=out)
        assert _plan_path("logical_not", d.T, out) == "ew_tile"
        assert_same(host(out), ~a.T)
    else:
        dpt.negative(d.T, out=out)
        assert _plan_path("negative", d.T, out) == "ew_tile"
        assert_same(host(out), orc.unary("negative", np.ascontiguousarray(a.T)))
    if dt != "?":  # allocation by the call itself
        assert_same(host(dpt.positive(d.T, order="C")), np.ascontiguousarray(a.T))


def test_transposed_binary_mixed_operands():
    rng = np.random.default_rng(103)
    m, n = 150, 260
    a = random_array(rng, (n, m), "f4")        # used as a.T: transposed
    b = random_array(rng, (m, n), "f4")        # row oriented
    row = random_array(rng, (1, n), "f4")      # broadcast along dT
    col = random_array(rng, (m, 1), "f4")      # broadcast along the inner dim
    b2 = random_array(rng, (m, 2 * n), "f4")   # stride 2 along the inner dim
    c = random_array(rng, (n, m), "f4")        # second transposed operand
    da, db, drow, dcol, db2, dc = map(dev, (a, b, row, col, b2, c))
    out = dpt.empty((m, n), dtype="f4")
    for name, x, y, hx, hy in [
        ("add", da.T, db, a.T, b),
        ("subtract", db, da.T, b, a.T),
        ("multiply", da.T, drow, a.T, np.broadcast_to(row, (m, n))),
        ("multiply", dcol, da.T, np.broadcast_to(col, (m, n)), a.T),
        ("add", da.T, db2[:, ::2], a.T, b2[:, ::2]),
        ("subtract", da.T, dc.T, a.T, c.T),
        ("add", da.T, da.T, a.T, a.T),
    ]:
        getattr(dpt, name)(x, y, out=out)
        assert _plan_path(name, x, y, out) == "ew_tile", name
        assert_same(host(out), orc.binary(name, np.ascontiguousarray(hx), np.ascontiguousarray(hy)))
    # mixed item sizes: comparison of a transposed float matrix writes bools
    ob = dpt.empty((m, n), dtype="?")
    dpt.greater(da.T, db, out=ob)
    assert _plan_path("greater", da.T, db, ob) == "ew_tile"
    assert_same(host(ob), a.T > b)
    # float64 against transposed float32 after promotion in Python: cast kernel + tile kernel
    d8 = dev(b.astype("f8"))
    assert_same(host(dpt.add(da.T, d8, order="C")), a.T.astype("f8") + b.astype("f8"))
    # where with a transposed condition and transposed branches
    cond = random_array(rng, (n, m), "?")
    assert_same(host(dpt.where(dev(cond).T, da.T, db, order="C")), np.where(cond.T, a.T, b))
    assert_same(host(dpt.where(dev(cond).T, da.T, dc.T, order="C")), np.where(cond.T, a.T, c.T))


def test_transposed_with_batch_dims_offsets_and_strided_output():
    rng = np.random.default_rng(107)
    a = random_array(rng, (3, 70, 5, 90), "i4")
    d = dev(a)
    # swap the two long axes, keep the short ones as batch dims
    v, hv = dpt.permute_dims(d, (0, 3, 2, 1)), np.transpose(a, (0, 3, 2, 1))
    assert_same(host(dpt.multiply(v, 3, order="C")), hv * np.int32(3))
    # views that start inside the allocation: 16-byte alignment is lost for some of them
    for lo in (1, 2, 3, 4):
        w, hw = d[0, lo:, 0, lo:].T, a[0, lo:, 0, lo:].T
        out = dpt.empty(hw.shape, dtype="i4")
        dpt.negative(w, out=out)
        assert_same(host(out), -hw)
    # output that is a row-contiguous slice of a wider matrix
    big = dpt.zeros((90, 200), dtype="i4")
    src, hsrc = d[1, :, 2, :].T, a[1, :, 2, :].T      # (90, 70)
    dpt.negative(src, out=big[:, 7:77])
    want = np.zeros((90, 200), dtype="i4")
    want[:, 7:77] = -hsrc
    assert_same(host(big), want)


# ---- functions of the reference's ufunc extension ----------------------------------------------
@pytest.mark.parametrize("dt", ["f2", "f4", "f8"])
def test_extension_unary_float(dt):
    rng = np.random.default_rng(301)
    a = random_array(rng, 5000, dt, -6, 6)
    a[:8] = [0.0, -0.0, np.inf, -np.inf, np.nan, 1.0, -1.0, 0.5]
    d = dev(a)
    assert_same(host(dpt.fabs(d)), orc.unary("fabs", a))
    sp = host(dpt.spacing(d))
    assert_same(sp, orc.unary("spacing", a))
    tol = 4.0
    for name in ("degrees", "radians"):
        assert_ulp(host(getattr(dpt, name)(d)), getattr(np, name)(a.astype(np.longdouble)), 1.0)
    import mpmath

    mpmath.mp.dps = 40  # sin(pi x) near its zeros needs the exact argument: numpy.sinc rounds pi * x first
    fin = np.isfinite(a)
    exact = np.array([np.longdouble(str(mpmath.sincpi(mpmath.mpf(float(v))))) for v in a[fin]], dtype=np.longdouble)
    got = host(dpt.sinc(d))
    assert_ulp(got[fin], exact, tol if dt != "f2" else 1.0)
    assert np.all(np.isnan(got[np.isnan(a)])) and np.all(got[np.isinf(a)] == 0) | np.all(np.isnan(got[np.isinf(a)]))
    mp_fn = {"erfc": mpmath.erfc, "erfcx": lambda v: mpmath.exp(v * v) * mpmath.erfc(v),
             "i0": lambda v: mpmath.besseli(0, v)}
    for name in ("erfc", "erfcx", "i0"):
        x = (a if name != "erfcx" else np.clip(a, -3, 6))[:1200]   # erfcx grows like exp(x^2) for negative x
        got = host(getattr(dpt, name)(dev(x)))
        assert got.dtype == orc.unary_result_dtype(name, dt), name
        fin = np.isfinite(x)
        # mpmath at 40 digits (scipy's float64 erfc is tens of ULPs off in the far tail)
        exact = np.array([np.longdouble(str(mp_fn[name](mpmath.mpf(float(v))))) for v in x[fin]], dtype=np.longdouble)
        assert_ulp(got[fin], exact, 8.0 if name == "i0" and dt == "f8" else tol)
        if name == "i0":
            assert np.all(got[np.isinf(x)] == np.inf) and np.all(np.isnan(got[np.isnan(x)]))
        elif name == "erfc":
            assert_same(got[~fin], np.array([0.0, 2.0, np.nan], dtype=got.dtype))
    p = random_array(rng, 3000, dt, -0.999, 0.999)
    assert_ulp(host(dpt.erfinv(dev(p))), orc.unary("erfinv", p).astype(np.longdouble), 8.0)
    q = random_array(rng, 3000, dt, 0.001, 1.999)
    assert_ulp(host(dpt.erfcinv(dev(q))), orc.unary("erfcinv", q).astype(np.longdouble), 8.0)
    # outside the domain: NaN; at the ends: infinities
    e = host(dpt.erfinv(dev(np.array([-1.0, 1.0, 2.0], dtype=dt))))
    assert e[0] == -np.inf and e[1] == np.inf and np.isnan(e[2])


def test_extension_sinc_complex_and_bitwise_count():
    rng = np.random.default_rng(303)
    for dt in ("c8", "c16"):
        z = random_array(rng, 2000, dt, -3, 3)
        z[0] = 0
        got = host(dpt.sinc(dev(z)))
        want = np.sinc(z.astype(np.clongdouble))
        np.testing.assert_allclose(got, want.astype(dt), rtol=2e-5 if dt == "c8" else 1e-13)
    for dt in ("i1", "u1", "i2", "u2", "i4", "u4", "i8", "u8"):
        info = np.iinfo(dt)
        a = rng.integers(info.min, info.max, 4000, dtype=dt, endpoint=True)
        a[:3] = [info.min, info.max, 0]
        r = dpt.bitwise_count(dev(a))
        assert r.dtype == np.dtype("u1")
        assert_same(host(r), orc.unary("bitwise_count", a))
    with pytest.raises((ValueError, TypeError)):
        dpt.bitwise_count(dev(np.ones(3, dtype="f4")))


@pytest.mark.parametrize("dt", [d for d in ALL])
def test_extension_fmax_fmin_all_types(dt):
    rng = np.random.default_rng(307)
    a, b = random_array(rng, 3000, dt), random_array(rng, 3000, dt)
    if np.dtype(dt).kind in "fc":
        a[::7] = np.nan
        b[::11] = np.nan
        if np.dtype(dt).kind == "c":
            a[1::13] = complex(1, np.nan)
    for name in ("fmax", "fmin"):
        assert_same(host(getattr(dpt, name)(dev(a), dev(b))), orc.binary(name, a, b))
    if np.dtype(dt).kind == "c":
        # every pair of a grid with signed zeros, infinities and NaN parts (the oracle's rule is pinned on the same
        # grid against a scalar transcription of math_utils.hpp:73-95)
        vals = [0.0, -0.0, 1.0, -1.0, 2.5, np.inf, -np.inf, np.nan]
        grid = np.array([complex(re, im) for re in vals for im in vals], dtype=dt)
        ga, gb = (g.ravel() for g in np.meshgrid(grid, grid, indexing="ij"))
        for name in ("fmax", "fmin", "less_equal", "greater_equal", "less", "greater", "maximum", "minimum"):
            got, want = host(getattr(dpt, name)(dev(ga), dev(gb))), orc.binary(name, ga, gb)
            if want.dtype.kind == "c":
                assert_same(got.real, want.real)
                assert_same(got.imag, want.imag)
            else:
                assert_same(got, want)


def test_extension_binary_misc():
    rng = np.random.default_rng(311)
    for dt in ("i1", "u1", "i2", "u2", "i4", "u4", "i8", "u8"):
        a, b = random_array(rng, 4000, dt, -120, 120), random_array(rng, 4000, dt, -12, 12)
        info = np.iinfo(dt)
        a[:2] = [info.min, info.max]
        b[:2] = [-1 if info.min < 0 else 1, 0]
        assert_same(host(dpt.fmod(dev(a), dev(b))), orc.binary("fmod", a, b))
        a2, b2 = a.copy(), b.copy()
        if info.min < 0:
            a2[a2 == info.min] = 0   # |INT_MIN| is not representable
        assert_same(host(dpt.gcd(dev(a2), dev(b2))), orc.binary("gcd", a2, b2))
        small = (a2 % 50).astype(dt) if info.max < 10**5 else a2
        small_b = (b2 % 11).astype(dt)
        if info.max >= 10**5:
            assert_same(host(dpt.lcm(dev(small), dev(small_b))), orc.binary("lcm", small, small_b))
    r = dpt.fmod(dev(np.array([True, False])), dev(np.array([True, True])))
    assert r.dtype == np.dtype("i1") and host(r).tolist() == [0, 0]
    for dt in ("f2", "f4", "f8"):
        a, b = random_array(rng, 4000, dt, -30, 30), random_array(rng, 4000, dt, -30, 30)
        a[:6] = [0.0, -0.0, np.nan, np.inf, -np.inf, 2.0]
        b[:6] = [0.5, 0.25, 1.0, 1.0, np.inf, np.nan]
        assert_same(host(dpt.heaviside(dev(a), dev(b))), orc.binary("heaviside", a, b))
        fm = host(dpt.fmod(dev(a), dev(b)))
        np.testing.assert_array_equal(fm, np.fmod(a, b))
        got = host(dpt.logaddexp2(dev(a), dev(b)))
        with np.errstate(all="ignore"):
            want = np.logaddexp2(a.astype(np.longdouble), b.astype(np.longdouble))
        ok = np.isfinite(want)
        # the reference's formula max + log2(1 + 2**-|d|) cancels near zero: ULPs of the operands
        scale = np.maximum(np.maximum(np.abs(a), np.abs(b)).astype(np.longdouble), np.abs(want))
        assert (np.abs(got[ok].astype(np.longdouble) - want[ok]) <= 4 * np.finfo(dt).eps * scale[ok]).all()
        assert np.array_equal(np.isnan(got), np.isnan(want.astype(dt)))
    with pytest.raises((ValueError, TypeError)):
        dpt.gcd(dev(np.ones(3, dtype="f4")), dev(np.ones(3, dtype="f4")))


# ---- mixed-dtype arithmetic: the cast of one operand is folded into the kernel -------------------
@pytest.mark.parametrize("op", ["add", "subtract", "multiply", "divide"])
@pytest.mark.parametrize("pair", [("f8", "f4"), ("f8", "i4"), ("f8", "i8"), ("f8", "?"), ("f4", "?"), ("f4", "i2"),
                                  ("f4", "i1"), ("f4", "u1")])
def test_mixed_dtype_arithmetic_equals_cast_then_compute(op, pair):
    import dpnp_amd._lib as L
    from dpnp_amd.tensor._dtypes import dtype_id

    rng = np.random.default_rng(151)
    wide, narrow = pair
    a = random_array(rng, (37, 130), wide, -9, 9)
    b = random_array(rng, (37, 130), narrow, -9, 9)
    if narrow != "?":
        b[b == 0] = 1
    assert L.lib.dpx_binary_fused_cast_result_type(L.BINARY_ID[op], dtype_id(np.dtype(wide)),
                                                   dtype_id(np.dtype(narrow))) == dtype_id(np.dtype(wide))
    for x, y in ((a, b), (b, a)):
        with np.errstate(all="ignore"):
            want = getattr(np, op if op != "divide" else "true_divide")(x.astype(wide), y.astype(wide))
        assert_same(host(getattr(dpt, op)(dev(x), dev(y))), want)                       # contiguous
        assert_same(host(getattr(dpt, op)(dev(x)[:, ::2], dev(y)[:, ::2])), want[:, ::2])  # strided
        assert_same(host(getattr(dpt, op)(dev(x.T.copy()).T, dev(y))), want)            # transposed operand
    # in place: the left operand has the result type
    d = dev(a)
    getattr(dpt, op)(d, dev(b), out=d)
    with np.errstate(all="ignore"):
        assert_same(host(d), getattr(np, op if op != "divide" else "true_divide")(a, b.astype(wide)))
    d2 = dev(a)
    if op == "add":
        d2 += dev(b)
        assert_same(host(d2), a + b.astype(wide))


@pytest.mark.parametrize("dt", ["?", "i1", "u2", "i4", "i8", "f2", "f4", "f8", "c8", "c16"])
def test_calls_that_only_write_outer_forms(dt):
    # a row vector with one value per row (an outer sum, a row minus a column, 3-d forms of the same): blocks of 64
    # rows, the per-row values handed from lane to lane.  Every row and column count around the block's edges, both
    # operand orders, results of another type (comparisons), rows of a wider matrix as output, a column read
    # backwards, and the same calls through dpnp's `outer`
    import dpnp_amd as dpnp

    rng = np.random.default_rng(61)
    ops = ["add", "subtract", "multiply", "less", "maximum"] if dt not in ("c8", "c16") else ["add", "subtract", "multiply", "equal"]
    if dt == "?":
        ops = ["logical_and", "logical_xor", "add", "not_equal"]
    for rows, cols in ((16, 64), (17, 67), (63, 256), (64, 1024), (65, 1031), (130, 4100), (1000, 259), (20, 20000)):
        r = random_array(rng, (1, cols), dt, -50, 50)
        c = random_array(rng, (rows, 1), dt, -50, 50)
        for op in ops:
            f = getattr(np, op)
            with np.errstate(all="ignore"):
                if op == "multiply" and dt in ("c8", "c16"):  # (the last bit of a complex product depends on fusion)
                    tol = 1e-6 if dt == "c8" else 1e-14
                    np.testing.assert_allclose(host(dpt.multiply(dev(r), dev(c))), f(r, c), rtol=tol, atol=tol * 2500)
                    np.testing.assert_allclose(host(dpt.multiply(dev(c), dev(r))), f(c, r), rtol=tol, atol=tol * 2500)
                    continue
                assert_same(host(getattr(dpt, op)(dev(r), dev(c))), f(r, c))
                assert_same(host(getattr(dpt, op)(dev(c), dev(r))), f(c, r))
    r = random_array(rng, (1, 777), dt, -50, 50)
    c = random_array(rng, (300, 1), dt, -50, 50)
    op = ops[1]
    with np.errstate(all="ignore"):
        want = getattr(np, op)(r, c[::-1])
    assert_same(host(getattr(dpt, op)(dev(r), dev(c)[::-1])), want)                    # the column read backwards
    big = dpt.zeros((300, 1000), dtype=want.dtype)
    getattr(dpt, op)(dev(r), dev(c)[::-1], out=big[:, 100:877])                         # rows of a wider matrix
    assert_same(host(big)[:, 100:877], want)
    assert not host(big)[:, :100].any() and not host(big)[:, 877:].any()
    # three dims: (B, 1, C) with (1, M, 1), and (B, M, 1) with (1, 1, C)
    p3, q3 = random_array(rng, (5, 1, 300), dt, -50, 50), random_array(rng, (1, 70, 1), dt, -50, 50)
    u3, v3 = random_array(rng, (5, 70, 1), dt, -50, 50), random_array(rng, (1, 1, 300), dt, -50, 50)
    with np.errstate(all="ignore"):
        assert_same(host(getattr(dpt, op)(dev(p3), dev(q3))), getattr(np, op)(p3, q3))
        assert_same(host(getattr(dpt, op)(dev(u3), dev(v3))), getattr(np, op)(u3, v3))
    # pairwise forms, X[:, None, :] with Y[None, :, :]: one operand's vector moves with the rows, the other's stays
    for n, m, d in ((7, 40, 64), (3, 17, 257), (20, 9, 1000)):
        xa, ya = random_array(rng, (n, 1, d), dt, -50, 50), random_array(rng, (1, m, d), dt, -50, 50)
        with np.errstate(all="ignore"):
            assert_same(host(getattr(dpt, op)(dev(xa), dev(ya))), getattr(np, op)(xa, ya))
            assert_same(host(getattr(dpt, op)(dev(ya), dev(xa))), getattr(np, op)(ya, xa))
    if dt in ("f4", "f8", "i4"):
        x, y = random_array(rng, (500,), dt, -50, 50), random_array(rng, (333,), dt, -50, 50)
        assert_same(dpnp.asnumpy(dpnp.multiply.outer(dpnp.array(x), dpnp.array(y))), np.multiply.outer(x, y))
        assert_same(dpnp.asnumpy(dpnp.subtract.outer(dpnp.array(x), dpnp.array(y))), np.subtract.outer(x, y))


@pytest.mark.parametrize("op", ["add", "subtract", "multiply", "divide"])
@pytest.mark.parametrize("idt", ["i4", "i8"])
def test_float32_with_integer_gives_float64_in_one_kernel(op, idt):
    # float32 (op) int32 / int64 promotes to float64 (the reference casts both operands into temporaries, then
    # computes): one kernel converts both while reading; the values are those of cast-then-compute
    import dpnp_amd._lib as L
    from dpnp_amd.tensor._dtypes import dtype_id

    rng = np.random.default_rng(152)
    a = random_array(rng, (37, 130), "f4", -9, 9)
    b = random_array(rng, (37, 130), idt, -9, 9)
    b[b == 0] = 3
    assert L.lib.dpx_binary_fused_cast_result_type(L.BINARY_ID[op], L.FLOAT, dtype_id(np.dtype(idt))) == L.DOUBLE
    npf = getattr(np, op if op != "divide" else "true_divide")
    for x, y in ((a, b), (b, a)):
        want = npf(x.astype("f8"), y.astype("f8"))
        got = getattr(dpt, op)(dev(x), dev(y))
        assert got.dtype == np.dtype("f8")
        assert_same(host(got), want)
        assert_same(host(getattr(dpt, op)(dev(x)[:, ::2], dev(y)[:, ::2])), want[:, ::2])
        assert_same(host(getattr(dpt, op)(dev(x.T.copy()).T, dev(y))), want)
        out = dpt.empty((37, 130), dtype="f8")
        getattr(dpt, op)(dev(x), dev(y), out=out)
        assert_same(host(out), want)
        assert_same(host(getattr(dpt, op)(dev(x), dev(y[:1]))), npf(x.astype("f8"), y[:1].astype("f8")))  # a broadcast row
    big = random_array(rng, (1 << 16,), "i8", -2 ** 62, 2 ** 62)  # integers float64 cannot hold exactly: rounded once
    f = random_array(rng, (1 << 16,), "f4", -9, 9)
    assert_same(host(getattr(dpt, op)(dev(big), dev(f))), npf(big.astype("f8"), f.astype("f8")))


@pytest.mark.parametrize("dt", ["i4", "u4"])
def test_floor_divide_of_32_bit_integers_on_hard_quotients(dt):
    """32-bit floor_divide goes through the double quotient: extremes, divisors of every size and sign, quotients
    that miss an integer by 1 / b, zero divisors (result 0, floor_divide.hpp:63-86), -2^31 // -1 (wraps)."""
    rng = np.random.default_rng(4242)
    info = np.iinfo(dt)
    edge = np.array([info.min, info.min + 1, -2, -1, 0, 1, 2, 3, 7, 46341, 65535, 65536, info.max - 1, info.max],
                    dtype=np.int64)
    edge = edge[(edge >= info.min) & (edge <= info.max)]
    a = np.concatenate([np.repeat(edge, len(edge)), rng.integers(info.min, info.max, 200000, endpoint=True)])
    b = np.concatenate([np.tile(edge, len(edge)), rng.integers(info.min, info.max, 200000, endpoint=True)])
    # k * b - 1, k * b, k * b + 1: quotients next to an integer
    bb = rng.integers(1, 1 << 16, 100000)
    kk = rng.integers(0, (info.max // (1 << 16)), 100000)
    for off in (-1, 0, 1):
        a = np.concatenate([a, np.clip(kk * bb + off, info.min, info.max)])
        b = np.concatenate([b, bb if dt == "u4" else bb * rng.choice([-1, 1], bb.size)])
    a, b = a.astype(dt), b.astype(dt)
    want = orc.binary("floor_divide", a, b)
    assert_same(host(dpt.floor_divide(dev(a), dev(b))), want)
    assert_same(host(dpt.remainder(dev(a), dev(b))), orc.binary("remainder", a, b))  # the same quotient
    # against a scalar divisor
    for d in ((7, 1, 3) if dt == "u4" else (7, -7, -1, 1)):
        x = dev(a)
        assert_same(host(dpt.floor_divide(x, d)), orc.binary("floor_divide", a, np.full_like(a, d)))
        assert_same(host(dpt.remainder(x, d)), orc.binary("remainder", a, np.full_like(a, d)))
