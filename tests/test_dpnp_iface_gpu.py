"""The NumPy-flavoured surface: keyword handling of ufuncs and reductions, methods and operators
(behaviour of dpnp/tests/test_mathematical.py, test_sum.py, test_statistics.py, test_search.py)."""
import numpy as np
import pytest

import dpnp_amd as dpnp
from tests.helpers import assert_same

pytestmark = pytest.mark.gpu


def test_array_roundtrip_and_views():
    a = np.arange(24, dtype="f4").reshape(4, 6)
    x = dpnp.array(a)
    assert isinstance(x, dpnp.ndarray) and x.shape == (4, 6) and x.strides == a.strides
    assert_same(x.asnumpy(), a)
    assert_same(x[:, ::2].asnumpy(), a[:, ::2])
    assert_same(x.T.asnumpy(), a.T)
    assert_same(dpnp.asnumpy(x[1]), a[1])
    assert_same(x.reshape(6, 4).asnumpy(), a.reshape(6, 4))
    assert_same(dpnp.asarray([[1, 2], [3, 4]]).asnumpy(), np.array([[1, 2], [3, 4]]))
    x[0, :] = 5
    a[0, :] = 5
    assert_same(x.asnumpy(), a)
    assert float(x[1, 1]) == a[1, 1] and x[1, 1].item() == a[1, 1]


def test_ufunc_keywords():
    a = np.linspace(-2, 2, 50, dtype="f4")
    x = dpnp.array(a)
    assert_same(dpnp.add(x, x).asnumpy(), a + a)
    out = dpnp.empty(50, dtype="f4")
    assert dpnp.multiply(x, 3, out=out) is out
    assert_same(out.asnumpy(), a * np.float32(3))
    r = dpnp.add(x, x, dtype="f8")
    assert r.dtype == np.dtype("f8")
    assert_same(r.asnumpy(), a.astype("f8") * 2)
    with pytest.raises(TypeError):
        dpnp.add(x, x, out=out, dtype="f8")
    with pytest.raises(NotImplementedError):
        dpnp.add(x, x, where=False)
    with pytest.raises(NotImplementedError):
        dpnp.exp(x, subok=False)
    with pytest.raises(ValueError):
        dpnp.add(x, x, order="Z")
    with pytest.raises(TypeError):
        dpnp.add(1, 2)
    with pytest.raises(TypeError):
        dpnp.exp([1.0, 2.0])
    y = dpnp.array(a)
    assert dpnp.add(y, 1, out=y) is y  # in-place kernel
    assert_same(y.asnumpy(), a + 1)
    np.testing.assert_allclose(dpnp.exp(x).asnumpy(), np.exp(a), rtol=1e-6)
    assert dpnp.exp(dpnp.arange(5)).dtype == np.dtype("f8")  # ints are cast to the default float
    assert_same((x > 0).asnumpy(), a > 0)
    assert_same((-x + 2 * x - x / 4).asnumpy(), (-a + 2 * a - a / 4))
    i = dpnp.arange(10, dtype="i4")
    assert_same((i & 6).asnumpy(), np.arange(10, dtype="i4") & 6)
    assert_same((i // 3).asnumpy(), np.arange(10, dtype="i4") // 3)
    assert_same((i % 3).asnumpy(), np.arange(10, dtype="i4") % 3)
    assert_same((i ** 2).asnumpy(), np.arange(10, dtype="i4") ** 2)


@pytest.mark.parametrize("x_shape", [(), (2,), (3, 4), (3, 4, 5)])
@pytest.mark.parametrize("y_shape", [(), (2,), (3, 4), (3, 4, 5)])
def test_elementwise_outer(x_shape, y_shape):
    # (the cases of test_elemenwise_outer and test_elemenwise_outer_scalar, dpnp/tests/test_mathematical.py:2833-2862;
    # the products and sums of two float64 numbers are exact or rounded once, alike on both sides)
    rng = np.random.default_rng(len(x_shape) * 4 + len(y_shape))
    a, b = rng.random(x_shape), rng.random(y_shape)
    x, y = dpnp.asarray(a), dpnp.asarray(b)
    for name in ("multiply", "add", "greater", "maximum"):
        got = getattr(dpnp, name).outer(x, y)
        want = getattr(np, name).outer(a, b)
        assert got.shape == want.shape == tuple(x_shape) + tuple(y_shape)
        assert_same(got.asnumpy(), want)
    out = dpnp.empty(tuple(x_shape) + tuple(y_shape), dtype="f8")
    assert dpnp.subtract.outer(x, y, out=out) is out
    assert_same(out.asnumpy(), np.subtract.outer(a, b))
    assert_same(dpnp.add.outer(x, 5).asnumpy(), a + 5)
    assert_same(dpnp.add.outer(5, y).asnumpy(), 5 + b)
    with pytest.raises(TypeError):
        dpnp.add.outer(2, 3)
    with pytest.raises(NotImplementedError):
        dpnp.add.outer(x, y, where=False)


def test_where():
    a = np.array([[0, 1, 2], [0, 2, 4], [0, 3, 6]])
    x = dpnp.array(a)
    assert_same(dpnp.where(x < 4, x, -1).asnumpy(), np.where(a < 4, a, -1))
    with pytest.raises(ValueError):
        dpnp.where(x < 4, x)
    f = dpnp.array(a.astype("f4"))
    r = dpnp.where_compare("greater", f, 0, f, 7)
    assert_same(r.asnumpy(), np.where(a > 0, a, 7).astype("f4"))


def test_reductions_keywords():
    rng = np.random.default_rng(83)
    a = rng.standard_normal((20, 30)).astype("f4")
    x = dpnp.array(a)
    np.testing.assert_allclose(dpnp.sum(x).asnumpy(), a.sum(dtype="f8"), rtol=1e-5)
    np.testing.assert_allclose(x.sum(axis=0).asnumpy(), a.sum(axis=0, dtype="f8"), rtol=1e-4, atol=1e-5)
    assert dpnp.sum(x, dtype="f8").dtype == np.dtype("f8")
    assert dpnp.sum(dpnp.ones(10, dtype="i4")).dtype == np.dtype("i8")
    o = dpnp.empty(20, dtype="f8")  # out of another dtype receives a cast of the result
    assert dpnp.sum(x, axis=1, out=o) is o
    np.testing.assert_allclose(o.asnumpy(), a.sum(axis=1, dtype="f8"), rtol=1e-5, atol=1e-5)
    with pytest.raises(NotImplementedError):
        dpnp.sum(x, initial=1)
    with pytest.raises(NotImplementedError):
        dpnp.max(x, where=False)
    assert_same(dpnp.max(x, axis=1).asnumpy(), a.max(axis=1))
    assert_same(x.min(axis=0, keepdims=True).asnumpy(), a.min(axis=0, keepdims=True))
    assert_same(dpnp.argmax(x).asnumpy(), np.array(a.argmax()))
    assert_same(x.argmin(axis=1).asnumpy(), a.argmin(axis=1))
    oi = dpnp.empty(30, dtype="i8")
    assert dpnp.argmax(x, axis=0, out=oi) is oi
    assert_same(oi.asnumpy(), a.argmax(axis=0))
    with pytest.raises(TypeError):
        dpnp.argmax(x, axis=0, out=dpnp.empty(30, dtype="f8"))
    np.testing.assert_allclose(dpnp.mean(x, axis=1).asnumpy(), a.mean(axis=1, dtype="f8"), rtol=1e-5, atol=1e-6)
    np.testing.assert_allclose(x.var(ddof=1).asnumpy(), a.astype("f8").var(ddof=1), rtol=1e-5)
    np.testing.assert_allclose(dpnp.std(x, axis=0).asnumpy(), a.astype("f8").std(axis=0), rtol=1e-5)
    m64 = dpnp.mean(x, dtype="f8")
    assert m64.dtype == np.dtype("f8")
    np.testing.assert_allclose(float(m64), a.astype("f8").mean(), rtol=1e-12)
    v64 = dpnp.var(x, dtype="f8")
    np.testing.assert_allclose(float(v64), a.astype("f8").var(), rtol=1e-12)
    assert dpnp.mean(dpnp.arange(5)).dtype == np.dtype("f8")


def test_black_scholes_entry_point():
    rng = np.random.default_rng(4)
    n = 10007
    p, s, t = rng.uniform(10, 50, n), rng.uniform(10, 50, n), rng.uniform(1, 2, n)
    call, put = dpnp.black_scholes(dpnp.array(p), dpnp.array(s), dpnp.array(t), 0.1, 0.2)
    from oracle import oracle as orc

    wc, wp = orc.black_scholes(p, s, t, 0.1, 0.2)
    np.testing.assert_allclose(call.asnumpy(), wc, rtol=1e-12, atol=1e-12)
    np.testing.assert_allclose(put.asnumpy(), wp, rtol=1e-12, atol=1e-12)
    # the same chain through separate kernels, as the reference runs it (examples/example_bs.py:50-78)
    P, S, T = dpnp.array(p), dpnp.array(s), dpnp.array(t)
    a = dpnp.log(P / S)
    b = T * -0.1
    z = T * (0.2 * 0.2 * 2)
    c = 0.25 * z
    y = 1.0 / dpnp.sqrt(z)
    w1, w2 = (a - b + c) * y, (a - b - c) * y
    d1, d2 = 0.5 + 0.5 * dpnp.erf(w1), 0.5 + 0.5 * dpnp.erf(w2)
    Se = dpnp.exp(b) * S
    r = P * d1 - Se * d2
    # fused against unfused: the fused kernel's own elementary functions are each good to an ULP of
    # their result, which the difference of the two products turns into a few ULP of the larger one
    scale = np.maximum(p, s)
    assert np.all(np.abs(call.asnumpy() - r.asnumpy()) <= 8 * np.finfo("f8").eps * scale)
    assert np.all(np.abs(put.asnumpy() - (r - P + Se).asnumpy()) <= 8 * np.finfo("f8").eps * scale)
    # inputs the short routines do not take (zero, negative, subnormal, infinite, NaN, huge maturities)
    # go through the long ones and give what the chain gives, bit for bit
    bad = np.array([0.0, -1.0, 5e-324, np.inf, np.nan, 30.0, 30.0, 30.0])
    pb, sb, tb = np.full(8, 30.0), np.full(8, 25.0), np.full(8, 1.5)
    pb[:5] = bad[:5]
    sb[5], tb[6], tb[7] = 0.0, np.nan, 1e300
    for arr in (pb, sb, tb):
        assert arr.shape == (8,)
    cb, qb = dpnp.black_scholes(dpnp.array(pb), dpnp.array(sb), dpnp.array(tb), 0.1, 0.2)
    with np.errstate(all="ignore"):
        wc, wp = orc.black_scholes(pb, sb, tb, 0.1, 0.2)
    fin = np.isfinite(wc)
    assert np.array_equal(np.isnan(cb.asnumpy()), np.isnan(wc)) and np.array_equal(np.isnan(qb.asnumpy()), np.isnan(wp))
    np.testing.assert_allclose(cb.asnumpy()[fin], wc[fin], rtol=1e-12, atol=1e-12)
    # the same inputs scattered over full chunks of the long array: their waves take the long routines,
    # the other waves the short ones
    where = np.array([3, 1000, 4100, 8191, 8200, 2047, 6000, 10006])
    p2, s2, t2 = p.copy(), s.copy(), t.copy()
    p2[where], s2[where], t2[where] = pb, sb, tb
    c2, q2 = dpnp.black_scholes(dpnp.array(p2), dpnp.array(s2), dpnp.array(t2), 0.1, 0.2)
    with np.errstate(all="ignore"):
        wc, wp = orc.black_scholes(p2, s2, t2, 0.1, 0.2)
    for got, want in ((c2.asnumpy(), wc), (q2.asnumpy(), wp)):
        fin = np.isfinite(want)
        assert np.array_equal(np.isnan(got), np.isnan(want))
        assert np.array_equal(got[~fin & ~np.isnan(want)], want[~fin & ~np.isnan(want)])
        np.testing.assert_allclose(got[fin], want[fin], rtol=1e-12, atol=1e-12)


def test_black_scholes_wide_ranges():
    """Prices and strikes over five decades, maturities from a thousandth of a year to thirty
    years: options deep in and out of the money (erf saturates), tiny and large variances."""
    from oracle import oracle as orc

    rng = np.random.default_rng(8)
    n = 3 * 4096 + 77
    p, s = 10.0 ** rng.uniform(-2, 3, n), 10.0 ** rng.uniform(-2, 3, n)
    t = 10.0 ** rng.uniform(-3, 1.5, n)
    for rate, vol in ((0.1, 0.2), (0.0, 0.05), (-0.01, 1.5)):
        call, put = dpnp.black_scholes(dpnp.array(p), dpnp.array(s), dpnp.array(t), rate, vol)
        wc, wp = orc.black_scholes(p, s, t, rate, vol)
        scale = np.maximum(p, s * np.exp(-rate * t))
        # a rounding error of the logarithm (or of rate * t) reaches erf's argument multiplied by
        # 1 / sqrt(2 vol^2 t), and erf' <= 1.13: the bound any two correct evaluations differ by
        z = 2 * vol * vol * t
        cond = (np.abs(np.log(p / s)) + np.abs(rate * t) + 0.25 * z) / np.sqrt(z)
        tol = np.finfo("f8").eps * scale * (4 + 4 * cond)
        for got, want in ((call.asnumpy(), wc), (put.asnumpy(), wp)):
            assert np.all(np.isfinite(got))
            assert np.all(np.abs(got - want) <= 1e-12 * np.abs(want) + tol)


# ---- dpnp-level functions built on the ufunc extension kernels ---------------------------------
def test_nan_to_num_reference_examples():
    # docstring of dpnp.nan_to_num, dpnp/dpnp_iface_mathematical.py:3640-3670
    x = np.array([np.inf, -np.inf, np.nan, -128, 128])
    d = dpnp.array(x)
    np.testing.assert_array_equal(dpnp.nan_to_num(d).asnumpy(), np.nan_to_num(x))
    np.testing.assert_array_equal(dpnp.nan_to_num(d, nan=-9999, posinf=33333333, neginf=33333333).asnumpy(),
                                  np.nan_to_num(x, nan=-9999, posinf=33333333, neginf=33333333))
    y = np.array([complex(np.inf, np.nan), np.nan, complex(np.nan, np.inf)])
    np.testing.assert_array_equal(dpnp.nan_to_num(dpnp.array(y), nan=111111, posinf=222222).asnumpy(),
                                  np.nan_to_num(y, nan=111111, posinf=222222))
    for dt in ("f2", "f4", "c8"):
        z = x.astype(dt)
        np.testing.assert_array_equal(dpnp.nan_to_num(dpnp.array(z)).asnumpy(), np.nan_to_num(z))
    i = dpnp.array(np.arange(4))
    assert dpnp.nan_to_num(i) is not i and dpnp.nan_to_num(i, copy=False) is i
    w = dpnp.array(x)
    assert dpnp.nan_to_num(w, copy=False) is w
    np.testing.assert_array_equal(w.asnumpy(), np.nan_to_num(x))
    # strided input
    s = dpnp.array(np.tile(x, 7))[::3]
    np.testing.assert_array_equal(dpnp.nan_to_num(s).asnumpy(), np.nan_to_num(np.tile(x, 7)[::3]))


def test_isclose_reference_examples():
    # docstring of dpnp.isclose, dpnp/dpnp_iface_logic.py:870-900
    cases = [([1e10, 1e-7], [1.00001e10, 1e-8], {}), ([1e10, 1e-8], [1.00001e10, 1e-9], {}),
             ([1e10, 1e-8], [1.0001e10, 1e-9], {}), ([1.0, np.nan], [1.0, np.nan], {}),
             ([1.0, np.nan], [1.0, np.nan], {"equal_nan": True}), ([0.0, 0.0], [1e-8, 1e-7], {}),
             ([0.0, 0.0], [1e-100, 1e-7], {"atol": 0.0}), ([1e-10, 1e-10], [1e-20, 0.0], {}),
             ([1e-10, 1e-10], [1e-20, 0.999999e-10], {"atol": 0.0}),
             ([np.inf, -np.inf, np.inf], [np.inf, np.inf, 1.0], {})]
    for a, b, kw in cases:
        got = dpnp.isclose(dpnp.array(a), dpnp.array(b), **kw).asnumpy()
        np.testing.assert_array_equal(got, np.isclose(np.array(a), np.array(b), **kw))
    rng = np.random.default_rng(401)
    a = rng.standard_normal((40, 50)).astype("f4")
    b = a + rng.standard_normal((1, 50)).astype("f4") * 1e-5
    np.testing.assert_array_equal(dpnp.isclose(dpnp.array(a), dpnp.array(b)[0:1]).asnumpy(), np.isclose(a, b[0:1]))
    np.testing.assert_array_equal(dpnp.isclose(dpnp.array(a), 0.5, atol=0.1).asnumpy(), np.isclose(a, 0.5, atol=0.1))
    z = (a + 1j * a.T[:40, :40].repeat(2, axis=1)[:, :50]).astype("c8")
    np.testing.assert_array_equal(dpnp.isclose(dpnp.array(z), dpnp.array(z * (1 + 1e-6))).asnumpy(),
                                  np.isclose(z, z * (1 + 1e-6)))
    ints = np.arange(10)
    np.testing.assert_array_equal(dpnp.isclose(dpnp.array(ints), dpnp.array(ints + 1), atol=1).asnumpy(),
                                  np.isclose(ints, ints + 1, atol=1))


def test_float_power_divmod_modf_aliases():
    rng = np.random.default_rng(403)
    a = rng.integers(1, 9, 50).astype("i4")
    b = rng.integers(-3, 4, 50).astype("i4")
    r = dpnp.float_power(dpnp.array(a), dpnp.array(b))
    assert r.dtype == np.dtype("f8")
    np.testing.assert_allclose(r.asnumpy(), np.float_power(a, b), rtol=1e-15)
    x = rng.uniform(-20, 20, 300).astype("f4")
    y = rng.uniform(-5, 5, 300).astype("f4")
    q, m = dpnp.divmod(dpnp.array(x), dpnp.array(y))
    wq, wm = np.divmod(x, y)
    np.testing.assert_array_equal(q.asnumpy(), wq)
    np.testing.assert_allclose(m.asnumpy(), wm, rtol=1e-6, atol=1e-6)
    qi, mi = dpnp.divmod(dpnp.array(a), dpnp.array(np.where(b == 0, 1, b).astype("i4")))
    wqi, wmi = np.divmod(a, np.where(b == 0, 1, b).astype("i4"))
    np.testing.assert_array_equal(qi.asnumpy(), wqi)
    np.testing.assert_array_equal(mi.asnumpy(), wmi)
    v = np.array([2.5, -2.5, 0.0, -0.0, np.inf, -np.inf, np.nan, 7.0], dtype="f8")
    f, w = dpnp.modf(dpnp.array(v))
    wf, ww = np.modf(v)
    np.testing.assert_array_equal(f.asnumpy(), wf)
    np.testing.assert_array_equal(w.asnumpy(), ww)
    np.testing.assert_array_equal(np.signbit(f.asnumpy()), np.signbit(wf))
    np.testing.assert_allclose(dpnp.rad2deg(dpnp.array(x)).asnumpy(), np.rad2deg(x), rtol=1e-6)
    np.testing.assert_allclose(dpnp.deg2rad(dpnp.array(x)).asnumpy(), np.deg2rad(x), rtol=1e-6)
    np.testing.assert_array_equal(dpnp.fmax(dpnp.array(x), np.float32(0.5)).asnumpy(), np.fmax(x, np.float32(0.5)))
    np.testing.assert_array_equal(dpnp.gcd(dpnp.array(a), 6).asnumpy(), np.gcd(a, 6))


# ---- host <-> device transfers through the pinned staging pool ------------------------------------
@pytest.mark.parametrize("nbytes", [1, 4095, (1 << 20) + 1, (16 << 20), (16 << 20) + 7, 5 * (16 << 20) + 12345])
def test_staged_transfers_round_trip(nbytes):
    rng = np.random.default_rng(nbytes % 1000)
    h = rng.integers(0, 256, nbytes, dtype=np.uint8)
    d = dpnp.array(h)
    back = d.asnumpy()
    assert back.dtype == h.dtype and np.array_equal(back, h)
    # a second upload reuses the staging buffers while the first download may still be pending
    h2 = h[::-1].copy()
    d2 = dpnp.array(h2)
    assert np.array_equal((d2 + np.uint8(1)).asnumpy(), h2 + np.uint8(1))
    assert np.array_equal(d.asnumpy(), h)


def test_transfer_entry_points_through_the_c_abi():
    import dpnp_amd._lib as L
    from dpnp_amd.tensor import _device

    n = (3 << 20) + 5
    h = np.random.default_rng(7).integers(0, 256, n, dtype=np.uint8)
    buf = _device.alloc(n)
    stream = _device.current_stream_ptr()
    L.check(L.lib.dpx_copy_from_host(buf.data_ptr(), h.ctypes.data, n, stream))
    if L.torch is not None:
        assert np.array_equal(buf.cpu().numpy(), h)
    out = np.zeros(n, dtype=np.uint8)
    L.check(L.lib.dpx_copy_to_host(out.ctypes.data, buf.data_ptr(), n, stream))
    assert np.array_equal(out, h)
    assert L.lib.dpx_copy_to_host(out.ctypes.data, buf.data_ptr(), 0, stream) == 0
    assert L.lib.dpx_copy_from_host(None, h.ctypes.data, 8, stream) != 0  # null pointer: an error, no crash
    assert b"null" in L.lib.dpx_last_error()


def test_copy_and_layout_constructors():
    # dpnp/tests/test_arraycreation.py: copy / ascontiguousarray / asfortranarray / asanyarray / full_like / linspace
    rng = np.random.default_rng(5)
    a = rng.normal(size=(37, 53)).astype("f4")
    d = dpnp.asarray(a)
    for order in ("C", "F", "K", "A"):
        c = dpnp.copy(d.T, order=order)
        want = np.copy(a.T, order=order)
        np.testing.assert_array_equal(c.asnumpy(), want)
        assert c.flags.c_contiguous == want.flags.c_contiguous and c.flags.f_contiguous == want.flags.f_contiguous
        assert c.get_array()._buf is not d.get_array()._buf
    c = dpnp.copy([[1, 2], [3, 4]])
    np.testing.assert_array_equal(c.asnumpy(), [[1, 2], [3, 4]])
    cc = dpnp.ascontiguousarray(d.T)
    assert cc.flags.c_contiguous and cc.shape == (53, 37)
    np.testing.assert_array_equal(cc.asnumpy(), a.T)
    assert dpnp.ascontiguousarray(d).get_array()._buf is d.get_array()._buf  # already C: no copy
    ff = dpnp.asfortranarray(d, dtype="f8")
    assert ff.flags.f_contiguous and ff.dtype == np.float64
    np.testing.assert_array_equal(ff.asnumpy(), a.astype("f8"))
    assert dpnp.ascontiguousarray(3.5).shape == (1,) and dpnp.asfortranarray(2).shape == (1,)
    assert dpnp.asanyarray(d) is d or dpnp.asanyarray(d).get_array()._buf is d.get_array()._buf
    np.testing.assert_array_equal(dpnp.asanyarray([1, 2, 3], dtype="i2").asnumpy(), np.array([1, 2, 3], "i2"))
    f = dpnp.full_like(d, 7, dtype="i4")
    assert f.shape == d.shape and f.dtype == np.int32 and (f.asnumpy() == 7).all()
    f = dpnp.full_like(d, 2.5, shape=(3, 2))
    assert f.shape == (3, 2) and f.dtype == np.float32 and (f.asnumpy() == 2.5).all()
    for num, endpoint in ((11, True), (10, False), (1, True)):
        r = dpnp.linspace(0, 5, num, endpoint=endpoint)
        np.testing.assert_allclose(r.asnumpy(), np.linspace(0, 5, num, endpoint=endpoint), rtol=1e-15)
    r, step = dpnp.linspace(1, 2, 5, dtype="f4", retstep=True)
    assert r.dtype == np.float32 and step == 0.25
    with pytest.raises(NotImplementedError):
        dpnp.copy(d, subok=True)


@pytest.mark.parametrize("fdt", ["f2", "f4", "f8"])
@pytest.mark.parametrize("idt", ["i1", "i2", "i4", "i8"])
def test_ldexp_matrix(fdt, idt):
    # dpnp/tests/test_mathematical.py (TestLdexp): float x int -> float, result bit-exact (ldexp is exact)
    rng = np.random.default_rng(21)
    a = rng.uniform(-8, 8, 4099).astype(fdt)
    a[:6] = [0.0, -0.0, np.inf, -np.inf, np.nan, 1.0]
    lim = 20 if fdt == "f2" else 100
    b = rng.integers(-lim, lim, 4099).astype(idt)
    with np.errstate(all="ignore"):
        want = np.ldexp(a, b)
    got = dpnp.ldexp(dpnp.asarray(a), dpnp.asarray(b))
    assert_same(got.asnumpy(), want)
    # broadcast, strided views and a scalar exponent
    m = rng.uniform(-2, 2, (17, 33)).astype(fdt)
    e = rng.integers(-5, 6, (33,)).astype(idt)
    assert_same(dpnp.ldexp(dpnp.asarray(m), dpnp.asarray(e)).asnumpy(), np.ldexp(m, e))
    assert_same(dpnp.ldexp(dpnp.asarray(m).T, dpnp.asarray(e)[:17]).asnumpy(), np.ldexp(m.T, e[:17]))
    assert_same(dpnp.ldexp(dpnp.asarray(m)[::2, 1::2], 3).asnumpy(), np.ldexp(m[::2, 1::2], 3))
    o = dpnp.empty(m.shape, dtype=fdt)
    r = dpnp.ldexp(dpnp.asarray(m), dpnp.asarray(e), out=o)
    assert r is o
    assert_same(o.asnumpy(), np.ldexp(m, e))


def test_ldexp_promotions_and_limits():
    x = dpnp.asarray(np.array([1, 2, 3], "i4"))
    r = dpnp.ldexp(x, dpnp.asarray(np.array([1, 2, 3], "u2")))
    assert r.dtype == np.float64
    assert_same(r.asnumpy(), np.array([2.0, 8.0, 24.0]))
    assert dpnp.ldexp(dpnp.asarray(np.array([1, 2], "i1")), 2).dtype == np.float16
    assert dpnp.ldexp(dpnp.asarray(np.array([1, 2], "u2")), 2).dtype == np.float32
    r = dpnp.ldexp(2.0, dpnp.asarray(np.array([1, -1], "i8")))
    assert_same(r.asnumpy(), np.array([4.0, 1.0]))
    # exponents beyond the int range: +inf for positive ones, 0 otherwise (ldexp.hpp:45-57)
    big = dpnp.asarray(np.array([2**40, -(2**40), 2**31, -(2**31) - 1], "i8"))
    r = dpnp.ldexp(dpnp.asarray(np.array([1.5, 1.5, -1.5, -1.5])), big)
    assert_same(r.asnumpy(), np.array([np.inf, 0.0, np.inf, 0.0]))
    assert_same(dpnp.ldexp(dpnp.asarray(np.array([1.0], "f4")), dpnp.asarray(np.array([2], "i4")), dtype="f8").asnumpy(),
                np.array([4.0]))
    with pytest.raises(ValueError):
        dpnp.ldexp(dpnp.asarray(np.array([1.0])), dpnp.asarray(np.array([1.0])))
    with pytest.raises(ValueError):
        dpnp.ldexp(dpnp.asarray(np.array([1.0])), dpnp.asarray(np.array([1], "u8")))
    with pytest.raises(ValueError):
        dpnp.ldexp(dpnp.asarray(np.array([1j])), 2)
    with pytest.raises(NotImplementedError):
        dpnp.ldexp(x, 1, where=False)


@pytest.mark.parametrize("dt", ["f2", "f4", "f8"])
def test_frexp_every_binade_and_special_values(dt):
    # dpnp/tests/test_mathematical.py (TestFrexp)
    rng = np.random.default_rng(23)
    info = np.finfo(dt)
    a = np.ldexp(rng.uniform(0.5, 1.0, 6000), rng.integers(info.minexp - info.nmant, info.maxexp + 1, 6000)).astype(dt)
    a[::2] *= -1
    a[:8] = [0.0, -0.0, np.inf, -np.inf, np.nan, info.tiny, info.max, info.smallest_subnormal]
    want_m, want_e = np.frexp(a)
    m, e = dpnp.frexp(dpnp.asarray(a))
    assert e.dtype == np.int32 and m.dtype == np.dtype(dt)
    assert_same(m.asnumpy(), want_m)
    assert_same(e.asnumpy(), want_e.astype("i4"))
    np.testing.assert_array_equal(np.signbit(m.asnumpy()), np.signbit(want_m))
    # views, out arguments, in-place mantissa
    a2 = rng.normal(size=(33, 65)).astype(dt)
    d2 = dpnp.asarray(a2)
    wm, we = np.frexp(a2.T[::2])
    m, e = dpnp.frexp(d2.T[::2])
    assert_same(m.asnumpy(), wm)
    assert_same(e.asnumpy(), we.astype("i4"))
    om, oe = dpnp.empty(a2.shape, dtype=dt), dpnp.empty(a2.shape, dtype="i4")
    rm, re_ = dpnp.frexp(d2, out=(om, oe))
    assert rm is om and re_ is oe
    assert_same(om.asnumpy(), np.frexp(a2)[0])
    assert_same(oe.asnumpy(), np.frexp(a2)[1].astype("i4"))
    rm, re_ = dpnp.frexp(d2, d2, None)
    assert_same(d2.asnumpy(), np.frexp(a2)[0])
    assert_same(re_.asnumpy(), np.frexp(a2)[1].astype("i4"))
    with pytest.raises(ValueError):
        dpnp.frexp(d2, out=(dpnp.empty((3,), dtype=dt), None))
    with pytest.raises(ValueError):
        dpnp.frexp(dpnp.asarray(np.array([1j])))
    mi, ei = dpnp.frexp(dpnp.asarray(np.array([8, 3], "i4")))
    assert mi.dtype == np.float64
    assert_same(mi.asnumpy(), np.array([0.5, 0.75]))
    assert_same(ei.asnumpy(), np.array([4, 2], "i4"))


# ---- the short call path of the ufunc wrappers against the general one ---------------------------
@pytest.mark.parametrize("dt", ["?", "i1", "u2", "i4", "i8", "f2", "f4", "f8", "c8", "c16"])
def test_short_call_path_gives_what_the_general_path_gives(dt):
    """Contiguous operands of one dtype (or an array and a Python number) with default keywords
    skip the general path's promotion search and layout logic; order="C" forces the general
    path, whose result for these operands must be the same array."""
    rng = np.random.default_rng(41)
    shape = (33, 65)
    if dt == "?":
        a, b = rng.integers(0, 2, shape).astype(dt), rng.integers(0, 2, shape).astype(dt)
    elif np.dtype(dt).kind in "iu":
        a, b = rng.integers(1, 100, shape).astype(dt), rng.integers(1, 100, shape).astype(dt)
    else:
        a, b = rng.uniform(1, 9, shape).astype(dt), rng.uniform(1, 9, shape).astype(dt)
    da, db = dpnp.array(a), dpnp.array(b)

    def same(short, general, c_contiguous=True):
        assert short.dtype == general.dtype and short.shape == general.shape
        assert short.flags.c_contiguous == c_contiguous
        assert_same(short.asnumpy(), general.asnumpy())

    for name in ("add", "multiply", "divide", "greater", "maximum", "logical_and", "bitwise_and", "power"):
        f = getattr(dpnp, name)
        try:
            general = f(da, db, order="C")
        except (ValueError, TypeError):
            with pytest.raises((ValueError, TypeError)):
                f(da, db)
            continue
        same(f(da, db), general)
        out = dpnp.empty(shape, dtype=general.dtype)
        assert f(da, db, out=out) is out
        assert_same(out.asnumpy(), general.asnumpy())
        for s in (2, 2.5):
            for args in ((da, s), (s, da)):
                try:
                    general = f(*args, order="C")
                except (ValueError, TypeError):
                    continue
                same(f(*args), general)
    for name in ("negative", "exp", "sqrt", "isnan", "abs", "logical_not", "square"):
        f = getattr(dpnp, name)
        try:
            general = f(da, order="C")
        except (ValueError, TypeError):
            with pytest.raises((ValueError, TypeError)):
                f(da)
            continue
        same(f(da), general)
        out = dpnp.empty(shape, dtype=general.dtype)
        assert f(da, out=out) is out
        assert_same(out.asnumpy(), general.asnumpy())
    # operands the short path must leave to the general one
    same(dpnp.add(da.T, db.T), dpnp.add(dpnp.array(a.T.copy()), dpnp.array(b.T.copy())), False)  # F-contiguous
    same(dpnp.add(da, db[0]), dpnp.add(da, dpnp.array(np.broadcast_to(b[0], shape).copy())))  # broadcast
    if dt not in ("?",):
        x = dpnp.array(a)
        dpnp.add(x, db, out=x)  # out is an input
        assert_same(x.asnumpy(), (dpnp.add(da, db, order="C")).asnumpy())
        y = dpnp.array(b)
        dpnp.add(da, y, out=y)
        assert_same(y.asnumpy(), (dpnp.add(da, db, order="C")).asnumpy())
    with pytest.raises(ValueError):
        dpnp.add(da, db, out=dpnp.empty((5, 5), dtype=dt))
    if dt != "?":
        # out overlaps an input without being it: both contiguous, the general path's temporary is needed
        base = np.arange(1, 201).astype(dt)
        x = dpnp.array(base)
        dpnp.add(x[:100], x[:100], out=x[50:150])
        want = base.copy()
        want[50:150] = base[:100] + base[:100]
        assert_same(x.asnumpy(), want)
        x = dpnp.array(base)
        dpnp.negative(x[:100], out=x[1:101])
        want = base.copy()
        want[1:101] = np.negative(base[:100])
        assert_same(x.asnumpy(), want)
