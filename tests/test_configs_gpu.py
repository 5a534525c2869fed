"""The five benchmark configurations at their full sizes: results checked through
size-independent properties and through the oracle on samples / reduced problems."""
import math

import numpy as np
import pytest

import dpnp_amd as dpnp
import dpnp_amd.tensor as dpt
from oracle import oracle as orc
from tests.helpers import assert_same, assert_ulp, dev, host

pytestmark = pytest.mark.gpu


def test_config1_add_then_sum_2p24():
    rng = np.random.default_rng(0)
    a = rng.uniform(-1, 1, 2**24).astype("f4")
    b = rng.uniform(-1, 1, 2**24).astype("f4")
    c = dpt.add(dev(a), dev(b))
    hc = host(c)
    assert_same(hc, a + b)  # IEEE add: bit-exact
    s = float(dpt.sum(c))
    exact = float(np.sum(hc, dtype="f8"))
    assert abs(s - exact) <= 1e-5 * max(abs(exact), 1e-3 * float(np.sum(np.abs(hc), dtype="f8")))


def test_config2_axis_sum_max_16384():
    rng = np.random.default_rng(1)
    a = rng.uniform(-1, 1, (16384, 16384)).astype("f4")
    d = dev(a)
    absum1 = np.abs(a).sum(axis=1, dtype="f8")
    absum0 = np.abs(a).sum(axis=0, dtype="f8")
    s1, s0 = host(dpt.sum(d, axis=1)), host(dpt.sum(d, axis=0))
    assert np.all(np.abs(s1 - a.sum(axis=1, dtype="f8")) <= 1e-5 * absum1)
    assert np.all(np.abs(s0 - a.sum(axis=0, dtype="f8")) <= 1e-5 * absum0)
    # relative to the value itself where the sum is not a heavy cancellation
    # (condition number sum|x| / |sum x| below 1e3)
    ex1 = a.sum(axis=1, dtype="f8")
    big = np.abs(ex1) * 1e3 > absum1
    assert big.any() and np.all(np.abs(s1[big] - ex1[big]) <= 1e-5 * np.abs(ex1[big]))
    assert_same(host(dpt.max(d, axis=1)), a.max(axis=1))
    assert_same(host(dpt.max(d, axis=0)), a.max(axis=0))
    # a checksum of checksums: both orders of reduction agree on the grand total
    t1, t0 = float(np.sum(s1, dtype="f8")), float(np.sum(s0, dtype="f8"))
    assert abs(t1 - t0) <= 1e-5 * float(absum1.sum())


def test_config3_argmax_mean_var_2p28():
    n = 2**28
    rng = np.random.default_rng(2)
    x = rng.standard_normal(n, dtype="f4")
    x[rng.choice(n, n // 100, replace=False)] = x.max()
    lo = x.min()
    x[rng.choice(n, n // 100, replace=False)] = lo
    d = dev(x)
    assert int(dpt.argmax(d)) == int(np.argmax(x))  # first of ~2.7M equal maxima
    assert int(dpt.argmin(d)) == int(np.argmin(x))
    # float32 data, statistics accumulated in float64 (1e-12 of the float64 answer)
    m = float(dpnp.mean(dpnp.ndarray._create_from_usm_ndarray(d), dtype="f8"))
    v = float(dpnp.var(dpnp.ndarray._create_from_usm_ndarray(d), dtype="f8"))
    x64 = x.astype("f8")
    want_m = float(np.mean(x64))
    want_v = float(np.mean((x64 - want_m) ** 2))
    assert abs(m - want_m) <= 1e-12 * max(abs(want_m), float(np.mean(np.abs(x64))))
    assert abs(v - want_v) <= 1e-12 * want_v
    # float64 input at the full 2^28 elements (the host check streams in chunks): 1e-12
    d64 = dev(x64)
    step = 1 << 24
    want_m2 = math.fsum(float(np.sum(x64[i:i + step], dtype=np.longdouble)) for i in range(0, n, step)) / n
    want_v2 = math.fsum(float(np.sum((x64[i:i + step] - want_m2) ** 2, dtype=np.longdouble))
                        for i in range(0, n, step)) / n
    mean_abs = math.fsum(float(np.sum(np.abs(x64[i:i + step]))) for i in range(0, n, step)) / n
    assert d64.shape == (n,) and d64.dtype == np.dtype("f8")
    assert abs(float(dpt.mean(d64)) - want_m2) <= 1e-12 * mean_abs
    assert abs(float(dpt.var(d64)) - want_v2) <= 1e-12 * want_v2
    del d64, x64
    # NaN variant: about 0.1 % NaNs -> index of the first NaN, NaN statistics
    x[rng.choice(n, n // 1000, replace=False)] = np.nan
    d = dev(x)
    first_nan = int(np.argmax(np.isnan(x)))
    assert int(dpt.argmax(d)) == first_nan == int(dpt.argmin(d))
    assert np.isnan(float(dpt.mean(d))) and np.isnan(float(dpt.var(d)))
    assert np.isnan(float(dpt.max(d)))


def test_config4_strided_broadcast_8192():
    rng = np.random.default_rng(3)
    A = rng.standard_normal((8192, 8192)).astype("f4")
    B = rng.standard_normal((1, 4096)).astype("f4")
    dA, dB = dev(A), dev(B)
    V1, V2 = dA[:, ::2], dA.T
    assert V1.strides == (8192, 2) and V2.strides == (1, 8192)
    assert_same(host(dpt.multiply(V1, dB)), A[:, ::2] * B)
    e1 = dpt.exp(V1)
    assert_ulp(host(e1)[::64], np.exp(A[::64, ::2].astype("f8")), 4.0)
    e2 = dpt.exp(V2)  # order K keeps the F layout
    assert e2.flags.f_contiguous
    assert_ulp(host(e2)[::64], np.exp(A.T[::64].astype("f8")), 4.0)
    e3 = dpt.exp(V2, order="C")  # transposing
    assert e3.flags.c_contiguous
    assert_same(host(e3), host(e2))
    w = dpt.where(dpt.greater(V1, 0), V1, dB)
    assert_same(host(w), np.where(A[:, ::2] > 0, A[:, ::2], B))
    w2 = dpnp.where_compare("greater", dpnp.ndarray._create_from_usm_ndarray(V1), 0,
                            dpnp.ndarray._create_from_usm_ndarray(V1),
                            dpnp.ndarray._create_from_usm_ndarray(dB))
    assert_same(w2.asnumpy(), host(w))
    I = rng.integers(-2**31, 2**31, (8192, 8192), dtype=np.int64).astype("i4")
    J = rng.integers(-2**31, 2**31, (8192, 8192), dtype=np.int64).astype("i4")
    dI, dJ = dev(I), dev(J)
    assert_same(host(dpt.bitwise_and(dI, dJ)), I & J)
    assert_same(host(dpt.bitwise_and(dI[:, ::2], dJ[:, ::2])), I[:, ::2] & J[:, ::2])


def test_config5_black_scholes_2p26():
    n = 2**26
    rng = np.random.default_rng(4)
    p, s, t = rng.uniform(10, 50, n), rng.uniform(10, 50, n), rng.uniform(1, 2, n)
    call, put = dpnp.black_scholes(dpnp.array(p), dpnp.array(s), dpnp.array(t), 0.1, 0.2)
    hc, hp = call.asnumpy(), put.asnumpy()
    # put-call parity holds for every option
    np.testing.assert_allclose(hc - hp, p - s * np.exp(-0.1 * t), rtol=1e-11, atol=1e-11)
    sl = slice(0, n, 1031)
    wc, wp = orc.black_scholes(p[sl], s[sl], t[sl], 0.1, 0.2)
    np.testing.assert_allclose(hc[sl], wc, rtol=1e-12, atol=1e-12)
    np.testing.assert_allclose(hp[sl], wp, rtol=1e-12, atol=1e-12)
