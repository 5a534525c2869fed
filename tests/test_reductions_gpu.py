"""sum / prod / max / min / argmax / argmin against the oracle.  Bar: integer, bool and index
results bit-exact; float32 sums within 1e-5 and float64 sums within 1e-12 of the exact sum
(relative to the sum of magnitudes, since the reference's summation order is unspecified)."""
import json
import os

import numpy as np
import pytest

import dpnp_amd.tensor as dpt
from oracle import oracle as orc
from tests.helpers import ALL, assert_same, dev, dev_view_like, host, random_array

pytestmark = pytest.mark.gpu
GOLD = json.load(open(os.path.join(os.path.dirname(__file__), "golden", "reference_known_answers.json")))
RTOL = {np.dtype("f2"): 2e-3, np.dtype("f4"): 1e-5, np.dtype("f8"): 1e-12, np.dtype("c8"): 1e-5,
        np.dtype("c16"): 1e-12}

# reduced lengths around every kernel-selection threshold (lanes per output, block, split)
LENGTHS = [1, 2, 7, 8, 9, 31, 33, 63, 64, 65, 255, 256, 257, 511, 1023, 1024, 1025, 2047, 4097, 16384, 65537, 300001]


def check_sum(got, a2d_or_1d, axis, dtype=None):
    want = np.sum(a2d_or_1d.astype(np.longdouble if a2d_or_1d.dtype.kind == "f" else a2d_or_1d.dtype), axis=axis)
    if got.dtype.kind in "fc":
        scale = np.sum(np.abs(a2d_or_1d).astype(np.float64), axis=axis)
        err = np.abs(got.astype(np.longdouble if got.dtype.kind == "f" else np.clongdouble) - want)
        assert (err <= RTOL[got.dtype] * np.maximum(scale, 1e-300)).all(), float(np.max(err / np.maximum(scale, 1e-300)))
    else:
        np.testing.assert_array_equal(got, want.astype(got.dtype))


@pytest.mark.parametrize("dt", ALL, ids=str)
def test_sum_ones_default_dtype(dt):
    # dpnp/tests/tensor/test_tensor_sum.py:56-101
    for n in GOLD["sum_ones"]["n"]:
        r = dpt.sum(dpt.ones(n, dtype=dt))
        assert r.dtype == orc.default_accumulation_dtype(dt) and r.shape == ()
        assert host(r) == n
    assert host(dpt.sum(dpt.ones(200, dtype=dt)[:1:-2])) == 99
    assert host(dpt.sum(dpt.flip(dpt.ones(100, dtype=dt)))) == 100


@pytest.mark.parametrize("arg", ALL, ids=str)
def test_sum_arg_out_dtype_matrix(arg):
    # dpnp/tests/tensor/test_tensor_sum.py:89-101: every (input, result) dtype pair works
    for out in ALL[1:]:
        r = dpt.sum(dpt.ones(100, dtype=arg), dtype=out)
        assert r.dtype == out and host(r) == 100


def test_sum_known_answers():
    g = GOLD["sum_gh1391"]
    a = dpt.reshape(dpt.arange(g["arange"], dtype="i4"), g["shape"])
    assert_same(host(dpt.sum(dpt.permute_dims(a, g["permute"]), axis=g["axis"])), np.array(g["expected"], dtype="i8"))
    g = GOLD["sum_axis0_3x4x5"]
    x = dpt.reshape(dpt.arange(g["arange"], dtype="f4"), g["shape"])
    assert_same(host(dpt.sum(x, axis=0)), np.array(g["expected"], dtype="f4"))
    g = GOLD["sum_flip_axis2_3x4x5"]
    assert_same(host(dpt.sum(dpt.flip(x, axis=2), axis=2)), np.array(g["expected"], dtype="f4"))
    g = GOLD["sum_bool_dtype_gh1944"]
    for dt in g["dtypes"]:
        assert bool(dpt.sum(dev(np.array(g["input"], dtype=dt)), dtype="?")) is True
    e = dpt.sum(dpt.empty((0,), dtype="u1"))
    assert e.shape == () and int(e) == 0
    assert int(dpt.prod(dpt.empty((0,), dtype="i4"))) == 1
    assert dpt.sum(dpt.empty((3, 0), dtype="f4"), axis=1).shape == (3,)
    assert (host(dpt.sum(dpt.empty((3, 0), dtype="f4"), axis=1)) == 0).all()
    assert dpt.sum(dpt.empty((0, 3), dtype="f4"), axis=1).shape == (0,)


@pytest.mark.parametrize("n", [1023, 1024, 1025])
def test_largish_reductions(n):
    # dpnp/tests/tensor/test_tensor_sum.py:184-212
    for dt in ("i8", "f4", "c8"):
        x = dpt.ones((5, n, 5), dtype=dt)
        assert (host(dpt.sum(x, axis=(0, 1))) == 5 * n).all() and (host(dpt.sum(x, axis=(1, 2))) == 5 * n).all()
    assert (host(dpt.sum(dpt.ones((25, n), dtype="f4"), axis=1)) == n).all()
    assert (host(dpt.sum(dpt.ones((n, 25), dtype="f4"), axis=0)) == n).all()


@pytest.mark.parametrize("dt", ["f4", "f8", "i4", "u1", "?", "f2", "c8"])
def test_rows_and_cols_all_lengths(dt):
    rng = np.random.default_rng(41)
    for n in LENGTHS:
        m = max(1, min(37, 600000 // n))
        a = random_array(rng, (m, n), dt, -3, 3)
        da = dev(a)
        check_sum(host(dpt.sum(da, axis=1)), a, 1)
        check_sum(host(dpt.sum(da.T, axis=0)), a.T, 0)
        at = np.ascontiguousarray(a.T)  # (n, m): reduce the outer axis of a C-contiguous matrix
        check_sum(host(dpt.sum(dev(at), axis=0)), at, 0)
        if dt != "c8":
            assert_same(host(dpt.max(da, axis=1)), orc.reduce("max", a, 1))
            assert_same(host(dpt.min(dev(at), axis=0)), orc.reduce("min", a, 1))
            assert_same(host(dpt.argmax(da, axis=1)), orc.argreduce("argmax", a, 1))
            assert_same(host(dpt.argmin(dev(at), axis=0)), orc.argreduce("argmin", a, 1))


@pytest.mark.parametrize("dt", ["f4", "i8", "f8"])
def test_full_reduction_sizes(dt):
    rng = np.random.default_rng(43)
    for n in (1, 100, 4096, 65536, 1 << 20, (1 << 22) + 3, 10_000_019):
        a = random_array(rng, n, dt, -1, 1) if dt != "i8" else random_array(rng, n, dt, -1000, 1000)
        da = dev(a)
        check_sum(host(dpt.sum(da)), a, None)
        assert host(dpt.max(da)) == a.max() and host(dpt.min(da)) == a.min()
        assert int(dpt.argmax(da)) == int(np.argmax(a)) and int(dpt.argmin(da)) == int(np.argmin(a))
        if n > 8:  # unaligned start
            check_sum(host(dpt.sum(da[3:])), a[3:], None)
            assert int(dpt.argmax(da[1:])) == int(np.argmax(a[1:]))


def test_prod():
    rng = np.random.default_rng(47)
    a = rng.uniform(0.9, 1.1, (7, 501)).astype("f4")
    np.testing.assert_allclose(host(dpt.prod(dev(a), axis=1)), np.prod(a.astype("f8"), axis=1), rtol=1e-4)
    i = rng.integers(-3, 4, (5, 40)).astype("i4")
    assert_same(host(dpt.prod(dev(i), axis=1)), np.prod(i, axis=1, dtype="i8"))
    u = rng.integers(1, 255, 100).astype("u1")
    assert_same(host(dpt.prod(dev(u))), np.prod(u, dtype="u8"))  # wraps modulo 2**64
    assert bool(dpt.prod(dev(np.array([True, True])), dtype="?")) and not bool(
        dpt.prod(dev(np.array([True, False])), dtype="?"))


def test_max_min_nan_propagation():
    # dpnp/tests/tensor/test_usm_ndarray_reductions.py:150-173
    for c in GOLD["max_min_nan"]["cases"]:
        x = dev(np.array([float(v) for v in c["values"]], dtype=c["dtype"]))
        assert np.isnan(host(dpt.max(x))) and np.isnan(host(dpt.min(x)))
    z = np.arange(4, dtype="c8")
    for bad in (complex(np.nan, 0), complex(0, np.nan)):
        z[0] = bad
        assert np.isnan(host(dpt.max(dev(z)))) and np.isnan(host(dpt.min(dev(z))))
    rng = np.random.default_rng(53)
    for n in (100, 5000, 1 << 20):
        a = rng.standard_normal((3, n)).astype("f4")
        a[1, rng.integers(0, n)] = np.nan
        r = host(dpt.max(dev(a), axis=1))
        assert np.isnan(r[1]) and r[0] == a[0].max() and r[2] == a[2].max()
        r = host(dpt.min(dev(np.ascontiguousarray(a.T)), axis=0))
        assert np.isnan(r[1]) and r[0] == a[0].min()
    g = GOLD["max_axis0_arange"]
    x = dpt.reshape(dpt.arange(g["arange"]), g["shape"])
    assert_same(host(dpt.max(x, axis=0)), host(x)[-1])
    xf = dpt.flip(x, axis=2)
    assert_same(host(dpt.max(xf, axis=2)), host(xf)[:, :, 0])
    with pytest.raises(ValueError):
        dpt.max(dpt.empty((3, 0)), axis=1)
    with pytest.raises(ValueError):
        dpt.argmax(dpt.empty((0,)))


def test_argmax_known_answers_and_ties():
    g = GOLD["argmax_2x3"]
    for order in ("C", "F"):
        x = dpt.asarray(np.array(g["input"], dtype=g["dtype"]), order=order)
        assert int(dpt.argmax(x)) == g["argmax_flat"]
        assert_same(host(dpt.argmax(x, axis=0)), np.array(g["argmax_axis0"], dtype="i8"))
        assert_same(host(dpt.argmax(x, axis=1)), np.array(g["argmax_axis1"], dtype="i8"))
    assert int(dpt.argmax(dpt.full(3, np.iinfo("i4").min, dtype="i4"))) == 0
    assert int(dpt.argmin(dpt.full(3, np.iinfo("i4").max, dtype="i4"))) == 0
    assert int(dpt.argmax(dpt.full(5000, -np.inf, dtype="f4"))) == 0
    for idx in range(4):
        for dt in ("f4", "c8"):
            x = np.arange(4, dtype=dt)
            x[idx] = np.nan
            assert int(dpt.argmax(dev(x))) == idx and int(dpt.argmin(dev(x))) == idx
    rng = np.random.default_rng(59)
    # planted extremum and duplicated extrema at random places, incl. views
    # (dpnp/tests/tensor/test_usm_ndarray_reductions.py:186-251)
    for n in (1025, 24 * 1024, 1 << 21):
        a = rng.standard_normal(n).astype("f4")
        dup = rng.choice(n, max(n // 100, 2), replace=False)
        a[dup] = a.max() + 1
        for v in (a, a[::-1], a[::2], a[::-2]):
            d = dev_view_like(v, a)
            assert int(dpt.argmax(d)) == int(np.argmax(v))
        a[dup] = a.min() - 1
        assert int(dpt.argmin(dev(a))) == int(np.argmin(a))
        a[rng.choice(n, max(n // 1000, 2), replace=False)] = np.nan  # several NaNs: the first one
        assert int(dpt.argmax(dev(a))) == int(np.argmax(a)) == int(dpt.argmin(dev(a)))
    m = rng.standard_normal((24, 1025)).astype("f4")
    m[:, 7] = 50
    m[:, 900] = 50
    assert (host(dpt.argmax(dev(m), axis=1)) == 7).all()
    assert_same(host(dpt.argmax(dev(m)[:, ::-2], axis=1)), np.argmax(m[:, ::-2], axis=1))
    assert_same(host(dpt.argmax(dev(m), axis=0)), np.argmax(m, axis=0))


def test_multi_axis_keepdims_out():
    rng = np.random.default_rng(61)
    a = random_array(rng, (6, 7, 8, 9), "f4", -2, 2)
    da = dev(a)
    for axis in (0, 1, -1, (0, 2), (1, 3), (0, 1, 2, 3), (3, 0), None):
        for keep in (False, True):
            r = dpt.sum(da, axis=axis, keepdims=keep)
            want = np.sum(a.astype("f8"), axis=axis, keepdims=keep)
            assert r.shape == want.shape
            np.testing.assert_allclose(host(r), want, rtol=1e-5, atol=1e-5)
            assert_same(host(dpt.max(da, axis=axis, keepdims=keep)), np.max(a, axis=axis, keepdims=keep))
    for axis in (0, 2, -1, None):
        assert_same(host(dpt.argmin(da, axis=axis, keepdims=True)), np.argmin(a, axis=axis, keepdims=True))
    # permuted and sliced inputs reach the generic kernel
    v = dpt.permute_dims(da, (2, 0, 3, 1))[::2, :, ::-1]
    hv = np.transpose(a, (2, 0, 3, 1))[::2, :, ::-1]
    np.testing.assert_allclose(host(dpt.sum(v, axis=(1, 2))), hv.astype("f8").sum(axis=(1, 2)), rtol=1e-5, atol=1e-5)
    assert_same(host(dpt.argmax(v, axis=1)), np.argmax(hv, axis=1))
    assert_same(host(dpt.argmax(v)), np.array(np.argmax(hv)))
    # out= into a strided slice of a zero array: neighbours stay zero
    # (dpnp/tests/tensor/test_usm_ndarray_reductions.py:518-628)
    big = dpt.zeros((7, 2), dtype="f4")
    r = dpt.sum(da, axis=(0, 2, 3), out=big[:, 1])
    hb = host(big)
    assert (hb[:, 0] == 0).all()
    np.testing.assert_allclose(hb[:, 1], a.astype("f8").sum(axis=(0, 2, 3)), rtol=1e-5)
    o = dpt.empty((6, 1, 8, 1), dtype="f4")
    r = dpt.max(da, axis=(1, 3), keepdims=True, out=o)  # a view of o's memory, as in the reference
    assert r.shape == o.shape and r._pointer == o._pointer
    assert_same(host(o), a.max(axis=(1, 3), keepdims=True))
    with pytest.raises(ValueError):
        dpt.sum(da, axis=0, out=dpt.empty((7, 8, 9), dtype="f8"))
    with pytest.raises(ValueError):
        dpt.sum(da, axis=0, out=dpt.empty((7, 8), dtype="f4"))
    # out overlapping the input goes through a temporary
    x = dev(np.arange(12, dtype="f4").reshape(3, 4))
    dpt.sum(x, axis=1, out=x[:, 0])
    assert_same(host(x)[:, 0], np.array([6, 22, 38], dtype="f4"))


def test_reduction_keepdims_reference_case():
    # dpnp/tests/tensor/test_usm_ndarray_reductions.py:94-106
    x = dpt.ones((3, 4, 5, 6, 7), dtype="i4")
    m = dpt.max(x, axis=(1, 2, -1), keepdims=True)
    xx = dpt.reshape(dpt.permute_dims(x, (0, 3, 1, 2, -1)), (3, 6, -1))
    p = dpt.argmax(xx, axis=-1, keepdims=True)
    assert m.shape == (3, 1, 1, 6, 1) and (host(m) == 1).all() and (host(p) == 0).all()


def test_results_are_reproducible_bit_for_bit():
    rng = np.random.default_rng(67)
    a = dev(rng.standard_normal(1 << 22).astype("f4"))
    m = dev(rng.standard_normal((2048, 2048)).astype("f4"))
    first = [host(dpt.sum(a)), host(dpt.sum(m, axis=0)), host(dpt.sum(m, axis=1))]
    for _ in range(3):
        again = [host(dpt.sum(a)), host(dpt.sum(m, axis=0)), host(dpt.sum(m, axis=1))]
        for x, y in zip(first, again):
            assert x.tobytes() == y.tobytes()


def test_all_any():
    a = np.array([[0, 1, 2], [0, 0, 0], [3, 4, 5]], dtype="f4")
    assert_same(host(dpt.any(dev(a), axis=1)), a.any(axis=1))
    assert_same(host(dpt.all(dev(a), axis=1)), a.all(axis=1))
    assert bool(dpt.all(dpt.empty((0,)))) and not bool(dpt.any(dpt.empty((0,))))


def test_logsumexp_hypot_count_nonzero():
    # dpnp/tests/tensor/test_usm_ndarray_reductions.py (logsumexp / reduce_hypot sections)
    rng = np.random.default_rng(103)
    for dt, rtol in (("f4", 1e-5), ("f8", 1e-12)):
        a = (rng.standard_normal((7, 3001)) * 20).astype(dt)
        want = np.log(np.sum(np.exp(a.astype(np.longdouble)), axis=1))
        np.testing.assert_allclose(host(dpt.logsumexp(dev(a), axis=1)).astype(np.longdouble), want, rtol=rtol)
        big = np.full(1000, 1000.0, dtype=dt)  # exp overflows, the pairwise combine does not
        np.testing.assert_allclose(float(dpt.logsumexp(dev(big))), 1000.0 + np.log(1000.0), rtol=rtol)
        want = np.sqrt(np.sum(a.astype(np.longdouble) ** 2, axis=0))
        np.testing.assert_allclose(host(dpt.reduce_hypot(dev(a), axis=0)).astype(np.longdouble), want, rtol=rtol)
        huge = np.full(100, np.finfo(dt).max / 100, dtype=dt)  # the squares overflow, the result does not
        assert np.isfinite(float(dpt.reduce_hypot(dev(huge))))
    assert float(dpt.logsumexp(dpt.empty((0,), dtype="f4"))) == -np.inf
    assert float(dpt.reduce_hypot(dpt.empty((0,), dtype="f4"))) == 0.0
    assert dpt.logsumexp(dpt.ones(5, dtype="i4")).dtype == np.dtype("f8")
    np.testing.assert_allclose(float(dpt.logsumexp(dpt.ones(5, dtype="i4"))), 1 + np.log(5), rtol=1e-14)
    m = rng.integers(-1, 2, (40, 50)).astype("i1")
    assert_same(host(dpt.count_nonzero(dev(m), axis=0)), np.count_nonzero(m, axis=0).astype("i8"))
    assert int(dpt.count_nonzero(dev(m))) == int(np.count_nonzero(m))
