"""sum / prod / max / min / argmax / argmin against the oracle.  Bar: integer, bool and index
results bit-exact; float32 sums within 1e-5 and float64 sums within 1e-12 of the exact sum
(relative to the sum of magnitudes, since the reference's summation order is unspecified)."""
import json
import os
import warnings

import numpy as np
import pytest

import dpnp_amd as dpnp
import dpnp_amd.tensor as dpt
from dpnp_amd.tensor import _nan_reductions as nr
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


@pytest.mark.parametrize("src", sorted(GOLD["sum_prod_type_pairs"]["pairs"]))
def test_sum_prod_every_reference_pair_in_one_pass(src):
    # sum.cpp:87-241, prod.cpp: each (input, result) pair of the reference's tables has a direct kernel;
    # values chosen so that narrow results wrap: the element is converted to the result type, then added
    import dpnp_amd._lib as L

    rng = np.random.default_rng(59)
    for dst in GOLD["sum_prod_type_pairs"]["pairs"][src]:
        names = [d.str[1:] if d.kind != "b" else "?" for d in ALL]
        for op in ("sum", "prod"):
            assert L.lib.dpx_reduce_dtype_supported(L.REDUCE_ID[op], names.index(src), names.index(dst)) == 1
        for shape, axis in (((5, 3001), 1), ((3001, 40), 0), ((1 << 20,), None)):
            a = random_array(rng, shape, src, -100, 100)
            got = host(dpt.sum(dev(a), axis=axis, dtype=dst))
            want = orc.reduce("sum", a if axis != 0 else a.T, 1, out_dtype=dst)
            if np.dtype(dst).kind in "fc":
                scale = np.abs(a.astype("f8")).sum(axis=axis)
                assert (np.abs(got - want) <= RTOL[np.dtype(dst)] * np.maximum(scale, 1)).all(), (src, dst, shape)
            else:
                assert_same(got, want)
            small = random_array(rng, (7, 9), src, -3, 3)  # products that neither overflow floats nor vanish
            gp = host(dpt.prod(dev(small), axis=1, dtype=dst))
            wp = orc.reduce("prod", small, 1, out_dtype=dst)
            if np.dtype(dst).kind in "fc":
                np.testing.assert_allclose(gp, wp, rtol=1e-3 if dst == "f2" else 1e-5)
            else:
                assert_same(gp, wp)


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


# ---- NaN-ignoring reductions (one-pass kernels behind dpnp.nansum, nanmax, ...) ---------------
def _with_nans(rng, shape, dt, frac=0.2):
    a = random_array(rng, shape, dt, -10, 10)
    a[rng.random(shape) < frac] = np.nan
    return a


@pytest.mark.parametrize("dt", ["f2", "f4", "f8"])
@pytest.mark.parametrize("axis", [None, 0, 1, -1, (0, 2)])
def test_nan_reductions_against_oracle(dt, axis):
    rng = np.random.default_rng(211)
    a = _with_nans(rng, (7, 33, 20), dt)
    a[3, :, 5] = np.nan       # all-NaN runs along axis 1
    d = dpnp.array(a)
    for name in ("nansum", "nanprod", "nanmax", "nanmin"):
        with warnings.catch_warnings():
            warnings.simplefilter("ignore", RuntimeWarning)
            got = getattr(dpnp, name)(d, axis=axis).asnumpy()
            want_np = getattr(np, name)(a.astype("f8") if name == "nanprod" else a, axis=axis)
        ax = tuple(range(a.ndim)) if axis is None else (axis if isinstance(axis, tuple) else (axis % a.ndim,))
        moved = np.moveaxis(a, ax, tuple(range(a.ndim - len(ax), a.ndim)))
        want, _ = orc.nan_reduce(name, moved, len(ax))
        assert got.dtype == a.dtype and got.shape == np.shape(want_np)
        if name in ("nanmax", "nanmin"):
            assert_same(got, want)
            assert_same(got, np.asarray(want_np, dtype=dt))
        else:
            scale = (np.nansum(np.abs(moved.astype("f8")), axis=tuple(range(moved.ndim - len(ax), moved.ndim)))
                     if name == "nansum" else np.abs(np.asarray(want, dtype="f8")))
            tol = {"f2": 2e-3, "f4": 1e-5, "f8": 1e-12}[dt]
            ok = np.abs(got.astype("f8") - np.asarray(want, dtype="f8")) <= tol * np.maximum(scale, 1e-30)
            both_inf = np.isinf(got) & (got == np.asarray(want, dtype=dt))
            assert np.all(ok | both_inf), name


def test_nan_extrema_all_nan_warns_and_arg_raises():
    a = np.arange(12, dtype="f4").reshape(2, 2, 3)
    a[:, :, 2] = np.nan
    d = dpnp.array(a)
    with pytest.warns(RuntimeWarning, match="All-NaN slice"):
        r = dpnp.nanmax(d, axis=0)
    assert_same(r.asnumpy(), np.array([[0 + 6, 7, np.nan], [9, 10, np.nan]], dtype="f4"))
    with pytest.raises(ValueError, match="All-NaN slice"):
        dpnp.nanargmax(d, axis=0)
    with pytest.raises(ValueError, match="All-NaN slice"):
        dpnp.nanargmin(d, axis=0)
    with warnings.catch_warnings():
        warnings.simplefilter("error")
        assert_same(dpnp.nanmin(d, axis=2).asnumpy(), np.nanmin(a, axis=2))  # no all-NaN run: no warning


@pytest.mark.parametrize("func", ["nanargmin", "nanargmax"])
@pytest.mark.parametrize("axis", [None, 0, 1, -1, 2, -2])
@pytest.mark.parametrize("keepdims", [False, True])
@pytest.mark.parametrize("dt", ["f4", "f8", "c8"])
def test_nanarg_reference_basic(func, axis, keepdims, dt):
    # dpnp/tests/test_nanfunctions.py:33-43
    a = np.arange(768, dtype=dt).reshape((4, 4, 6, 8))
    a[2:3, 2, 3:4, 4] = np.nan
    got = getattr(dpnp, func)(dpnp.array(a), axis=axis, keepdims=keepdims).asnumpy()
    assert_same(got, np.asarray(getattr(np, func)(a, axis=axis, keepdims=keepdims), dtype="i8"))


def test_nanarg_ties_infinities_and_large():
    rng = np.random.default_rng(223)
    # -inf present together with NaN: NaN reads as -inf, the first of either wins
    a = np.array([np.nan, -np.inf, 3.0, 3.0, np.nan], dtype="f4")
    assert int(dpnp.nanargmax(dpnp.array(a))) == 2
    assert int(dpnp.nanargmin(dpnp.array(a))) == 1
    b = np.array([np.nan, -np.inf, -np.inf], dtype="f8")
    assert int(dpnp.nanargmax(dpnp.array(b))) == int(orc.nan_argreduce("nanargmax", b, 1)) == 0
    # long 1-D input: split over blocks
    n = 3_000_003
    x = rng.standard_normal(n).astype("f4")
    x[rng.choice(n, n // 50, replace=False)] = np.nan
    x[rng.choice(n, 100, replace=False)] = np.nanmax(x)
    d = dpnp.array(x)
    assert int(dpnp.nanargmax(d)) == int(np.nanargmax(x))
    assert int(dpnp.nanargmin(d)) == int(np.nanargmin(x))
    assert float(dpnp.nanmax(d)) == float(np.nanmax(x))
    s, want = float(dpnp.nansum(d)), float(np.nansum(x.astype("f8")))
    assert abs(s - want) <= 1e-5 * float(np.nansum(np.abs(x.astype("f8"))))
    m = x.reshape(3, -1)[:, :1_000_000].T.copy()      # (1000000, 3): column reductions over a long axis
    dm = dpnp.array(m)
    assert_same(dpnp.nanargmax(dm, axis=0).asnumpy(), np.nanargmax(m, axis=0))
    assert_same(dpnp.nanmin(dm, axis=0).asnumpy(), np.nanmin(m, axis=0))


_NANARG_SHAPES = [((5000,), None), ((3_000_003,), None), ((300, 700), 1), ((300, 700), 0), ((40_000, 24), 0),
                  ((40_000, 12), 1)]


@pytest.mark.parametrize("dt, shape, axis", [(dt, sh, ax) for dt in ("f2", "f4", "f8") for sh, ax in _NANARG_SHAPES] +
                         [("f4", (70_000, 1500), 0)])  # one dtype is enough for the large matrix
def test_nanarg_runs_whose_extreme_is_the_infinity_nan_counts_as(dt, shape, axis):
    """nanargmax reads NaN as -inf (dpnp/dpnp_iface_nanfunctions.py:195-200): a run with a NaN before a real -inf
    gives the position of the NaN, an all-NaN run raises, and the search kernel alone tells which runs need a
    second look."""
    rng = np.random.default_rng(5)
    a = rng.standard_normal(shape).astype(dt)
    a[rng.random(shape) < 0.05] = np.nan
    runs = a.reshape(1, -1) if axis is None else (a if axis == 1 else a.T)  # views: one run per row
    assert np.shares_memory(runs, a)
    # some runs hold nothing but NaN and -inf, with the NaNs first
    for r in range(0, runs.shape[0], max(1, runs.shape[0] // 7)):
        runs[r] = -np.inf
        runs[r, : max(1, runs.shape[1] // 3)] = np.nan
    assert_same(dpnp.nanargmax(dpnp.array(a), axis=axis).asnumpy(), np.asarray(np.nanargmax(a, axis=axis), dtype="i8"))
    assert_same(dpnp.nanargmin(dpnp.array(-a), axis=axis).asnumpy(), np.asarray(np.nanargmin(-a, axis=axis), dtype="i8"))
    # an all-NaN run raises and leaves `out` as it was
    runs[runs.shape[0] // 2] = np.nan
    d = dpnp.array(a)
    out = dpnp.full(() if axis is None else (runs.shape[0],), -7, dtype="i8")
    with pytest.raises(ValueError, match="All-NaN slice"):
        dpnp.nanargmax(d, axis=axis, out=out)
    with pytest.raises(ValueError, match="All-NaN slice"):
        dpnp.nanargmin(d, axis=axis, out=out)
    assert (out.asnumpy() == -7).all()


@pytest.mark.parametrize("dt, res", [("f2", None), ("f4", None), ("f8", None), ("c8", None), ("c16", None), ("f2", "f4"),
                                     ("f4", "f8"), ("c8", "c16")])
@pytest.mark.parametrize("shape, axis", [((4099,), None), ((2_000_003,), None), ((300, 700), 1), ((300, 700), 0),
                                         ((40_000, 24), 0), ((40_000, 12), 1), ((60_000, 40), 0), ((9, 50, 11), (0, 2))])
def test_nanmean_one_pass_over_every_kernel_family(dt, res, shape, axis):
    """Sum and count of the numbers travel together through the reduction kernels; the quotient equals the one of
    the reference's composition nansum / count (dpnp/dpnp_iface_nanfunctions.py:600-636) to rounding."""
    rng = np.random.default_rng(31)
    a = rng.uniform(0.5, 1.5, shape).astype(dt)
    if a.dtype.kind == "c":
        a = a + 1j * rng.uniform(0.5, 1.5, shape).astype(a.real.dtype)
        a.imag[rng.random(shape) < 0.1] = np.nan
    a[rng.random(shape) < 0.2] = np.nan
    # a run without any number
    if axis == 1:
        a[0, :] = np.nan
    elif axis == 0:
        a[:, 0] = np.nan
    elif axis == (0, 2):
        a[:, 0, :] = np.nan
    out_dt = np.dtype(res or dt)
    got = nr.nanmean(dev(a), axis=axis, dtype=res)
    assert got.dtype == out_dt
    wide = a.astype("c16" if a.dtype.kind == "c" else "f8")
    good = ~np.isnan(wide)
    with np.errstate(all="ignore"):
        want = (np.where(good, wide, 0).sum(axis=axis) / good.sum(axis=axis)).astype(out_dt)
    eps = float(np.finfo(out_dt).eps)
    rtol = 2e-3 if eps > 1e-4 else (2e-5 if eps > 1e-10 else 1e-12)
    np.testing.assert_allclose(host(got), want, rtol=rtol, equal_nan=True)
    if axis is not None:
        assert np.isnan(host(got)).any()


@pytest.mark.parametrize("dt, res", [("f2", None), ("f4", None), ("f8", None), ("f2", "f4"), ("f4", "f8")])
@pytest.mark.parametrize("shape, axis", [((4099,), None), ((2_000_003,), None), ((300, 700), 1), ((300, 700), 0),
                                         ((40_000, 24), 0), ((40_000, 12), 1), ((60_000, 40), 0), ((9, 50, 11), (0, 2))])
@pytest.mark.parametrize("ddof", [0, 1, 2.5])
def test_nanvar_second_pass_over_every_kernel_family(dt, res, shape, axis, ddof):
    """Squared deviations and count of the numbers travel together through the reduction kernels and are divided by
    count - ddof at the end; slices with count <= ddof give NaN (dpnp/dpnp_iface_nanfunctions.py:1318-1390)."""
    rng = np.random.default_rng(37)
    a = rng.uniform(0.5, 1.5, shape).astype(dt)
    a[rng.random(shape) < 0.2] = np.nan
    if axis == 1:
        a[0, :] = np.nan          # no number at all
        a[1, 2:] = np.nan         # two numbers: NaN for ddof 2.5
    elif axis == 0:
        a[:, 0] = np.nan
        a[2:, 1] = np.nan
    elif axis == (0, 2):
        a[:, 0, :] = np.nan
        a[:, 1, :] = np.nan
        a[0, 1, :2] = 1.0
    out_dt = np.dtype(res or dt)
    got = dpnp.nanvar(dpnp.array(a), axis=axis, dtype=res, ddof=ddof)
    assert got.dtype == out_dt
    with warnings.catch_warnings():
        warnings.simplefilter("ignore", RuntimeWarning)
        want = np.nanvar(a.astype("f8"), axis=axis, ddof=ddof)
    want = np.where(np.isfinite(want) & (want >= 0), want, np.nan)  # NumPy divides by a negative count - ddof
    eps = float(np.finfo(out_dt).eps)
    rtol = 4e-3 if eps > 1e-4 else (4e-5 if eps > 1e-10 else 1e-11)
    np.testing.assert_allclose(got.asnumpy().astype("f8"), want, rtol=rtol, atol=rtol * 1e-2, equal_nan=True)
    if axis is not None:
        assert np.isnan(got.asnumpy()).any()
    # a mean handed in by the caller is taken as it is
    mu = dpnp.nanmean(dpnp.array(a), axis=axis, dtype=res, keepdims=True)
    again = dpnp.nanvar(dpnp.array(a), axis=axis, dtype=res, ddof=ddof, mean=mu)
    np.testing.assert_array_equal(again.asnumpy(), got.asnumpy())


@pytest.mark.parametrize("dt", ["f4", "f8"])
@pytest.mark.parametrize("axis", [None, 0, 1, (0, 1)])
@pytest.mark.parametrize("keepdims", [False, True])
def test_nanmean_nanvar_nanstd(dt, axis, keepdims):
    rng = np.random.default_rng(227)
    a = _with_nans(rng, (19, 23, 5), dt, 0.3)
    a[:, 4, 1] = np.nan
    a[2, :, :] = np.nan
    d = dpnp.array(a)
    tol = {"f4": 2e-5, "f8": 1e-12}[dt]
    with warnings.catch_warnings():
        warnings.simplefilter("ignore", RuntimeWarning)
        for name, kw in (("nanmean", {}), ("nanvar", {}), ("nanvar", {"ddof": 1}), ("nanstd", {"ddof": 2})):
            got = getattr(dpnp, name)(d, axis=axis, keepdims=keepdims, **kw).asnumpy()
            want = getattr(np, name)(a.astype("f8"), axis=axis, keepdims=keepdims, **kw)
            assert got.dtype == a.dtype and got.shape == np.shape(want), name
            np.testing.assert_allclose(got, want, rtol=tol * 20, atol=tol, equal_nan=True, err_msg=name)
    # the oracle's restatement of the reference's composition agrees as well
    ax = tuple(range(3)) if axis is None else (axis if isinstance(axis, tuple) else (axis,))
    moved = np.moveaxis(a, ax, tuple(range(3 - len(ax), 3)))
    with warnings.catch_warnings():
        warnings.simplefilter("ignore", RuntimeWarning)
        np.testing.assert_allclose(dpnp.nanvar(d, axis=axis).asnumpy(), orc.nanvar(moved, len(ax)),
                                   rtol=tol * 20, atol=tol, equal_nan=True)
        np.testing.assert_allclose(dpnp.nanmean(d, axis=axis).asnumpy(), orc.nanmean(moved, len(ax)),
                                   rtol=tol * 20, atol=tol, equal_nan=True)


def test_nan_functions_arguments_and_other_dtypes():
    a = np.array([[1, np.nan], [3, 4]], dtype="f8")
    d = dpnp.array(a)
    # docstring examples of the reference (dpnp_iface_nanfunctions.py:583-590, 1301-1306)
    np.testing.assert_allclose(float(dpnp.nanmean(d)), 2.6666666666666665, rtol=1e-15)
    assert_same(dpnp.nanmean(d, axis=0).asnumpy(), np.array([2.0, 4.0]))
    np.testing.assert_allclose(float(dpnp.nanvar(d)), 1.5555555555555556, rtol=1e-14)
    assert_same(dpnp.nanvar(d, axis=0).asnumpy(), np.array([1.0, 0.0]))
    np.testing.assert_allclose(float(dpnp.nanstd(d)), 1.247219128924647, rtol=1e-14)
    # integer input takes the plain functions
    i = dpnp.array(np.arange(12, dtype="i4").reshape(3, 4))
    assert int(dpnp.nansum(i)) == 66 and dpnp.nansum(i).dtype == np.dtype("i8")
    assert int(dpnp.nanargmax(i)) == 11 and int(dpnp.nanmax(i)) == 11
    assert float(dpnp.nanmean(i)) == 5.5
    # out=, dtype=
    out = dpnp.empty(2, dtype="f8")
    assert dpnp.nansum(d, axis=1, out=out) is out
    assert_same(out.asnumpy(), np.array([1.0, 7.0]))
    assert dpnp.nansum(dpnp.array(a.astype("f4")), dtype="f8").dtype == np.dtype("f8")
    oi = dpnp.empty(2, dtype="i8")
    assert dpnp.nanargmin(d, axis=0, out=oi) is oi
    assert_same(oi.asnumpy(), np.array([0, 1]))
    with pytest.raises(TypeError):
        dpnp.nanmean(d, dtype="i4")
    with pytest.raises(TypeError):
        dpnp.nanmean(d, out=dpnp.empty((), dtype="i4"))
    with pytest.raises(NotImplementedError):
        dpnp.nanmean(d, where=False)
    with pytest.raises(TypeError):
        dpnp.nanargmax(d, axis=0, out=dpnp.empty(2, dtype="f4"))
    # complex sums skip NaN in either part
    c = np.array([1 + 2j, np.nan + 1j, 3 - 1j, 2 + np.nan * 1j], dtype="c8")
    assert complex(dpnp.nansum(dpnp.array(c))) == 4 + 1j
    assert complex(dpnp.nanprod(dpnp.array(c))) == (1 + 2j) * (3 - 1j)
    np.testing.assert_allclose(complex(dpnp.nanmean(dpnp.array(c))), 2 + 0.5j)
    # mean= keyword of nanvar (dpnp/tests/test_nanfunctions.py:716-717)
    b = np.array([[14, 8, np.nan, 10], [7, 9, 10, 11], [np.nan, 15, 5, 10]])
    db = dpnp.array(b)
    mu = dpnp.nanmean(db, axis=1, keepdims=True)
    np.testing.assert_allclose(dpnp.nanvar(db, axis=1, mean=mu).asnumpy(), [6.22222222, 2.1875, 16.66666667], rtol=1e-8)
    # empty input
    e = dpnp.array(np.zeros((0, 3), dtype="f4"))
    assert_same(dpnp.nansum(e, axis=0).asnumpy(), np.zeros(3, dtype="f4"))
    with pytest.raises(ValueError):
        dpnp.nanmax(e, axis=0)


@pytest.mark.parametrize("dt", [str(np.dtype(d)) for d in ALL])
def test_all_any_count_nonzero_every_dtype_in_one_pass(dt):
    rng = np.random.default_rng(241)
    a = random_array(rng, (9, 70, 11), dt, -2, 2)
    if np.dtype(dt).kind in "fc":
        a[0, 0, 0] = np.nan                      # NaN is true
    if np.dtype(dt).kind == "c":
        a[1, 1, 1] = 1j                          # a non-zero imaginary part alone is true
    a[:, 5, :] = 0                               # an all-false run along axis 1 ... not a full one
    a[3] = 0
    d = dev(a)
    for axis in (None, 0, 1, 2, (0, 2), (1, 2)):
        assert_same(host(dpt.all(d, axis=axis)), np.all(a, axis=axis))
        assert_same(host(dpt.any(d, axis=axis)), np.any(a, axis=axis))
        assert_same(host(dpt.count_nonzero(d, axis=axis)), np.asarray(np.count_nonzero(a, axis=axis), dtype="i8"))
    v = d[::2, ::-3, 1:]
    hv = a[::2, ::-3, 1:]
    assert_same(host(dpt.any(v, axis=1, keepdims=True)), np.any(hv, axis=1, keepdims=True))
    assert_same(host(dpt.count_nonzero(v, axis=(0, 1))), np.asarray(np.count_nonzero(hv, axis=(0, 1)), dtype="i8"))
    e = dpt.empty((0, 4), dtype=dt)
    assert_same(host(dpt.all(e, axis=0)), np.ones(4, dtype=bool))
    assert_same(host(dpt.any(e, axis=0)), np.zeros(4, dtype=bool))
    assert int(dpt.count_nonzero(e)) == 0
    big = np.zeros(3_000_001, dtype=dt)
    big[-1] = 1
    assert bool(dpt.any(dev(big))) and not bool(dpt.all(dev(big))) and int(dpt.count_nonzero(dev(big))) == 1


# (beyond 256 columns of 1-byte elements a block has fewer threads than the matrix has columns)
FLAT_COLS = [2, 3, 5, 7, 10, 16, 17, 31, 33, 60, 64, 100, 127, 200, 255, 256, 257, 300, 500, 511]


@pytest.mark.parametrize("dt", ["?", "i1", "u2", "i4", "f2", "f4", "f8", "c8", "c16"])
def test_axis0_of_matrices_with_short_rows(dt):
    # a row shorter than 512 bytes: the reduction over rows reads the matrix as one flat stream
    rng = np.random.default_rng(41)
    itemsize = np.dtype(dt).itemsize
    for cols in FLAT_COLS:
        if cols * itemsize >= 512:
            continue
        for rows in (16, 17, 255, 4099, 60013):
            a = random_array(rng, (rows, cols), dt, lo=-3, hi=3)
            da = dev(a)
            check_sum(host(dpt.sum(da, axis=0)), a, 0)
            assert_same(host(dpt.max(da, axis=0)), orc.reduce("max", a.T, 1))
            assert_same(host(dpt.min(da, axis=0)), orc.reduce("min", a.T, 1))
            assert_same(host(dpt.any(da, axis=0)), a.astype(bool).any(axis=0))
            assert_same(host(dpt.all(da, axis=0)), a.astype(bool).all(axis=0))
            assert_same(host(dpt.count_nonzero(da, axis=0)), np.count_nonzero(a, axis=0).astype("i8"))
    # a view that starts at a later row, and a strided destination
    a = random_array(rng, (5000, 17), dt, lo=-3, hi=3)
    da = dev(a)
    check_sum(host(dpt.sum(da[3:], axis=0)), a[3:], 0)
    assert_same(host(dpt.max(da[1:4001], axis=0)), orc.reduce("max", a[1:4001].T, 1))
    out = dpt.zeros(34, dtype=dpt.max(da, axis=0).dtype)
    dpt.max(da, axis=0, out=out[::2])
    assert_same(host(out)[::2], orc.reduce("max", a.T, 1))
    assert (host(out)[1::2] == 0).all()


@pytest.mark.parametrize("dt", ["?", "i1", "u2", "i4", "i8", "f2", "f4", "f8", "c8", "c16"])
def test_argmax_argmin_axis0_of_matrices_with_short_rows(dt):
    # the flat stream again: the row of each column's extremum; values in -3..3 tie all the time (the first row
    # wins), NaNs beat every number (the first one wins), enough rows for several blocks
    rng = np.random.default_rng(43)
    itemsize = np.dtype(dt).itemsize
    for cols in FLAT_COLS:
        if cols * itemsize >= 512:
            continue
        # (the oracle compares complex values one by one in Python: fewer rows for them)
        for rows in ((16, 17, 255, 4099) if np.dtype(dt).kind == "c" else (16, 17, 255, 4099, 60013, 300007)):
            a = random_array(rng, (rows, cols), dt, lo=-3, hi=3)
            da = dev(a)
            assert_same(host(dpt.argmax(da, axis=0)), orc.argreduce("argmax", a.T, 1))
            assert_same(host(dpt.argmin(da, axis=0)), orc.argreduce("argmin", a.T, 1))
            if np.dtype(dt).kind in "fc" and rows > 255:
                a[rng.random(a.shape) < 0.001] = np.nan
                a[rows // 2:, 0] = 0  # a column whose NaNs, if any, lie in the first half
                da = dev(a)
                assert_same(host(dpt.argmax(da, axis=0)), orc.argreduce("argmax", a.T, 1))
                assert_same(host(dpt.argmin(da, axis=0)), orc.argreduce("argmin", a.T, 1))
    a = random_array(rng, (3000, 17), dt, lo=-3, hi=3)
    da = dev(a)
    assert_same(host(dpt.argmax(da[3:], axis=0)), orc.argreduce("argmax", a[3:].T, 1))
    out = dpt.zeros(34, dtype="i8")
    dpt.argmin(da, axis=0, out=out[::2])
    assert_same(host(out)[::2], orc.argreduce("argmin", a.T, 1))
    assert (host(out)[1::2] == 0).all()
    if np.dtype(dt).kind == "f":  # the NaN-ignoring searches take the same kernel
        a = random_array(rng, (70001, 5), dt, lo=-3, hi=3)
        a[rng.random(a.shape) < 0.3] = np.nan
        a[0, :] = 0
        assert_same(dpnp.asnumpy(dpnp.nanargmax(dpnp.array(a), axis=0)), np.nanargmax(a, axis=0))
        assert_same(dpnp.asnumpy(dpnp.nanargmin(dpnp.array(a), axis=0)), np.nanargmin(a, axis=0))


@pytest.mark.parametrize("dt", ["i1", "i4", "f2", "f4", "f8", "c16"])
def test_argmax_argmin_down_few_long_columns(dt):
    # rows of 512 bytes and more, few column blocks, so many blocks per column: their (value, row) pairs are
    # folded group by group and then across the groups.  Ties all over (the first row wins, in whichever block
    # it lies), the extremum planted in the first and in the last block, NaNs that beat every number
    import dpnp_amd._lib as L
    rng = np.random.default_rng(44)
    itemsize = np.dtype(dt).itemsize
    for cols, rows in ((512 // itemsize, 150_000), (512 // itemsize + 3, 70_001), (1024 // itemsize, 40_000)):
        if np.dtype(dt).kind == "c":  # (the oracle compares complex values one by one in Python)
            rows = 4200 + rows // 100
        a = random_array(rng, (rows, cols), dt, lo=-3, hi=3)
        da = dev(a)
        p = L.Plan()
        res = dpt.empty(cols, dtype="i8")
        L.check(L.lib.dpx_argreduce_plan(L.SEARCH_ID["argmax"], da.T._as_view(), 1, res._as_view(), p))
        assert L.PATH_NAMES[p.path] == "red_cols_split" and p.splits >= 64, (cols, p.splits)
        assert_same(host(dpt.argmax(da, axis=0)), orc.argreduce("argmax", a.T, 1))
        assert_same(host(dpt.argmin(da, axis=0)), orc.argreduce("argmin", a.T, 1))
        if np.dtype(dt).kind != "c":
            b = a.copy()
            b[5, 0], b[rows - 2, 1], b[rows // 2, 2] = 100, 100, 100
            b[7, 3], b[rows - 1, 4] = -100, -100
            db = dev(b)
            got = host(dpt.argmax(db, axis=0))
            assert_same(got, np.argmax(b, axis=0))
            assert (got[0], got[1], got[2]) == (5, rows - 2, rows // 2)
            assert_same(host(dpt.argmin(db, axis=0)), np.argmin(b, axis=0))
        if np.dtype(dt).kind in "fc":
            a[rng.random(a.shape) < 0.0005] = np.nan
            a[rows // 2:, 0] = 0
            da = dev(a)
            assert_same(host(dpt.argmax(da, axis=0)), orc.argreduce("argmax", a.T, 1))
            assert_same(host(dpt.argmin(da, axis=0)), orc.argreduce("argmin", a.T, 1))
        if np.dtype(dt).kind == "f":
            a[0, :] = 0
            assert_same(dpnp.asnumpy(dpnp.nanargmax(dpnp.array(a), axis=0)), np.nanargmax(a, axis=0))


@pytest.mark.parametrize("dt", ["i1", "u2", "i4", "f2", "f4", "f8", "c8"])
def test_argmax_argmin_along_a_short_middle_axis(dt):
    # batch x (8 to 64) x features: a block takes several batch indices, a thread walks its whole column.  Ties
    # (the first wins), NaNs, batch counts that do not fill the last block, feature counts that end inside a
    # pack, a sliced and a transposed source, a strided result
    import dpnp_amd._lib as L
    rng = np.random.default_rng(45)
    for shape in ((300, 32, 70), (1000, 8, 128), (77, 64, 33), (4099, 16, 7), (50, 40, 1030)):
        if np.dtype(dt).kind == "c" and shape[0] > 300:
            continue  # (the oracle compares complex values one by one in Python)
        a = random_array(rng, shape, dt, lo=-3, hi=3)
        da = dev(a)
        want_max, want_min = orc.argreduce("argmax", np.moveaxis(a, 1, 2), 1), orc.argreduce("argmin", np.moveaxis(a, 1, 2), 1)
        assert_same(host(dpt.argmax(da, axis=1)), want_max)
        assert_same(host(dpt.argmin(da, axis=1)), want_min)
        if np.dtype(dt).kind in "fc":
            a[rng.random(shape) < 0.01] = np.nan
            da = dev(a)
            assert_same(host(dpt.argmax(da, axis=1)), orc.argreduce("argmax", np.moveaxis(a, 1, 2), 1))
        if np.dtype(dt).kind == "f":
            a[:, 0, :] = 0
            assert_same(dpnp.asnumpy(dpnp.nanargmin(dpnp.array(a), axis=1)), np.nanargmin(a, axis=1))
    a = random_array(rng, (301, 34, 72), dt, lo=-3, hi=3)
    da = dev(a)
    if np.dtype(dt).kind != "c":
        assert_same(host(dpt.argmax(da[1:, 1:-1, 2:], axis=1)), np.argmax(a[1:, 1:-1, 2:], axis=1))
        out = dpt.zeros((301, 144), dtype="i8")
        dpt.argmin(da, axis=1, out=out[:, ::2])
        assert_same(host(out)[:, ::2], np.argmin(a, axis=1))
        assert (host(out)[:, 1::2] == 0).all()
        at = np.ascontiguousarray(a.transpose(1, 0, 2))  # the same data with the short axis outermost in memory
        assert_same(host(dpt.argmax(dpt.permute_dims(dev(at), (1, 0, 2)), axis=1)), np.argmax(a, axis=1))
    p = L.Plan()
    res = dpt.empty((300, 70), dtype="i8")
    v = dpt.permute_dims(dev(random_array(rng, (300, 32, 70), dt, lo=-3, hi=3)), (0, 2, 1))
    L.check(L.lib.dpx_argreduce_plan(L.SEARCH_ID["argmax"], v._as_view(), 1, res._as_view(), p))
    assert L.PATH_NAMES[p.path] == "red_cols" and p.block == 256 and p.splits == 1


@pytest.mark.parametrize("dt", ["?", "i1", "u1", "i2", "u2"])
@pytest.mark.parametrize("odt", ["f4", "f8"])
def test_sums_of_narrow_integers_into_floats_are_exact(dt, odt):
    # added up in 64-bit integers and converted once: the exact sum, correctly rounded, in every kernel family
    # (rows, columns, flat short rows, staged short rows, walked views, split runs), and mean through them
    rng = np.random.default_rng(46)
    def exact(a, axis):
        return np.sum(a.astype("i8"), axis=axis).astype(odt)
    for shape, axis in (((1 << 22,), None), ((3000, 4097), 1), ((3000, 4097), 0), ((100003, 7), 0), ((100003, 7), 1),
                        ((64, 7, 4096), (0, 2)), ((300, 1100), None), ((5, 1 << 20), 1), ((1 << 18, 40), 0)):
        a = random_array(rng, shape, dt, -300, 300)
        assert_same(host(dpt.sum(dev(a), axis=axis, dtype=odt)), exact(a, axis))
    a = random_array(rng, (700, 900), dt, -300, 300)
    assert_same(host(dpt.sum(dev(a)[1:-1, ::2], dtype=odt)), exact(a[1:-1, ::2], None))
    assert_same(host(dpt.sum(dev(a)[:, ::2], axis=0, dtype=odt)), exact(a[:, ::2], 0))
    out = dpt.zeros(1800, dtype=odt)
    dpt.sum(dev(a), axis=0, dtype=odt, out=out[::2])
    assert_same(host(out)[::2], exact(a, 0))
    if dt != "?":  # the mean of integers is their float64 sum over the count
        img = random_array(rng, (50, 64, 300), dt, -300, 300)
        np.testing.assert_allclose(host(dpt.mean(dev(img), axis=0)), img.astype("f8").mean(axis=0), rtol=1e-15)
        np.testing.assert_allclose(dpnp.asnumpy(dpnp.mean(dpnp.array(img), axis=(1, 2))), img.astype("f8").mean(axis=(1, 2)),
                                   rtol=1e-15)


@pytest.mark.parametrize("dt", ["f4", "f8"])
def test_statistics_over_samples_of_few_features(dt):
    # (samples, features) with few features: mean / var / std / logsumexp / hypot / nan forms over axis 0
    rng = np.random.default_rng(43)
    for cols in (3, 8, 17, 64 if dt == "f8" else 100):
        if cols * np.dtype(dt).itemsize >= 512:
            continue
        a = rng.normal(2.0, 3.0, (100003, cols)).astype(dt)
        da = dev(a)
        tol = dict(rtol=2e-5, atol=1e-5) if dt == "f4" else dict(rtol=1e-12, atol=1e-12)
        a64 = a.astype("f8") if dt == "f4" else a.astype(np.longdouble)
        np.testing.assert_allclose(host(dpt.mean(da, axis=0)), a64.mean(axis=0).astype(dt), **tol)
        np.testing.assert_allclose(host(dpt.var(da, axis=0)), a64.var(axis=0).astype(dt), **tol)
        np.testing.assert_allclose(host(dpt.std(da, axis=0, correction=1)), a64.std(axis=0, ddof=1).astype(dt), **tol)
        np.testing.assert_allclose(host(dpt.reduce_hypot(da, axis=0)), np.sqrt((a64 * a64).sum(axis=0)).astype(dt), **tol)
        m = a64.max(axis=0)
        np.testing.assert_allclose(host(dpt.logsumexp(da, axis=0)), (m + np.log(np.exp(a64 - m).sum(axis=0))).astype(dt), **tol)
        b = a.copy()
        b[rng.random(b.shape) < 0.1] = np.nan
        b64 = b.astype("f8") if dt == "f4" else b.astype(np.longdouble)
        db = dpnp.asarray(b)
        np.testing.assert_allclose(dpnp.nansum(db, axis=0).asnumpy(), np.nansum(b64, axis=0).astype(dt), **tol)
        np.testing.assert_allclose(dpnp.nanmean(db, axis=0).asnumpy(), np.nanmean(b64, axis=0).astype(dt), **tol)
        np.testing.assert_allclose(dpnp.nanvar(db, axis=0).asnumpy(), np.nanvar(b64, axis=0).astype(dt), **tol)
        assert_same(dpnp.nanmax(db, axis=0).asnumpy(), np.nanmax(b, axis=0))
    # results are reproducible bit for bit
    a = rng.normal(size=(200003, 17)).astype(dt)
    r1, r2 = host(dpt.sum(dev(a), axis=0)), host(dpt.sum(dev(a), axis=0))
    assert_same(r1, r2)


@pytest.mark.parametrize("dt", ["?", "i1", "u1", "i2", "u2", "f2"])
def test_column_reductions_of_narrow_types_every_row_count(dt):
    # 1- and 2-byte inputs go down the columns two packs at a time with the next two in flight, the integer sums
    # through dot-product instructions: every count of rows per thread around the loop's steps, the extreme values
    # of the type, whole packs and a row length that ends inside one, one block and several
    rng = np.random.default_rng(53)
    lo, hi = (0, 2) if dt == "?" else ((-4, 5) if dt == "f2" else (np.iinfo(dt).min, np.iinfo(dt).max + 1))
    for rows in list(range(1, 40)) + [63, 64, 65, 97, 130, 257, 1000, 4099, 70001]:
        for cols in (1024, 1000 + 7):
            if rows > 5000 and cols != 1024:
                continue
            a = rng.integers(lo, hi, (rows, cols)).astype(dt)
            if dt not in ("?", "f2"):
                a[rng.random(a.shape) < 0.2] = np.iinfo(dt).min
                a[rng.random(a.shape) < 0.2] = np.iinfo(dt).max
            da = dev(a)
            if dt == "f2":
                np.testing.assert_allclose(host(dpt.sum(da, axis=0)).astype("f8"), a.astype("f8").sum(axis=0), rtol=2e-3, atol=0.5)
            else:
                wide = "u8" if dt in ("u1", "u2") else "i8"
                assert_same(host(dpt.sum(da, axis=0)), a.astype(wide).sum(axis=0))
                assert_same(host(dpt.sum(da, axis=0, dtype="i4")), a.astype("i8").sum(axis=0).astype("i4"))
            assert_same(host(dpt.count_nonzero(da, axis=0)), np.count_nonzero(a, axis=0).astype("i8"))
            assert_same(host(dpt.max(da, axis=0)), a.max(axis=0))
            assert_same(host(dpt.min(da, axis=0)), a.min(axis=0))
            assert_same(host(dpt.any(da, axis=0)), a.astype(bool).any(axis=0))
    # rows that are slices of wider rows, and every other row (a walked view)
    a = rng.integers(lo, hi, (3001, 2100)).astype(dt)
    da = dev(a)
    if dt != "f2":
        wide = "u8" if dt in ("u1", "u2") else "i8"
        assert_same(host(dpt.sum(da[:, 16:1040], axis=0)), a[:, 16:1040].astype(wide).sum(axis=0))
        assert_same(host(dpt.sum(da[::2, 16:1040], axis=0)), a[::2, 16:1040].astype(wide).sum(axis=0))
        assert_same(host(dpt.count_nonzero(da[1::3, :1024], axis=0)), np.count_nonzero(a[1::3, :1024], axis=0).astype("i8"))
    assert_same(host(dpt.max(da[::2, 16:1040], axis=0)), a[::2, 16:1040].max(axis=0))


@pytest.mark.parametrize("dt", ["?", "i1", "u1"])
def test_one_byte_counting_reductions_word_arithmetic(dt):
    # sum / any / all / count_nonzero of one-byte types fold 16 elements at a time with word arithmetic:
    # every byte value, lengths around the pack and wave sizes, offsets, rows and full reductions
    rng = np.random.default_rng(47)
    every = np.arange(256, dtype="u1").view(dt) if dt != "?" else (np.arange(256) % 2).astype(bool)
    for n in (1, 15, 16, 17, 255, 1024, 4099, 65536 + 5, 3000017):
        a = np.resize(every, n).copy()
        rng.shuffle(a)
        for k in (0, 1, 3):
            v, dv = a[k:], dev(a)[k:]
            assert_same(host(dpt.sum(dv)), orc.reduce("sum", v, 1))
            assert_same(host(dpt.count_nonzero(dv)), np.array(np.count_nonzero(v), "i8"))
            assert bool(dpt.any(dv)) == bool(v.any()) and bool(dpt.all(dv)) == bool(v.all())
            if dt != "?" and v.size:  # max and min fold a pack with packed 16-bit instructions
                assert_same(host(dpt.max(dv)), np.array(v.max(), dt))
                assert_same(host(dpt.min(dv)), np.array(v.min(), dt))
    z = np.zeros(100003, dtype=dt)
    assert not bool(dpt.any(dev(z))) and int(dpt.count_nonzero(dev(z))) == 0
    z[77777] = True if dt == "?" else (-128 if dt == "i1" else 128)
    assert bool(dpt.any(dev(z))) and int(dpt.count_nonzero(dev(z))) == 1 and not bool(dpt.all(dev(z)))
    o = np.full(100003, 1 if dt != "i1" else -1, dtype=dt)
    assert bool(dpt.all(dev(o)))
    o[3] = 0
    assert not bool(dpt.all(dev(o)))
    m = np.resize(every, (257, 1031)).copy()
    dm = dev(m)
    assert_same(host(dpt.sum(dm, axis=1)), orc.reduce("sum", m, 1))
    assert_same(host(dpt.count_nonzero(dm, axis=1)), np.count_nonzero(m, axis=1).astype("i8"))
    assert_same(host(dpt.all(dm, axis=1)), m.astype(bool).all(axis=1))
    if dt != "?":
        # the extreme of each row planted at every place of a pack, among values next to it
        lo, hi = (np.iinfo(dt).min, np.iinfo(dt).max)
        e = rng.integers(lo + 2, hi - 1, (64, 4099)).astype(dt)
        for r in range(64):
            e[r, 2048 + r] = hi if r % 2 else hi - 1
            e[r, 1000 + 3 * r] = lo if r % 3 else lo + 1
        de = dev(e)
        assert_same(host(dpt.max(de, axis=1)), e.max(axis=1))
        assert_same(host(dpt.min(de, axis=1)), e.min(axis=1))
        assert_same(host(dpt.max(de[:, 1:])), np.array(e[:, 1:].max(), dt))
        assert_same(host(dpt.min(de[3:, 5:4000], axis=1)), e[3:, 5:4000].min(axis=1))
    assert_same(host(dpt.any(dm[:, :5], axis=1)), m[:, :5].astype(bool).any(axis=1))
    assert_same(host(dpt.sum(dm, axis=1, dtype="i4")), orc.reduce("sum", m, 1, out_dtype="i4"))


@pytest.mark.parametrize("dt", ["?", "i1", "u2", "i4", "f2", "f4", "f8", "c8", "c16"])
def test_last_axis_of_matrices_with_short_rows(dt):
    # rows of at most 256 bytes reduced along the row: a block stages whole rows in LDS
    rng = np.random.default_rng(53)
    itemsize = np.dtype(dt).itemsize
    for cols in (2, 3, 4, 5, 8, 10, 16, 17, 31, 32, 33, 63, 64, 128, 256):
        if cols * itemsize > 256:
            continue
        for rows in (64, 65, 255, 256, 257, 1000, 40009):
            a = random_array(rng, (rows, cols), dt, lo=-3, hi=3)
            da = dev(a)
            check_sum(host(dpt.sum(da, axis=1)), a, 1)
            assert_same(host(dpt.max(da, axis=-1)), orc.reduce("max", a, 1))
            assert_same(host(dpt.min(da, axis=-1)), orc.reduce("min", a, 1))
            assert_same(host(dpt.all(da, axis=1)), a.astype(bool).all(axis=1))
            assert_same(host(dpt.count_nonzero(da, axis=1)), np.count_nonzero(a, axis=1).astype("i8"))
    a = random_array(rng, (5000, 3, 7), dt, lo=-3, hi=3)  # outer dims collapse into the rows
    da = dev(a)
    assert_same(host(dpt.max(da, axis=2)), orc.reduce("max", a, 1))
    check_sum(host(dpt.sum(da, axis=(1, 2))), a.reshape(5000, 21), 1)
    b = random_array(rng, (5000, 10), dt, lo=-3, hi=3)
    db = dev(b)
    assert_same(host(dpt.max(db[7:], axis=1)), orc.reduce("max", b[7:], 1))  # view that starts at a later row
    out = dpt.zeros(10000, dtype=dt)
    dpt.max(db, axis=1, out=out[::2])
    assert_same(host(out)[::2], orc.reduce("max", b, 1))


@pytest.mark.parametrize("dt", ["f4", "f8"])
def test_per_row_statistics_of_short_rows(dt):
    # (points, 3) norms, (samples, classes) softmax statistics: mean / var / logsumexp / hypot / nan forms
    rng = np.random.default_rng(59)
    tol = dict(rtol=2e-5, atol=1e-5) if dt == "f4" else dict(rtol=1e-12, atol=1e-12)
    for cols in (3, 10, 17, 32 if dt == "f8" else 64):
        a = rng.normal(1.0, 2.0, (30011, cols)).astype(dt)
        da = dev(a)
        a64 = a.astype("f8") if dt == "f4" else a.astype(np.longdouble)
        np.testing.assert_allclose(host(dpt.mean(da, axis=1)), a64.mean(axis=1).astype(dt), **tol)
        np.testing.assert_allclose(host(dpt.var(da, axis=1)), a64.var(axis=1).astype(dt), **tol)
        np.testing.assert_allclose(host(dpt.std(da, axis=1, correction=1)), a64.std(axis=1, ddof=1).astype(dt), **tol)
        np.testing.assert_allclose(host(dpt.reduce_hypot(da, axis=1)), np.sqrt((a64 * a64).sum(axis=1)).astype(dt), **tol)
        mx = a64.max(axis=1, keepdims=True)
        np.testing.assert_allclose(host(dpt.logsumexp(da, axis=1)),
                                   (mx[:, 0] + np.log(np.exp(a64 - mx).sum(axis=1))).astype(dt), **tol)
        np.testing.assert_allclose(host(dpt.prod(dev(a[:, :5]), axis=1)), a64[:, :5].prod(axis=1).astype(dt), **tol)
        b = a.copy()
        b[rng.random(b.shape) < 0.2] = np.nan
        b[:, 0] = 1.0
        b64 = b.astype("f8") if dt == "f4" else b.astype(np.longdouble)
        db = dpnp.asarray(b)
        np.testing.assert_allclose(dpnp.nansum(db, axis=1).asnumpy(), np.nansum(b64, axis=1).astype(dt), **tol)
        np.testing.assert_allclose(dpnp.nanmean(db, axis=1).asnumpy(), np.nanmean(b64, axis=1).astype(dt), **tol)
        np.testing.assert_allclose(dpnp.nanvar(db, axis=1).asnumpy(), np.nanvar(b64, axis=1).astype(dt), **tol)
        assert_same(dpnp.nanmin(db, axis=1).asnumpy(), np.nanmin(b, axis=1))


@pytest.mark.parametrize("dt", ["?", "i1", "u2", "i4", "f2", "f4", "f8", "c8"])
def test_argmax_argmin_along_short_rows(dt):
    # the predicted class of each sample: first position of the extremum, the first NaN wins
    rng = np.random.default_rng(61)
    itemsize = np.dtype(dt).itemsize
    for cols in (2, 3, 5, 10, 17, 32, 33, 64, 100):
        if cols * itemsize > 256:
            continue
        for rows in (64, 257, 3001, 50021):
            a = random_array(rng, (rows, cols), dt, lo=-4, hi=4)  # many ties
            if np.dtype(dt).kind == "f":
                a[rng.random(a.shape) < 0.02] = np.nan
                a[1, :] = np.nan
            da = dev(a)
            assert_same(host(dpt.argmax(da, axis=1)), orc.argreduce("argmax", a, 1))
            assert_same(host(dpt.argmin(da, axis=-1)), orc.argreduce("argmin", a, 1))
    a = rng.normal(size=(4001, 3, 7)).astype("f4") if dt == "f4" else None
    if a is not None:
        a[rng.random(a.shape) < 0.1] = np.nan
        a[:, 0, 0] = 0.0
        da = dpnp.asarray(a)
        assert_same(host(dpt.argmax(dev(a), axis=2)), orc.argreduce("argmax", a, 1))
        assert_same(dpnp.nanargmax(da, axis=2).asnumpy(), np.nanargmax(a, axis=2))
        assert_same(dpnp.nanargmin(da[:, 0, :], axis=1).asnumpy(), np.nanargmin(a[:, 0, :], axis=1))
        out = dpt.zeros(2 * 4001, dtype="i8")
        dpt.argmax(dev(a[:, 1, :]), axis=1, out=out[::2])
        assert_same(host(out)[::2], orc.argreduce("argmax", a[:, 1, :], 1))


# Reduced dims that do not collapse into one run: (base shape, view, axes).  The runs of the last reduced dim are
# whole packs, ragged (a partial pack ends each run), shorter than a pack, strided, reversed; one, few and many
# outputs; reductions large enough to be split over blocks.
_WALKED = [
    ((40, 50), np.s_[:, 1:-1], None),
    ((40, 50), np.s_[1:-1, 3:], None),
    ((700, 900), np.s_[:, 1:-1], None),
    ((700, 900), np.s_[::2, ::2], None),
    ((700, 900), np.s_[::-1, ::3], None),
    ((300, 1100), np.s_[:, ::2], 1),
    ((300, 1100), np.s_[:, ::-2], 1),
    ((300, 1100), np.s_[:, 5:1001:3], 1),
    ((9, 1000, 33), np.s_[:], (0, 2)),
    ((9, 1000, 32), np.s_[:], (0, 2)),
    ((9, 1000, 3), np.s_[:], (0, 2)),
    ((9, 1000, 1), np.s_[:, ::2], (0, 2)),
    ((64, 7, 4096), np.s_[:], (0, 2)),
    ((33, 5, 4100), np.s_[:, :, 1:-2], (0, 2)),
    ((5, 3, 70000), np.s_[:, :, 1:], (0, 2)),
    ((2, 3, 70000), np.s_[:, :, ::2], (0, 2)),
    ((12, 13, 14, 15), np.s_[:], (0, 2)),
    ((12, 13, 14, 15), np.s_[:], (1, 3)),
    ((12, 13, 14, 15), np.s_[:], (0, 3)),
    ((12, 13, 14, 15), np.s_[:], (0, 1, 3)),
    ((12, 13, 14, 15), np.s_[:, 1:, :, 2:], (0, 2, 3)),
    ((12, 13, 14, 15), np.s_[:, 1:, 1:, 2:], (1, 2, 3)),
    ((12, 13, 14, 16), np.s_[1:, 1:, 1:, ::2], None),
    ((6, 5, 4, 3, 8), np.s_[:, 1:, 1:, 1:, 1:], None),
    ((6, 5, 4, 3, 8), np.s_[:, 1:, 1:, 1:, 1:], (0, 2, 4)),
    ((3, 200000), np.s_[:, 1:], None),
    ((200000, 3), np.s_[:, 1:], None),
    ((200000, 3), np.s_[:, :2], 1),
    # the inner iteration dim is the one src moves least along: columns side by side, rows walked
    ((300, 1100), np.s_[:, ::2], 0),
    ((300, 1100), np.s_[:, ::-1], 0),
    ((300, 1100), np.s_[::2, 7::3], 0),
    ((12, 13, 14, 16), np.s_[:, :, :, ::2], (0, 2)),
    ((12, 13, 14, 16), np.s_[:, :, 1:, 1:], (0, 2)),
    ((64, 5, 64, 130), np.s_[:], (0, 2)),
    ((3000, 2, 50, 9), np.s_[:], (0, 2)),
    ((40, 3, 50, 2, 70), np.s_[:], (0, 2)),
    ((7, 3, 6, 2, 5, 70), np.s_[:], (0, 2, 4)),
    ((150000, 2, 9), np.s_[:, :, ::2], 0),
    # more outputs than a split plan has blocks, long walked spaces: fewer lanes per output than a whole block
    ((8, 1024, 1024), np.s_[:], (0, 2)),
    ((8, 2048, 512), np.s_[:], (0, 2)),
    ((8, 4096, 512), np.s_[:, :, 1:], (0, 2)),
    ((1024, 4100), np.s_[:, ::2], 1),
]


@pytest.mark.parametrize("dt", ["?", "i1", "u2", "i4", "i8", "f2", "f4", "f8", "c8", "c16"])
@pytest.mark.parametrize("case", range(len(_WALKED)))
def test_reduced_dims_that_stay_apart(case, dt):
    shape, sl, axis = _WALKED[case]
    rng = np.random.default_rng(7000 + case)
    base = random_array(rng, shape, dt, -3, 3)
    hv = base[sl]
    v = dev_view_like(hv, base)
    dt = np.dtype(dt)
    check_sum(host(dpt.sum(v, axis=axis)), hv, axis)
    if dt.kind != "c":
        assert_same(host(dpt.max(v, axis=axis)), np.max(hv, axis=axis))
        assert_same(host(dpt.min(v, axis=axis)), np.min(hv, axis=axis))
    assert_same(host(dpt.count_nonzero(v, axis=axis)), np.asarray(np.count_nonzero(hv, axis=axis), dtype="i8"))
    assert_same(host(dpt.any(v, axis=axis)), np.asarray(np.any(hv, axis=axis)))
    if dt.kind == "f" and dt.itemsize >= 4:
        tol = 1e-5 if dt.itemsize == 4 else 1e-12
        want = np.mean(hv.astype(np.longdouble), axis=axis)
        np.testing.assert_allclose(host(dpt.mean(v, axis=axis)), want.astype("f8"), rtol=0, atol=4 * tol)
        want = np.var(hv.astype(np.longdouble), axis=axis)
        np.testing.assert_allclose(host(dpt.var(v, axis=axis)), want.astype("f8"), rtol=10 * tol, atol=10 * tol)
    if axis is None or isinstance(axis, int):
        if dt.kind != "c":
            assert_same(host(dpt.argmax(v, axis=axis)), np.asarray(np.argmax(hv, axis=axis)))
            assert_same(host(dpt.argmin(v, axis=axis)), np.asarray(np.argmin(hv, axis=axis)))
        if dt.kind == "f":  # the first NaN wins, as in NumPy
            base = base.copy()
            base[rng.random(shape) < 0.001] = np.nan
            hv = base[sl]
            v = dev_view_like(hv, base)
            assert_same(host(dpt.argmax(v, axis=axis)), np.asarray(np.argmax(hv, axis=axis)))
            assert_same(host(dpt.argmin(v, axis=axis)), np.asarray(np.argmin(hv, axis=axis)))
            assert_same(host(dpt.max(v, axis=axis)), np.max(hv, axis=axis))


def _exact_var(a, axis, ddof=0):
    a = a.astype(np.longdouble)
    m = a.mean(axis=axis, keepdims=True)
    n = a.size if axis is None else a.shape[axis]
    return (((a - m) ** 2).sum(axis=axis) / (n - ddof)).astype("f8")


@pytest.mark.parametrize("dt", ["f4", "f8"])
def test_variance_in_one_pass_over_contiguous_runs(dt):
    # float64 accumulation over the last axes of a C-contiguous array takes the one-pass kernel: data far from
    # zero, outliers at the places lanes start from, constants, tiny and split runs; 1e-12 of the exact variance
    rng = np.random.default_rng(97)
    def check(a, axis, ddof=0):
        got = host(dpt.var(dev(a), axis=axis, correction=ddof, dtype="f8"))
        want = _exact_var(a, axis, ddof)
        np.testing.assert_allclose(got, want, rtol=1e-12, atol=0)
    for n in (1, 2, 3, 5, 63, 64, 257, 4099, 70001, 2_000_003, 1 << 24):
        a = rng.standard_normal(n).astype(dt)
        if n > 1:
            check(a, None)
            check(a, None, ddof=1)
        else:
            assert host(dpt.var(dev(a), dtype="f8")) == 0.0
        big = (a.astype("f8") * 3 + 1e6).astype(dt)  # mean / sigma = 3e5
        if n > 1:
            check(big, None)
    a = rng.standard_normal(1 << 22).astype(dt)
    a[::4096] = 1e6  # outliers where lanes take their shift from
    check(a, None)
    a[:] = 7.25
    assert host(dpt.var(dev(a), dtype="f8")) == 0.0
    for shape in ((1000, 3), (300, 700), (7, 100003), (64, 65, 66)):
        a = (rng.standard_normal(shape) * 2 - 50).astype(dt)
        check(a, -1)
        check(a, -1, ddof=1)
        if len(shape) == 3:
            got = host(dpt.var(dev(a), axis=(1, 2), dtype="f8"))
            np.testing.assert_allclose(got, _exact_var(a.reshape(shape[0], -1), 1), rtol=1e-12)
    # down the columns (and over the leading axes): the column kernel's one-pass form
    for shape in ((1000, 3), (300, 700), (100003, 7), (5, 20011), (4099, 1001), (20000, 128)):
        a = (rng.standard_normal(shape) * 2 + 1e5).astype(dt)
        a[::97] += 1e4  # outliers
        check(a, 0)
        check(a, 0, ddof=1)
    a = (rng.standard_normal((40, 50, 600)) - 7).astype(dt)
    got = host(dpt.var(dev(a), axis=(0, 1), dtype="f8"))
    np.testing.assert_allclose(got, _exact_var(a.reshape(-1, 600), 0), rtol=1e-12)
    got = host(dpt.var(dev(a), axis=1, dtype="f8"))  # a middle axis: outputs contiguous under it
    np.testing.assert_allclose(got, _exact_var(a, 1), rtol=1e-12)
    # reduced dims that stay apart (lanes walk them): axes (0, 2), sliced matrices, every other element, ragged runs
    a = (rng.standard_normal((40, 50, 601)) * 3 + 1e5).astype(dt)
    np.testing.assert_allclose(host(dpt.var(dev(a), axis=(0, 2), dtype="f8")),
                               _exact_var(np.moveaxis(a, 1, 0).reshape(50, -1), 1), rtol=1e-12)
    np.testing.assert_allclose(host(dpt.var(dev(a)[:, :, ::2], axis=(0, 2), dtype="f8")),
                               _exact_var(np.moveaxis(a[:, :, ::2], 1, 0).reshape(50, -1), 1), rtol=1e-12)
    m = (rng.standard_normal((700, 900)) - 1e4).astype(dt)
    m[::31, ::29] = 1e3
    for sl in (np.s_[1:-1, 1:-1], np.s_[:, ::2], np.s_[::2, 3:], np.s_[:, :5]):
        np.testing.assert_allclose(host(dpt.var(dev(m)[sl], dtype="f8")), _exact_var(m[sl].reshape(-1), None), rtol=1e-12)
        np.testing.assert_allclose(host(dpt.var(dev(m)[sl], axis=1, dtype="f8", correction=1)),
                                   _exact_var(m[sl], 1, 1), rtol=1e-12)
    # columns side by side with the rows of the reduced space walked (every other column, every third, a 4-d
    # array over axes (0, 2)), and reduced dims the kernels index one element at a time (more than three apart)
    import dpnp_amd._lib as L
    for sl in (np.s_[:, ::2], np.s_[:, 7::3], np.s_[::2, ::-1], np.s_[:, :3:2]):
        v = dev(m)[sl]
        p = L.Plan()
        res = dpt.empty(v.shape[1], dtype="f8")
        L.check(L.lib.dpx_reduce_plan(L.REDUCE_ID["sqdev_onepass"], v.T._as_view(), 1, res._as_view(), p))
        assert L.PATH_NAMES[p.path] in ("red_cols", "red_cols_split", "red_generic"), L.PATH_NAMES[p.path]
        np.testing.assert_allclose(host(dpt.var(v, axis=0, dtype="f8")), _exact_var(m[sl], 0), rtol=1e-12)
        np.testing.assert_allclose(host(dpt.var(v, axis=0, dtype="f8", correction=1)), _exact_var(m[sl], 0, 1), rtol=1e-12)
    big = (rng.standard_normal((60013, 40)) * 2 + 1e5).astype(dt)  # columns split over blocks
    np.testing.assert_allclose(host(dpt.var(dev(big)[:, ::2], axis=0, dtype="f8")), _exact_var(big[:, ::2], 0), rtol=1e-12)
    np.testing.assert_allclose(host(dpt.var(dev(big)[:, ::3], axis=0, dtype="f8")), _exact_var(big[:, ::3], 0), rtol=1e-12)
    a4 = (rng.standard_normal((12, 13, 14, 16)) * 3 - 1e4).astype(dt)
    np.testing.assert_allclose(host(dpt.var(dev(a4), axis=(0, 2), dtype="f8")),
                               _exact_var(a4.transpose(1, 3, 0, 2).reshape(13, 16, -1), 2), rtol=1e-12)
    a6 = (rng.standard_normal((5, 4, 6, 3, 7, 9)) * 3 + 1e4).astype(dt)
    for sl6, axes in ((np.s_[:, 1:, 1:, 1:, 1:, 1:], None), (np.s_[:, 1:, 1:, 1:, 1:, 1:], (1, 2, 3, 4, 5)),
                      (np.s_[1:, :, 1:, :, 1:, :], (0, 2, 4))):
        h6 = a6[sl6]
        keep = [d for d in range(6) if axes is not None and d not in axes]
        flat = h6.transpose(keep + [d for d in range(6) if d not in keep]).reshape([h6.shape[d] for d in keep] + [-1])
        np.testing.assert_allclose(host(dpt.var(dev(a6)[sl6], axis=axes, dtype="f8")), _exact_var(flat, -1), rtol=1e-12)
    # non-finite values spread as in the two-pass form
    a = rng.standard_normal(5000).astype(dt)
    a[123] = np.nan
    assert np.isnan(host(dpt.var(dev(a), dtype="f8")))
    a[123] = np.inf
    assert np.isnan(host(dpt.var(dev(a), dtype="f8")))
    # float16 input with a float16 result: accumulated in float64, rounded once (runs whose float16 sum would overflow)
    if dt == "f4":
        h = (rng.standard_normal((300, 70000)) * 3 + 40).astype("f2")
        for ax in (None, 0, 1):
            got = host(dpt.var(dev(h), axis=ax))
            assert got.dtype == np.float16
            np.testing.assert_array_equal(got, _exact_var(h, ax).astype("f2"))
        # (std is the square root of the rounded variance, taken in float16: within an ULP of the exact one)
        np.testing.assert_allclose(host(dpt.std(dev(h), axis=1, correction=1)).astype("f8"), np.sqrt(_exact_var(h, 1, 1)),
                                   rtol=1e-3)
    # integer input: float64 result straight from the integers
    for idt in ("i1", "u2", "i4", "u8"):
        a = rng.integers(0, 100, (300, 700)).astype(idt)
        for ax in (None, 0, 1):
            np.testing.assert_allclose(host(dpt.var(dev(a), axis=ax)), _exact_var(a, ax), rtol=1e-12)
    # std, and the dpnp layer
    a = rng.standard_normal((50, 4001)).astype(dt)
    np.testing.assert_allclose(host(dpt.std(dev(a), axis=1, dtype="f8")), np.sqrt(_exact_var(a, 1)), rtol=1e-12)
    np.testing.assert_allclose(dpnp.asnumpy(dpnp.var(dpnp.array(a), axis=1, dtype="f8", ddof=1)), _exact_var(a, 1, 1),
                               rtol=1e-12)


@pytest.mark.parametrize("dt", ["f2", "f4", "f8"])
def test_logsumexp_every_kernel_family_and_special_values(dt):
    # (largest element, sum of exponentials relative to it) pairs: rows, columns, flat and walked kernels, split
    # runs, infinities and NaN
    rng = np.random.default_rng(211)
    rtol = {"f2": 2e-3, "f4": 1e-5, "f8": 1e-12}[dt]
    def want(a, axis):
        a = a.astype(np.longdouble)
        m = np.max(a, axis=axis, keepdims=True)
        m = np.where(np.isfinite(m), m, 0)
        with np.errstate(divide="ignore", invalid="ignore"):
            r = np.log(np.sum(np.exp(a - m), axis=axis)) + np.squeeze(m, axis=axis) if axis is not None \
                else np.log(np.sum(np.exp(a - m))) + m.reshape(())
        return np.asarray(r)
    for shape, axis in (((2_000_003,), None), ((4099,), None), ((300, 700), 1), ((300, 700), 0), ((100003, 7), 0),
                        ((1000, 3), 1), ((40, 50, 60), (0, 2)), ((5, 20011), 0), ((700, 900), None)):
        a = (rng.standard_normal(shape) * (3 if dt == "f2" else 30)).astype(dt)
        got = host(dpt.logsumexp(dev(a), axis=axis)).astype(np.longdouble)
        np.testing.assert_allclose(got, want(a, axis), rtol=rtol, atol=rtol)
    a = (rng.standard_normal((700, 900)) * 5).astype(dt)
    got = host(dpt.logsumexp(dev(a)[1:-1, 1:-1])).astype(np.longdouble)  # a sliced matrix: the walked kernel
    np.testing.assert_allclose(got, want(a[1:-1, 1:-1], None), rtol=rtol)
    # special values, alone and among numbers, in runs long enough for the batched path
    base = (rng.standard_normal(5000) * 3).astype(dt)
    for v, res in ((-np.inf, None), (np.inf, np.inf), (np.nan, np.nan)):
        a = base.copy()
        a[[0, 17, 4999]] = v
        got = float(dpt.logsumexp(dev(a)))
        if res is None:
            np.testing.assert_allclose(got, float(want(a, None)), rtol=rtol)
        elif np.isnan(res):
            assert np.isnan(got)
        else:
            assert got == res
    assert float(dpt.logsumexp(dev(np.full(3000, -np.inf, dtype=dt)))) == -np.inf
    assert float(dpt.logsumexp(dev(np.full(3000, np.inf, dtype=dt)))) == np.inf
    assert np.isnan(float(dpt.logsumexp(dev(np.array([np.inf, -np.inf, np.nan], dtype=dt)))))
    assert float(dpt.logsumexp(dev(np.array([np.inf, -np.inf], dtype=dt)))) == np.inf
