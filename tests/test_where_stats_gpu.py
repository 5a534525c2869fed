"""where, mean, var, std against the oracle and the reference's known answers."""
import json
import os

import numpy as np
import pytest

import dpnp_amd.tensor as dpt
from oracle import oracle as orc
from tests.helpers import ALL, assert_same, dev, host, random_array

pytestmark = pytest.mark.gpu
GOLD = json.load(open(os.path.join(os.path.dirname(__file__), "golden", "reference_known_answers.json")))


def test_where_basic():
    # dpnp/tests/tensor/test_usm_ndarray_search_functions.py:69-100
    g = GOLD["where_basic"]
    cond = dev(np.array(g["cond"], dtype=bool))
    want = np.array(g["expected"])
    assert (host(dpt.where(cond, dpt.asarray(1), dpt.asarray(0))) == want).all()
    assert (host(dpt.where(cond, dpt.ones(cond.shape), dpt.zeros(cond.shape))) == want).all()
    r = dpt.where(cond, dpt.ones(cond.shape[0], dtype="i4")[:, None], dpt.zeros(cond.shape[0], dtype="i4")[:, None])
    assert (host(r) == want).all() and r.dtype == np.dtype("i4")


@pytest.mark.parametrize("cdt", ALL, ids=str)
def test_where_condition_dtypes_and_value_sizes(cdt):
    rng = np.random.default_rng(71)
    c = random_array(rng, 3001, cdt, -2, 2)
    if cdt.kind == "f":
        c[:3] = [-0.0, np.nan, 0.0]
    for vdt in ("i1", "f2", "f4", "f8", "c16", "?"):
        x1, x2 = random_array(rng, 3001, vdt), random_array(rng, 3001, vdt)
        assert_same(host(dpt.where(dev(c), dev(x1), dev(x2))), orc.where(c, x1, x2))


def test_where_promotion_broadcast_scalars_out():
    rng = np.random.default_rng(73)
    c = random_array(rng, (50, 60), "?")
    a = random_array(rng, (50, 60), "i4")
    b = random_array(rng, (1, 60), "f4")
    r = dpt.where(dev(c), dev(a), dev(b))
    assert r.dtype == np.result_type("i4", "f4")
    assert_same(host(r), np.where(c, a, b))
    assert_same(host(dpt.where(dev(c), dev(a), 7)), np.where(c, a, np.int32(7)))
    assert dpt.where(dev(c), 1.5, dev(a)).dtype == np.dtype("f8")
    assert dpt.where(dev(c), True, False).dtype == np.dtype("?")
    o = dpt.empty((50, 60), dtype="i4")
    assert dpt.where(dev(c), dev(a), dev(a[::-1].copy()), out=o) is o
    assert_same(host(o), np.where(c, a, a[::-1]))
    x = dev(a)
    dpt.where(dev(c), x, dev(a[::-1].copy()), out=x)  # out is x1
    assert_same(host(x), np.where(c, a, a[::-1]))
    # unaligned operands (dpnp/tests/tensor/test_usm_ndarray_search_functions.py:451)
    n = 1001
    cc, xx = random_array(rng, n, "?"), random_array(rng, n, "f4")
    assert_same(host(dpt.where(dev(cc)[1:], dev(xx)[1:], dev(xx)[:-1])), np.where(cc[1:], xx[1:], xx[:-1]))
    assert dpt.where(dpt.empty((0,), dtype="?"), dpt.empty((0,)), dpt.empty((0,))).shape == (0,)
    with pytest.raises(ValueError):
        dpt.where(dev(c), dev(a), dev(a), out=dpt.empty((50, 60), dtype="f4"))


def test_mean_var_std_known_answers():
    # dpnp/tests/tensor/test_tensor_statistical_functions.py:159-241
    g, v = GOLD["mean_3x3"], GOLD["var_3x3"]
    x = dpt.reshape(dpt.arange(9, dtype="f4"), (3, 3))
    assert float(dpt.mean(x)) == g["mean"] and dpt.mean(x).dtype == np.dtype("f4")
    np.testing.assert_allclose(host(dpt.mean(x, axis=0)), g["mean_axis0"], rtol=1e-6)
    np.testing.assert_allclose(host(dpt.mean(x, axis=1)), g["mean_axis1"], rtol=1e-6)
    np.testing.assert_allclose(float(dpt.var(x)), v["var"], rtol=1e-6)
    np.testing.assert_allclose(float(dpt.var(x, correction=3)), v["var_corr3"], rtol=1e-6)
    np.testing.assert_allclose(host(dpt.var(x, axis=0)), v["var_axis0"], rtol=1e-6)
    np.testing.assert_allclose(host(dpt.var(x, axis=0, correction=1)), v["var_axis0_corr1"], rtol=1e-6)
    np.testing.assert_allclose(host(dpt.var(x, axis=1)), v["var_axis1"], rtol=1e-6)
    np.testing.assert_allclose(host(dpt.var(x, axis=1, correction=1)), v["var_axis1_corr1"], rtol=1e-6)
    np.testing.assert_allclose(float(dpt.std(x)), np.sqrt(v["var"]), rtol=1e-6)
    np.testing.assert_allclose(host(dpt.std(x, axis=0, correction=1)), np.sqrt(v["var_axis0_corr1"]), rtol=1e-6)
    assert np.isnan(float(dpt.var(x, correction=9)))
    assert np.isnan(host(dpt.var(x, axis=0, correction=3))).all()
    assert np.isnan(host(dpt.var(x, axis=1, correction=3))).all()
    # dtype rule and empty input (:55-122)
    for dt in ALL:
        if dt.kind == "c":
            continue
        r = dpt.mean(dpt.ones(10, dtype=dt))
        assert r.dtype == (dt if dt.kind == "f" else np.dtype("f8")) and float(r) == 1.0
        assert dpt.var(dpt.ones(10, dtype=dt)).dtype == (dt if dt.kind == "f" else np.dtype("f8"))
    assert np.isnan(float(dpt.mean(dpt.empty((0,), dtype="f4"))))
    assert np.isnan(float(dpt.var(dpt.empty((0,), dtype="f4"))))
    assert dpt.mean(x, axis=()).shape == (3, 3) and (host(dpt.var(x, axis=())) == 0).all()
    assert dpt.mean(x, axis=1, keepdims=True).shape == (3, 1) and dpt.var(x, axis=0, keepdims=True).shape == (1, 3)
    with pytest.raises(ValueError):
        dpt.var(dpt.ones(3, dtype="c8"))


@pytest.mark.parametrize("dt,rtol", [("f4", 1e-5), ("f8", 1e-12)])
def test_mean_var_random(dt, rtol):
    rng = np.random.default_rng(79)
    a = (rng.standard_normal((64, 5000)) * 3 + 10).astype(dt)
    da = dev(a)
    for axis, tr in ((1, a), (0, a.T), (None, a.reshape(1, -1))):
        want_m, want_v = orc.mean(tr, 1), orc.var(tr, 1)
        got_m, got_v = host(dpt.mean(da, axis=axis)), host(dpt.var(da, axis=axis))
        np.testing.assert_allclose(got_m.reshape(want_m.shape), want_m, rtol=rtol)
        np.testing.assert_allclose(got_v.reshape(want_v.shape), want_v, rtol=max(rtol, 1e-5 if dt == "f4" else rtol))
    if dt == "f4":  # accumulation in float64 on request: float64 accuracy from float32 data
        got = float(dpt.var(da, dtype="f8"))
        np.testing.assert_allclose(got, float(orc.var(a.reshape(1, -1), 1, out_dtype="f8")[0]), rtol=1e-12)
        got = float(dpt.mean(da, dtype="f8"))
        np.testing.assert_allclose(got, float(orc.mean(a.reshape(1, -1), 1, out_dtype="f8")[0]), rtol=1e-12)
    i = rng.integers(-50, 50, (30, 40)).astype("i4")
    np.testing.assert_allclose(host(dpt.var(dev(i), axis=1, correction=1)), orc.var(i, 1, correction=1), rtol=1e-12)
    nanned = a.copy()
    nanned[3, 17] = np.nan
    r = host(dpt.var(dev(nanned), axis=1))
    assert np.isnan(r[3]) and not np.isnan(np.delete(r, 3)).any()


@pytest.mark.parametrize("dt", ["?", "i1", "u1", "i2", "u2", "i4", "u4", "i8", "u8"])
def test_mean_var_of_integer_arrays_in_one_pass(dt):
    """Integer input is summed straight into float64 (no cast copy): same values as the cast path."""
    import dpnp_amd._lib as L
    from dpnp_amd.tensor._dtypes import dtype_id

    rng = np.random.default_rng(61)
    a = random_array(rng, (37, 501), dt, -100, 100)
    d = dev(a)
    for axis in (None, 0, 1):
        m, v = host(dpt.mean(d, axis=axis)), host(dpt.var(d, axis=axis))
        assert m.dtype == np.dtype("f8") and v.dtype == np.dtype("f8")
        np.testing.assert_allclose(m, np.mean(a.astype("f8"), axis=axis), rtol=1e-13)
        np.testing.assert_allclose(v, np.var(a.astype("f8"), axis=axis), rtol=1e-12, atol=1e-12)
    assert L.lib.dpx_reduce_dtype_supported(L.REDUCE_ID["sum"], dtype_id(np.dtype(dt)), dtype_id(np.dtype("f8"))) == 1
    s = dpt.sum(d, dtype="f4")
    np.testing.assert_allclose(float(s), float(np.sum(a.astype("f8"))), rtol=1e-5, atol=1e-2)


@pytest.mark.parametrize("dt", ["f4", "f8"])
def test_one_pass_variance_propagates_inf_and_nan_in_every_kernel_form(dt):
    """inf or NaN anywhere in a run gives NaN (inf - mean is inf, inf * 0 in the merge is NaN), a run without
    them its variance: short rows (one lane per row), long rows, columns, reduced dims that stay apart, a
    sliced matrix.  The one-pass kernels keep (count, mean, M2) triples; a clamp of a NaN M2 to zero, or a merge
    with an untouched accumulator skipped, would give a finite result here."""
    rng = np.random.default_rng(83)
    cases = [((600, 5), 1), ((600, 8), 1), ((40, 3000), 1), ((3, 200000), 1), ((3000, 70), 0), ((40000, 6), 0),
             ((6, 300, 40), (0, 2)), ((50, 40, 30), (0, 2))]
    for shape, axis in cases:
        a = rng.standard_normal(shape).astype(dt) + 5
        out_shape = np.var(a, axis=axis).shape
        for bad in (np.inf, -np.inf, np.nan):
            h = a.copy()
            hit = np.zeros(out_shape, bool)
            for o in rng.choice(hit.size, size=min(3, hit.size), replace=False):
                oi = np.unravel_index(o, out_shape)
                hit[oi] = True
                # one element of that output's run, first, last or inside
                full = [slice(None)] * len(shape)
                keep = [d for d in range(len(shape)) if d not in (axis if isinstance(axis, tuple) else (axis,))]
                for d, i in zip(keep, oi):
                    full[d] = i
                run = np.ascontiguousarray(h[tuple(full)])
                run.reshape(-1)[rng.choice([0, run.size - 1, run.size // 2])] = bad
                h[tuple(full)] = run
            got = host(dpt.var(dev(h), axis=axis, dtype="f8"))
            assert np.isnan(got[hit]).all(), (shape, axis, bad)
            np.testing.assert_allclose(got[~hit], np.var(a.astype("f8"), axis=axis)[~hit], rtol=1e-10)
    # a sliced matrix reduced whole, the bad element at a corner of the slice and just outside it
    h = rng.standard_normal((300, 400)).astype(dt)
    h[0, 0] = np.nan  # outside the slice
    d = dev(h)
    assert np.isfinite(float(dpt.var(d[1:-1, 1:-1], dtype="f8")))
    h[1, 1] = np.inf
    assert np.isnan(float(dpt.var(dev(h)[1:-1, 1:-1], dtype="f8")))
