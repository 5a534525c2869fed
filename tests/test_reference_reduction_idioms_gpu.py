"""Reduction calls written the way the reference's own tests write them
(dpnp/tests/tensor/test_usm_ndarray_reductions.py, test_tensor_sum.py,
test_tensor_statistical_functions.py): the same entry points, keywords, views as `out=`, shapes
and error classes, so a user of the reference's tensor namespace finds the same behaviour."""
import numpy as np
import pytest

import dpnp_amd.tensor as dpt

pytestmark = pytest.mark.gpu

NUMERIC = ["i1", "u1", "i2", "u2", "i4", "u4", "i8", "u8", "f2", "f4", "f8", "c8", "c16"]
NO_COMPLEX = ["?", "i1", "u1", "i2", "u2", "i4", "u4", "i8", "u8", "f2", "f4", "f8"]


# ---- logsumexp / reduce_hypot: test_usm_ndarray_reductions.py:321-490 -----------------------------
@pytest.mark.parametrize("arg_dtype", NO_COMPLEX[1:])
def test_logsumexp_default_result_dtype(arg_dtype):
    m = dpt.ones(100, dtype=arg_dtype)
    r = dpt.logsumexp(m)
    assert isinstance(r, dpt.usm_ndarray) and r.dtype.kind == "f"
    tol = dpt.finfo(r.dtype).resolution
    # float16 accumulates in float32 here (the reference and NumPy round every partial to float16):
    # compare with the value accumulated in float64
    want = np.logaddexp.reduce(dpt.asnumpy(m).astype("f8")).astype(r.dtype)
    np.testing.assert_allclose(dpt.asnumpy(r), want, rtol=tol, atol=tol)


@pytest.mark.parametrize("arg_dtype", NO_COMPLEX[1:])
@pytest.mark.parametrize("out_dtype", ["f2", "f4", "f8"])
def test_logsumexp_and_hypot_result_dtype_matrix(arg_dtype, out_dtype):
    m = dpt.ones(100, dtype=arg_dtype)
    for fn in (dpt.logsumexp, dpt.reduce_hypot):
        r = fn(m, dtype=out_dtype)
        assert isinstance(r, dpt.usm_ndarray) and r.dtype == dpt.dtype(out_dtype)
    np.testing.assert_allclose(float(dpt.reduce_hypot(m, dtype=out_dtype)), 10.0, rtol=1e-3)


def test_logsumexp_empty_axis_keepdims_scalar_and_errors():
    y = dpt.logsumexp(dpt.empty((0,), dtype="f4"))
    assert y.shape == () and y == -dpt.inf
    assert dpt.reduce_hypot(dpt.empty((0,), dtype="f4")) == 0

    m = dpt.ones((3, 4, 5, 6, 7), dtype="f4")
    s = dpt.logsumexp(m, axis=(1, 2, -1))
    assert s.shape == (3, 6)
    tol = dpt.finfo(s.dtype).resolution
    np.testing.assert_allclose(dpt.asnumpy(s), np.logaddexp.reduce(dpt.asnumpy(m), axis=(1, 2, -1), dtype=s.dtype),
                               rtol=tol, atol=tol)
    assert dpt.logsumexp(dpt.ones((3, 4, 5, 6, 7), dtype="i4"), axis=(1, 2, -1), keepdims=True).shape == (3, 1, 1, 6, 1)

    n = 10
    a = dpt.ones((n, 0, n))
    assert dpt.logsumexp(a, keepdims=True).shape == (1, 1, 1)
    assert dpt.logsumexp(a, axis=(0, 1), keepdims=True).shape == (1, 1, n)
    assert dpt.logsumexp(a, axis=(1, 2), keepdims=True).shape == (n, 1, 1)
    assert dpt.logsumexp(a, axis=(0, 2), keepdims=True).shape == (1, 0, 1)
    assert dpt.logsumexp(a[0], keepdims=True).shape == (1, 1)

    assert dpt.logsumexp(dpt.ones(())).shape == ()
    res = dpt.logsumexp(dpt.zeros((8, 10), dtype="f4"), axis=0)
    assert res.ndim == 1 and res.shape[0] == 10
    with pytest.raises(ValueError):
        dpt.logsumexp(dpt.zeros(1, dtype="c8"))
    with pytest.raises(ValueError):
        dpt.reduce_hypot(dpt.zeros(1, dtype="c8"))
    with pytest.raises(TypeError):
        dpt.logsumexp({})


def test_tree_reduction_over_either_axis():
    x = dpt.reshape(dpt.arange(3 * 4 * 5, dtype="f4"), (3, 4, 5))
    m = dpt.logsumexp(x, axis=0)
    tol = dpt.finfo(m.dtype).resolution
    np.testing.assert_allclose(dpt.asnumpy(m), np.logaddexp.reduce(dpt.asnumpy(x), axis=0, dtype=m.dtype), rtol=tol, atol=tol)
    x = dpt.flip(x, axis=2)
    m = dpt.logsumexp(x, axis=2)
    np.testing.assert_allclose(dpt.asnumpy(m), np.logaddexp.reduce(dpt.asnumpy(x), axis=2, dtype=m.dtype), rtol=tol, atol=tol)


# ---- `out=`: test_usm_ndarray_reductions.py:518-687 ------------------------------------------------
def test_sum_into_views_of_a_larger_array():
    n1, n2, n3 = 3, 4, 5
    x = dpt.ones((n1, n2, n3), dtype="i8")
    out = dpt.zeros((2 * n1, 3 * n2), dtype="i8")
    res = dpt.sum(x, axis=-1, out=out[::-2, 1::3])
    assert dpt.all(out[::-2, 0::3] == 0) and dpt.all(out[::-2, 2::3] == 0)
    assert dpt.all(out[::-2, 1::3] == res) and dpt.all(out[::-2, 1::3] == 5)

    out = dpt.zeros((2 * n1, 3 * n2, 1), dtype="i8")
    res = dpt.sum(x, axis=-1, keepdims=True, out=out[::-2, 1::3])
    assert res.shape == (n1, n2, 1)
    assert dpt.all(out[::-2, 0::3] == 0) and dpt.all(out[::-2, 2::3] == 0)
    assert dpt.all(out[::-2, 1::3] == res) and dpt.all(out[::-2, 1::3] == 5)

    res = dpt.sum(x, axis=0, out=x[-1])          # the destination is part of the source
    assert dpt.all(x[-1] == res) and dpt.all(x[-1] == 3) and dpt.all(x[0:-1] == 1)

    x = dpt.ones((n1, n2, n3), dtype="i8")       # no axis reduced: a copy
    out = dpt.zeros((2 * n1, 3 * n2, n3), dtype="i8")
    dpt.sum(x, axis=(), out=out[::-2, 1::3])
    assert dpt.all(out[::-2, 0::3] == 0) and dpt.all(out[::-2, 2::3] == 0) and dpt.all(out[::-2, 1::3] == x)

    x = dpt.ones((n1, n2, n3), dtype="i4")       # with dtype=
    out = dpt.zeros((2 * n1, 3 * n2), dtype="f4")
    res = dpt.sum(x, axis=-1, dtype="f4", out=out[::-2, 1::3])
    assert dpt.allclose(out[::-2, 0::3], dpt.zeros_like(res)) and dpt.allclose(out[::-2, 2::3], dpt.zeros_like(res))
    assert dpt.allclose(out[::-2, 1::3], res) and dpt.allclose(out[::-2, 1::3], dpt.full_like(res, 5, dtype="f4"))


def test_max_and_argmax_into_views():
    n1, n2, n3 = 3, 4, 5
    x = dpt.reshape(dpt.arange(n1 * n2 * n3, dtype="i4"), (n1, n2, n3))
    out = dpt.zeros((2 * n1, 3 * n2), dtype="i4")
    res = dpt.max(x, axis=-1, out=out[::-2, 1::3])
    assert dpt.all(out[::-2, 0::3] == 0) and dpt.all(out[::-2, 2::3] == 0)
    assert dpt.all(out[::-2, 1::3] == res) and dpt.all(out[::-2, 1::3] == x[:, :, -1])
    out = dpt.zeros((2 * n1, 3 * n2, 1), dtype="i4")
    res = dpt.max(x, axis=-1, keepdims=True, out=out[::-2, 1::3])
    assert res.shape == (n1, n2, 1) and dpt.all(out[::-2, 1::3] == x[:, :, -1, dpt.newaxis])
    out = dpt.zeros((2 * n1, 3 * n2, n3), dtype="i4")
    dpt.max(x, axis=(), out=out[::-2, 1::3])
    assert dpt.all(out[::-2, 0::3] == 0) and dpt.all(out[::-2, 1::3] == x)
    res = dpt.max(x, axis=0, out=x[0])
    assert dpt.all(x[0] == res) and dpt.all(x[0] == x[-1])

    dt = dpt.__array_namespace_info__().default_dtypes()["indexing"]
    x = dpt.reshape(dpt.arange(n1 * n2 * n3, dtype=dt), (n1, n2, n3))
    out = dpt.zeros((2 * n1, 3 * n2), dtype=dt)
    res = dpt.argmax(x, axis=-1, out=out[::-2, 1::3])
    assert dpt.all(out[::-2, 0::3] == 0) and dpt.all(out[::-2, 2::3] == 0)
    assert dpt.all(out[::-2, 1::3] == res) and dpt.all(out[::-2, 1::3] == n3 - 1)
    out = dpt.zeros((2 * n1, 3 * n2, 1), dtype=dt)
    res = dpt.argmax(x, axis=-1, keepdims=True, out=out[::-2, 1::3])
    assert res.shape == (n1, n2, 1) and dpt.all(out[::-2, 1::3] == n3 - 1)
    x0 = dpt.ones((), dtype=dt)
    out = dpt.ones(2, dtype=dt)
    dpt.argmax(x0, axis=None, out=out[1])
    assert dpt.all(out[0] == 1) and dpt.all(out[1] == 0)
    x = dpt.reshape(dpt.arange(n1 * n2, dtype=dt), (n1, n2))
    res = dpt.argmax(x, axis=0, out=x[0])
    assert dpt.all(x[0] == res) and dpt.all(x[0] == n1 - 1)


def test_out_argument_validation():
    ind_dt = dpt.__array_namespace_info__().default_dtypes()["indexing"]
    x = dpt.ones(10, dtype="f4")
    wrong_dtype = dpt.empty((), dtype="i4")
    wrong_shape = dpt.empty(1, dtype="f4")
    scalar_out = dpt.empty((), dtype="f4")
    read_only = dpt.empty((), dtype="f4")
    read_only.flags["W"] = False
    for fn in (dpt.sum, dpt.max, dpt.argmax):
        with pytest.raises(TypeError):
            fn(x, out=dict())
    with pytest.raises(ValueError):
        dpt.sum(x, out=wrong_dtype)
    with pytest.raises(ValueError):
        dpt.max(x, out=wrong_dtype)
    with pytest.raises(ValueError):
        dpt.argmax(x, out=dpt.empty_like(wrong_dtype, dtype="f4"))
    with pytest.raises(ValueError):
        dpt.sum(x, out=wrong_shape)
    with pytest.raises(ValueError):
        dpt.max(x, out=wrong_shape)
    with pytest.raises(ValueError):
        dpt.argmax(x, out=dpt.empty_like(wrong_shape, dtype=ind_dt))
    with pytest.raises(ValueError):
        dpt.sum(x, out=read_only)
    with pytest.raises(ValueError):
        dpt.max(x, out=read_only)
    with pytest.raises(ValueError):
        ro = dpt.empty_like(read_only, dtype=ind_dt)
        ro.flags["W"] = False
        dpt.argmax(x, out=ro)
    with pytest.raises(ValueError):
        dpt.sum(x, keepdims=True, out=scalar_out)
    with pytest.raises(ValueError):
        dpt.max(x, keepdims=True, out=scalar_out)
    with pytest.raises(ValueError):
        dpt.argmax(x, keepdims=True, out=dpt.empty_like(scalar_out, dtype=ind_dt))


@pytest.mark.parametrize("dt", ["?"] + NUMERIC)
def test_count_nonzero_every_dtype(dt):
    res = dpt.count_nonzero(dpt.ones(10, dtype=dt))
    assert res == 10 and res.dtype == dpt.dtype("i8")


# ---- max/min/argmax basics: test_usm_ndarray_reductions.py:64-316 ---------------------------------
def test_max_min_of_an_arange_cube():
    x = dpt.reshape(dpt.arange((3 * 4 * 5 * 6 * 7), dtype="i4"), (3, 4, 5, 6, 7))
    m = dpt.max(x, axis=(1, 2, -1))
    assert m.shape == (3, 6)
    assert dpt.all(m == x[:, -1, -1, :, -1])
    m = dpt.min(x, axis=(1, 2, -1))
    assert dpt.all(m == x[:, 0, 0, :, 0])
    x = dpt.reshape(dpt.arange(11 * 17, dtype="i4"), (11, 17))
    assert dpt.all(dpt.max(x, axis=0) == x[-1, :]) and dpt.all(dpt.max(x, axis=1) == x[:, -1])
    assert dpt.max(dpt.ones(())).shape == ()


def test_max_min_nan_with_infinities():
    x = dpt.reshape(dpt.arange(3 * 4 * 5, dtype="f4"), (3, 4, 5))
    x[0, 0, 0] = dpt.nan
    for fn in (dpt.max, dpt.min):
        assert dpt.isnan(fn(x))
        assert dpt.isnan(fn(x, axis=0)[0, 0]) and not dpt.any(dpt.isnan(fn(x, axis=0)[1:, :]))
    x = dpt.asarray([dpt.nan, dpt.inf, -dpt.inf], dtype="f4")
    assert dpt.isnan(dpt.max(x)) and dpt.isnan(dpt.min(x))


def test_argmax_argmin_first_occurrence_and_layouts():
    x = dpt.reshape(dpt.arange(3 * 4 * 5 * 6 * 7, dtype="i4"), (3, 4, 5, 6, 7))
    m = dpt.argmax(x, axis=1, keepdims=True)
    assert m.shape == (3, 1, 5, 6, 7) and dpt.all(m == 3)
    x = dpt.asarray([dpt.nan, 0.0, dpt.nan, 5.0], dtype="f4")
    assert dpt.argmax(x) == 0 and dpt.argmin(x) == 0      # the first NaN
    x = dpt.zeros(100, dtype="i4")
    assert dpt.argmax(x) == 0 and dpt.argmin(x) == 0      # ties: the first position
    for order in ("C", "F"):
        x = dpt.asarray([[1, 0], [0, 1]], dtype="i4", order=order)
        assert list(dpt.asnumpy(dpt.argmax(x, axis=0))) == [0, 1]
        assert list(dpt.asnumpy(dpt.argmax(x, axis=1))) == [0, 1]
        assert dpt.argmax(x) == 0
    with pytest.raises(TypeError):
        dpt.argmax(dpt.ones((2, 2)), axis=(0, 1))
    with pytest.raises(ValueError):
        dpt.max(dpt.empty((0,), dtype="f4"))
    with pytest.raises(ValueError):
        dpt.argmax(dpt.empty((0, 3), dtype="f4"), axis=0)
    with pytest.raises(TypeError):
        dpt.sum({})


# ---- sum / prod: test_tensor_sum.py ---------------------------------------------------------------
@pytest.mark.parametrize("arg_dtype", ["?"] + NUMERIC)
def test_sum_default_dtype_and_all_ones(arg_dtype):
    m = dpt.ones(100, dtype=arg_dtype)
    r = dpt.sum(m)
    kind = m.dtype.kind
    assert r.dtype.kind == {"b": "i", "i": "i", "u": "u", "f": "f", "c": "c"}[kind]
    assert dpt.all(r == 100)
    assert dpt.all(dpt.sum(m[::-1]) == 100) and dpt.all(dpt.sum(m[::2]) == 50)
    p = dpt.prod(dpt.full(7, 2, dtype=arg_dtype) if kind != "b" else m)
    assert p == (128 if kind != "b" else 1)


@pytest.mark.parametrize("n", [1023, 1024, 1025])
def test_sum_sizes_around_a_block_and_strided_blocks(n):
    for dt in ("i4", "f4"):
        assert dpt.sum(dpt.ones(n, dtype=dt)) == n
    x = dpt.reshape(dpt.arange(3 * n, dtype="i8"), (3, n))
    want = np.arange(3 * n, dtype="i8").reshape(3, n)
    assert np.array_equal(dpt.asnumpy(dpt.sum(x, axis=1)), want.sum(axis=1))
    assert np.array_equal(dpt.asnumpy(dpt.sum(x, axis=0)), want.sum(axis=0))
    assert np.array_equal(dpt.asnumpy(dpt.sum(x[:, ::-2], axis=1)), want[:, ::-2].sum(axis=1))


def test_sum_misc():
    assert dpt.sum(dpt.asarray([-1, 1], dtype="i1"), dtype="?") == True  # noqa: E712  (convert first, then or)
    assert dpt.sum(dpt.empty((0,), dtype="f4")) == 0 and dpt.prod(dpt.empty((0,), dtype="i4")) == 1
    s = dpt.sum(dpt.ones((3, 4, 5, 6, 7), dtype="i4"), axis=(1, 2, -1), keepdims=True)
    assert s.shape == (3, 1, 1, 6, 1) and dpt.all(s == 4 * 5 * 7)
    n = 10
    a = dpt.ones((n, 0, n))
    assert dpt.sum(a, keepdims=True).shape == (1, 1, 1) and dpt.sum(a, axis=(0, 2), keepdims=True).shape == (1, 0, 1)
    assert dpt.sum(dpt.ones(())).shape == ()
    x = dpt.ones((2, 3), dtype="u1")
    assert dpt.sum(x, dtype="u1").dtype == dpt.dtype("u1") and dpt.sum(x).dtype == dpt.dtype("u8")


# ---- mean / var / std: test_tensor_statistical_functions.py ---------------------------------------
def test_statistics_closed_forms_and_edge_cases():
    x = dpt.reshape(dpt.arange(9, dtype="f4"), (3, 3))
    assert dpt.mean(x) == 4 and dpt.all(dpt.mean(x, axis=0) == dpt.asarray([3, 4, 5], dtype="f4"))
    np.testing.assert_allclose(float(dpt.var(x)), 6.6666665, rtol=1e-6)
    np.testing.assert_allclose(dpt.asnumpy(dpt.var(x, axis=1)), [2 / 3] * 3, rtol=1e-6)
    np.testing.assert_allclose(dpt.asnumpy(dpt.std(x, axis=0, correction=1)), [3.0] * 3, rtol=1e-6)
    for dt, want in (("i4", "f8"), ("?", "f8"), ("f2", "f2"), ("f4", "f4"), ("f8", "f8")):
        assert dpt.mean(dpt.ones(10, dtype=dt)).dtype == dpt.dtype(want)
        assert dpt.var(dpt.ones(10, dtype=dt)).dtype == dpt.dtype(want)
    assert dpt.mean(dpt.ones(10, dtype="c8")).dtype == dpt.dtype("c8")
    assert dpt.isnan(dpt.mean(dpt.empty((0,), dtype="f4"))) and dpt.isnan(dpt.var(dpt.empty((0,), dtype="f4")))
    assert dpt.isnan(dpt.var(dpt.ones(3, dtype="f4"), correction=3)) and dpt.isnan(dpt.std(dpt.ones(3), correction=4))
    assert dpt.mean(dpt.ones((3, 4, 5)), axis=(0, -1), keepdims=True).shape == (1, 4, 1)
    with pytest.raises(ValueError):
        dpt.var(dpt.ones(4, dtype="c8"))
    with pytest.raises(TypeError):
        dpt.var(dpt.ones(4), correction="1")
    with pytest.raises(TypeError):
        dpt.mean([1.0, 2.0])
