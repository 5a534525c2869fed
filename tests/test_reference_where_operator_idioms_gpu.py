"""`where` and the array operators exercised the way the reference's tests do
(dpnp/tests/tensor/test_usm_ndarray_search_functions.py, test_usm_ndarray_operators.py)."""
import ctypes
import itertools

import numpy as np
import pytest

import dpnp_amd.tensor as dpt

pytestmark = pytest.mark.gpu

ALL = ["?", "i1", "u1", "i2", "u2", "i4", "u4", "i8", "u8", "f2", "f4", "f8", "c8", "c16"]


def _tile_rows(pattern, reps):
    """A 2-D bool array whose rows repeat `pattern` (stand-in for dpt.tile in the reference's tests)."""
    return dpt.asarray(np.tile(np.asarray(pattern, dtype=bool), reps))


# ---- where: test_usm_ndarray_search_functions.py ----------------------------------------------------
def test_where_basic_and_broadcast():
    # :69-110
    cond = dpt.asarray([[True, False, False], [False, True, False], [False, False, True],
                        [False, False, False], [True, True, True]])
    out = dpt.where(cond, dpt.asarray(1), dpt.asarray(0))
    assert np.array_equal(dpt.asnumpy(out), dpt.asnumpy(cond).astype("i8"))
    out = dpt.where(cond, dpt.ones(cond.shape), dpt.zeros(cond.shape))
    assert np.array_equal(dpt.asnumpy(out), dpt.asnumpy(cond).astype("f8"))
    out = dpt.where(cond, dpt.ones(cond.shape[0])[:, dpt.newaxis], dpt.zeros(cond.shape[0])[:, dpt.newaxis])
    assert np.array_equal(dpt.asnumpy(out), dpt.asnumpy(cond).astype("f8"))
    # :281-291 (a 1-D condition against 2-D branches)
    cond = dpt.asarray([False, True, True, False], dtype="?")
    res = dpt.where(cond, dpt.ones((3, 4), dtype="i4"), dpt.zeros((3, 4), dtype="i4"))
    assert np.array_equal(dpt.asnumpy(res), np.broadcast_to(dpt.asnumpy(cond).astype("i4"), (3, 4)))


@pytest.mark.parametrize("dt1", ALL)
@pytest.mark.parametrize("dt2", ["?", "i4", "u8", "f2", "f8", "c8"])
def test_where_result_types(dt1, dt2):
    # :114-133: the branches promote like NumPy
    cond = dpt.asarray(np.random.default_rng(0).integers(0, 2, 10).astype(bool))
    x1, x2 = dpt.ones(10, dtype=dt1), dpt.zeros(10, dtype=dt2)
    res = dpt.where(cond, x1, x2)
    want = np.where(dpt.asnumpy(cond), dpt.asnumpy(x1), dpt.asnumpy(x2))
    assert res.dtype == want.dtype
    assert np.array_equal(dpt.asnumpy(res), want)


@pytest.mark.parametrize("dt", ALL)
def test_where_condition_of_any_dtype(dt):
    # :136-168: a condition element is true when it is not zero
    c = np.asarray([0, 1, 2, 0, 3], dtype="i1").astype(dt)
    res = dpt.where(dpt.asarray(c), dpt.ones(5, dtype="i4"), dpt.zeros(5, dtype="i4"))
    assert np.array_equal(dpt.asnumpy(res), (c != 0).astype("i4"))
    a = dpt.asarray(c)
    assert np.array_equal(dpt.asnumpy(dpt.where(a, a, dpt.zeros_like(a))), c)


def test_where_nan_inf_and_empty():
    # :189-237
    cond = dpt.asarray([True, False, True, False], dtype="?")
    x1 = dpt.asarray([np.nan, 2.0, np.inf, 3.0], dtype="f4")
    x2 = dpt.asarray([2.0, np.nan, 3.0, np.inf], dtype="f4")
    want = np.where(dpt.asnumpy(cond), dpt.asnumpy(x1), dpt.asnumpy(x2))
    np.testing.assert_array_equal(dpt.asnumpy(dpt.where(cond, x1, x2)), want)
    empty = dpt.empty(0, dtype="i2")
    m, x1, x2 = dpt.asarray(True), dpt.asarray(1, dtype="i2"), dpt.asarray(2, dtype="i2")
    assert dpt.where(empty, x1, x2).shape == (0,) and dpt.where(empty, x1, x2).dtype == dpt.dtype("i2")
    assert dpt.where(m, empty, x2).shape == (0,)
    with pytest.raises(ValueError):
        dpt.where(empty, x1, dpt.empty((1, 2)))


def test_where_strided_views_and_invariants():
    # :294-359
    rng = np.random.default_rng(1)
    s0, s1 = 4, 9
    x1 = dpt.reshape(dpt.arange(0, s0 * s1, dtype="i4"), (s0, s1))[::-2, ::-2]
    x2 = dpt.reshape(dpt.arange(s0 * s1, 2 * s0 * s1, dtype="i4"), (s1, s0))[::2, ::2].mT
    cond = dpt.asarray(rng.integers(0, 2, x1.shape).astype(bool))
    want = np.where(dpt.asnumpy(cond), dpt.asnumpy(x1), dpt.asnumpy(x2))
    assert np.array_equal(dpt.asnumpy(dpt.where(cond, x1, x2)), want)
    assert np.array_equal(dpt.asnumpy(dpt.where(cond, dpt.copy(x1), dpt.copy(x2))), want)
    mask = dpt.asarray(rng.integers(0, 2, (6, 8)).astype(bool))
    p, m = dpt.ones((6, 8), dtype=dpt.int16), dpt.full((6, 8), -1, dtype=dpt.int16)
    for ind in [(np.s_[:3], np.s_[::2]), (np.s_[::2], np.s_[::2]), (np.s_[::-1], np.s_[:])]:
        r1 = dpt.where(mask, p, m)[ind]
        r2 = dpt.where(mask[ind], p[ind], m[ind])
        assert (dpt.asnumpy(r1) == dpt.asnumpy(r2)).all()
    x = dpt.ones(513, dtype="i4")     # :451-459, a condition that starts off a 16-byte boundary
    assert dpt.all(dpt.where(x[1:], dpt.full(512, 2, dtype="i4"), dpt.zeros(512, dtype="i4")) == dpt.full(512, 2, dtype="i4"))


def test_where_argument_validation():
    # :362-374, :519-543
    x1, x2 = dpt.empty((1,), dtype="i4"), dpt.empty((1,), dtype="i4")
    with pytest.raises(TypeError):
        dpt.where({}, x1, x2)
    with pytest.raises(ValueError):
        dpt.where(x1, {}, x2)
    with pytest.raises(ValueError):
        dpt.where(x1, x2, {})
    condition = dpt.ones(5, dtype="i4")
    a, b = dpt.ones(5, dtype="i4"), dpt.ones(5, dtype="i4")
    read_only = dpt.empty_like(condition)
    read_only.flags["W"] = False
    with pytest.raises(TypeError):
        dpt.where(condition, a, b, out=dict())
    with pytest.raises(ValueError):
        dpt.where(condition, a, b, out=dpt.empty_like(condition, dtype="f4"))
    with pytest.raises(ValueError):
        dpt.where(condition, a, b, out=dpt.empty(6, dtype="i4"))
    with pytest.raises(ValueError):
        dpt.where(condition, a, b, out=read_only)


def test_where_order_of_the_result():
    # :393-448
    sh, sh2, n = (20, 20), (40, 40), 20
    for dt1, dt2 in zip(["i4", "i4", "f4"], ["i4", "f4", "i4"]):
        ar1, ar2 = dpt.zeros(sh, dtype=dt1, order="C"), dpt.ones(sh, dtype=dt2, order="C")
        condition = dpt.zeros(sh, dtype="?", order="C")
        assert dpt.where(condition, ar1, ar2, order="C").flags.c_contiguous
        assert dpt.where(condition, ar1, ar2, order="F").flags.f_contiguous
        assert dpt.where(condition, ar1, ar2, order="A").flags.c_contiguous
        assert dpt.where(condition, ar1, ar2, order="K").flags.c_contiguous
        ar1, ar2 = dpt.ones(sh, dtype=dt1, order="F"), dpt.ones(sh, dtype=dt2, order="F")
        condition = dpt.zeros(sh, dtype="?", order="F")
        assert dpt.where(condition, ar1, ar2, order="C").flags.c_contiguous
        assert dpt.where(condition, ar1, ar2, order="F").flags.f_contiguous
        assert dpt.where(condition, ar1, ar2, order="A").flags.f_contiguous
        assert dpt.where(condition, ar1, ar2, order="K").flags.f_contiguous
        ar1 = dpt.ones(sh2, dtype=dt1, order="C")[:20, ::-2]
        ar2 = dpt.ones(sh2, dtype=dt2, order="C")[:20, ::-2]
        condition = dpt.zeros(sh2, dtype="?", order="C")[:20, ::-2]
        assert dpt.where(condition, ar1, ar2, order="K").strides == (n, -1)
        assert dpt.where(condition, ar1, ar2, order="C").strides == (n, 1)
        ar1, ar2, condition = ar1.mT, ar2.mT, condition.mT
        assert dpt.where(condition, ar1, ar2, order="K").strides == (-1, n)
        assert dpt.where(condition, ar1, ar2, order="C").strides == (n, 1)
        ar1 = dpt.ones(n, dtype=dt1, order="C")
        ar2 = dpt.broadcast_to(dpt.ones(n, dtype=dt2, order="C"), sh)
        condition = dpt.zeros(n, dtype="?", order="C")
        assert dpt.where(condition, ar1, ar2, order="K").strides == (20, 1)


def test_where_out_views_and_overlap():
    # :462-516
    n1, n2, n3 = 3, 4, 5
    ar1 = dpt.reshape(dpt.arange(n1 * n2 * n3, dtype="i4"), (n1, n2, n3))
    ar2 = dpt.full_like(ar1, -5)
    pattern = np.tile(np.asarray([True, False, False, True]).reshape(1, n2, 1), (n1, 1, n3))
    condition = dpt.asarray(pattern)
    out = dpt.zeros((2 * n1, 3 * n2, n3), dtype="i4")
    res = dpt.where(condition, ar1, ar2, out=out[::-2, 1::3, :])
    assert dpt.all(res == out[::-2, 1::3, :])
    assert dpt.all(out[::-2, 0::3, :] == 0) and dpt.all(out[::-2, 2::3, :] == 0)
    assert dpt.all(res[:, 1:3, :] == -5) and dpt.all(res[:, 0, :] == ar1[:, 0, :]) and dpt.all(res[:, 3, :] == ar1[:, 3, :])

    condition = dpt.asarray(np.tile(np.asarray([1, 0], dtype="i4").reshape(1, 2, 1), (n1, 2, n3)))
    res = dpt.where(condition[:, ::-1, :], condition[:, ::-1, :], condition, out=condition)
    assert dpt.all(res == condition) and dpt.all(condition == 1)

    condition = dpt.asarray(np.tile(np.asarray([True, False]).reshape(1, 2, 1), (n1, 2, n3)))
    ar1 = dpt.full((n1, n2, n3), 7, dtype="i4")
    ar2 = dpt.full_like(ar1, -5)
    res = dpt.where(condition, ar1, ar2, out=ar2[:, ::-1, :])
    assert dpt.all(ar2[:, ::-1, :] == res) and dpt.all(ar2[:, ::2, :] == -5) and dpt.all(ar2[:, 1::2, :] == 7)
    ar1 = dpt.full((n1, n2, n3), 7, dtype="i4")
    ar2 = dpt.full_like(ar1, -5)
    res = dpt.where(condition, ar1, ar2, out=ar1[:, ::-1, :])
    assert dpt.all(ar1[:, ::-1, :] == res) and dpt.all(ar1[:, ::2, :] == -5) and dpt.all(ar1[:, 1::2, :] == 7)


@pytest.mark.parametrize("arr_dt", ALL)
def test_where_python_scalar_branches(arr_dt):
    # :546-596
    condition = _tile_rows([True, False], (10, 5))
    x = dpt.zeros((10, 10), dtype=arr_dt)
    scalars = (bool(0), int(0), float(0), complex(0), np.float32(0), ctypes.c_int(0))
    for sc in scalars:
        assert isinstance(dpt.where(condition, x, sc), dpt.usm_ndarray)
        assert isinstance(dpt.where(condition, sc, x), dpt.usm_ndarray)
    if arr_dt == "?":
        for sc1, sc2 in itertools.product(scalars, repeat=2):
            assert isinstance(dpt.where(condition, sc1, sc2), dpt.usm_ndarray)


# ---- operators: test_usm_ndarray_operators.py:63-160 ---------------------------------------------
def test_every_floating_operator_runs():
    X = dpt.ones(1)
    assert X.__array_namespace__() is dpt
    X[0] = -2.5
    for name in ("__add__", "__radd__", "__sub__", "__rsub__", "__mul__", "__rmul__", "__truediv__", "__rtruediv__",
                 "__floordiv__", "__rfloordiv__"):
        assert isinstance(getattr(X, name)(1.0), dpt.usm_ndarray), name
    assert X.__abs__() == 2.5 and X.__pos__() == -2.5 and X.__neg__() == 2.5
    assert X.__eq__(-2.5) and not X.__ne__(-2.5) and X.__le__(-2.5) and X.__ge__(-2.5) and not X.__gt__(-2.0)
    X.__iadd__(X)
    assert X == -5.0
    X.__isub__(X)
    assert X == 0.0
    X[0] = 3.0
    X.__imul__(X)
    assert X == 9.0
    X.__itruediv__(2.0)
    assert X == 4.5
    X.__ifloordiv__(2.0)
    assert X == 2.0


def test_every_integer_operator_runs():
    X = dpt.full(1, 6, dtype="i4")
    assert X.__lshift__(2) == 24 and X.__rshift__(1) == 3 and X.__rlshift__(2) == 128 and X.__rrshift__(1 << 10) == 16
    assert X.__and__(X) == 6 and X.__or__(X) == 6 and X.__xor__(X) == 0 and X.__invert__() == -7
    assert X.__rand__(3) == 2 and X.__ror__(1) == 7 and X.__rxor__(5) == 3
    assert X.__mod__(5) == 1 and X.__rmod__(20) == 2 and X.__pow__(2) == 36 and X.__rpow__(2) == 64
    X.__ilshift__(2)
    assert X == 24
    X.__irshift__(3)
    assert X == 3
    X.__iand__(dpt.full(1, 2, dtype="i4"))
    assert X == 2
    X.__ior__(dpt.full(1, 5, dtype="i4"))
    assert X == 7
    X.__ixor__(dpt.full(1, 1, dtype="i4"))
    assert X == 6
    X.__imod__(4)
    assert X == 2
    X.__ipow__(5)
    assert X == 32


def test_comparisons_of_uint64_with_negative_python_ints():
    X = dpt.asarray(1, dtype="u8")
    assert X.__gt__(-1) and X.__ge__(-1) and not X.__lt__(-1) and not X.__le__(-1) and not X.__eq__(-1) and X.__ne__(-1)
