"""concatenate / stack / hstack / vstack, diff and trapezoid against NumPy, with the cases of the reference's
dpnp/tests/test_manipulation.py (TestConcatenate, TestStack, TestHstack, TestVstack), dpnp/tests/test_mathematical.py
(TestDiff, TestTrapezoid) and dpnp/tests/tensor/test_usm_ndarray_manipulation.py (test_concat_*, test_stack_*)."""
import numpy as np
import pytest

import dpnp_amd as dpnp
import dpnp_amd.tensor as dpt

pytestmark = pytest.mark.gpu


def same(result, expected):
    got = result.asnumpy()
    assert got.shape == expected.shape and got.dtype == expected.dtype, (got.shape, expected.shape, got.dtype, expected.dtype)
    np.testing.assert_array_equal(got, expected)


@pytest.mark.parametrize("axis", [0, 1, -1, None])
@pytest.mark.parametrize("dts", [("f4", "f4"), ("i4", "f4"), ("i1", "u1"), ("?", "i8"), ("f8", "c8"), ("f2", "i2")])
def test_concatenate_two_matrices(axis, dts):
    rng = np.random.default_rng(1)
    a = rng.integers(0, 9, (5, 7)).astype(dts[0])
    shape_b = (5, 7) if axis is None else ((3, 7) if axis == 0 else (5, 4))
    b = rng.integers(0, 9, shape_b).astype(dts[1])
    same(dpnp.concatenate((dpnp.array(a), dpnp.array(b)), axis=axis), np.concatenate((a, b), axis=axis))
    # views as inputs
    if axis == 0:
        same(dpnp.concatenate([dpnp.array(a)[::2], dpnp.array(b)[::-1]], axis=0), np.concatenate([a[::2], b[::-1]], axis=0))
    if axis in (1, -1):
        same(dpnp.concatenate([dpnp.array(a.T).T, dpnp.array(b)], axis=1), np.concatenate([a, b], axis=1))


def test_concatenate_many_out_dtype_and_errors():
    parts = [np.arange(i * 3, dtype="i4").reshape(i, 3) for i in (1, 0, 4, 2)]
    dparts = [dpnp.array(p) for p in parts]
    same(dpnp.concatenate(dparts), np.concatenate(parts))
    same(dpnp.concat(dparts, axis=0), np.concatenate(parts))
    out = dpnp.empty((7, 3), dtype="f4")
    assert dpnp.concatenate(dparts, out=out) is out
    same(out, np.concatenate(parts).astype("f4"))
    same(dpnp.concatenate(dparts, dtype="f8"), np.concatenate(parts, dtype="f8"))
    with pytest.raises(TypeError):
        dpnp.concatenate(dparts, out=out, dtype="f4")
    with pytest.raises(TypeError):
        dpnp.concatenate(dparts, dtype="i1", casting="safe")
    with pytest.raises(ValueError):
        dpnp.concatenate([dpnp.ones((2, 3)), dpnp.ones((2, 4))], axis=0)
    with pytest.raises(ValueError):
        dpnp.concatenate([dpnp.ones((2, 3)), dpnp.ones(3)])
    with pytest.raises(ValueError):
        dpnp.concatenate([dpnp.array(1.0), dpnp.array(2.0)])
    with pytest.raises(TypeError):
        dpnp.concatenate([])
    with pytest.raises(np.exceptions.AxisError):
        dpnp.concatenate(dparts, axis=2)
    with pytest.raises(TypeError):
        dpt.concat([np.ones(3)])
    # a long 1-D join
    big = [np.arange(n, dtype="f4") for n in (1_000_003, 17, 65536)]
    same(dpnp.concatenate([dpnp.array(p) for p in big]), np.concatenate(big))


@pytest.mark.parametrize("axis", [0, 1, 2, -1, -3])
def test_stack_hstack_vstack(axis):
    rng = np.random.default_rng(2)
    arrs = [rng.integers(0, 9, (3, 4)).astype(dt) for dt in ("i2", "f4", "i4")]
    darrs = [dpnp.array(a) for a in arrs]
    same(dpnp.stack(darrs, axis=axis), np.stack(arrs, axis=axis))
    if axis == 0:
        same(dpnp.hstack(darrs), np.hstack(arrs))
        same(dpnp.vstack(darrs), np.vstack(arrs))
        v = [np.arange(3), np.arange(3, 6), np.arange(6, 9)]
        dv = [dpnp.array(x) for x in v]
        same(dpnp.hstack(dv), np.hstack(v))
        same(dpnp.vstack(dv), np.vstack(v))
        same(dpnp.stack(dv, axis=1, dtype="f4"), np.stack(v, axis=1, dtype="f4"))
        out = dpnp.empty((3, 3), dtype="i8")
        assert dpnp.stack(dv, out=out) is out
        same(out, np.stack(v))
        with pytest.raises(ValueError):
            dpnp.stack([dpnp.ones(3), dpnp.ones(4)])
        with pytest.raises(np.exceptions.AxisError):
            dpnp.stack(dv, axis=2)
        with pytest.raises(TypeError):
            dpnp.stack(dv, out=out, dtype="i8")


@pytest.mark.parametrize("dt", ["?", "i1", "u2", "i4", "i8", "f2", "f4", "f8", "c8"])
@pytest.mark.parametrize("n", [0, 1, 2, 3])
@pytest.mark.parametrize("axis", [0, 1, -1])
def test_diff(dt, n, axis):
    rng = np.random.default_rng(3)
    a = rng.integers(0, 50, (6, 9)).astype(dt)
    d = dpnp.array(a)
    same(dpnp.diff(d, n=n, axis=axis), np.diff(a, n=n, axis=axis))


def test_diff_prepend_append_and_errors():
    a = np.array([[1, 4, 9, 16], [2, 3, 5, 8]], dtype="i4")
    d = dpnp.array(a)
    pre = np.array([[0], [10]], dtype="i4")
    same(dpnp.diff(d, prepend=dpnp.array(pre)), np.diff(a, prepend=pre))
    same(dpnp.diff(d, append=dpnp.array(pre), n=2), np.diff(a, append=pre, n=2))
    # Python scalars are weakly typed (dpnp/tensor/_utility_functions.py:195-330, `_resolve_one_strong_two_weak_types`):
    # the result keeps the array's int32 where NumPy goes to int64
    same(dpnp.diff(d, prepend=0), np.diff(a, prepend=0).astype("i4"))
    same(dpnp.diff(d, axis=0, prepend=1, append=7), np.diff(a, axis=0, prepend=1, append=7).astype("i4"))
    same(dpnp.diff(dpnp.array(a.astype("f4")), append=0.5), np.diff(a.astype("f4"), append=np.float32(0.5)))
    with pytest.raises(ValueError):
        dpnp.diff(d, prepend=dpnp.ones((3, 1), dtype="i4"))
    same(dpnp.diff(d, n=10), np.diff(a, n=10))
    x = np.arange(1_000_003, dtype="f4") ** 2
    same(dpnp.diff(dpnp.array(x)), np.diff(x))
    with pytest.raises(ValueError):
        dpnp.diff(d, n=-1)
    with pytest.raises(np.exceptions.AxisError):
        dpnp.diff(d, axis=2)


@pytest.mark.parametrize("dt", ["i4", "f4", "f8"])
def test_trapezoid(dt):
    rng = np.random.default_rng(4)
    y = rng.integers(0, 20, (5, 33)).astype(dt)
    x1 = np.sort(rng.random(33)).astype("f8")
    x2 = np.sort(rng.random((5, 33)), axis=1).astype("f8")
    dy = dpnp.array(y)
    tol = dict(rtol=1e-6 if dt == "f4" else 1e-12)
    np.testing.assert_allclose(dpnp.trapezoid(dy).asnumpy(), np.trapezoid(y), **tol)
    np.testing.assert_allclose(dpnp.trapezoid(dy, dx=0.5, axis=0).asnumpy(), np.trapezoid(y, dx=0.5, axis=0), **tol)
    np.testing.assert_allclose(dpnp.trapezoid(dy, dpnp.array(x1)).asnumpy(), np.trapezoid(y, x1), **tol)
    np.testing.assert_allclose(dpnp.trapezoid(dy, dpnp.array(x2), axis=1).asnumpy(), np.trapezoid(y, x2, axis=1), **tol)
    with pytest.raises(TypeError):
        dpnp.trapezoid(y)
