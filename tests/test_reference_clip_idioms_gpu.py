"""clip through the tensor layer and the dpnp layer: parity with the oracle for every dtype and layout,
and the behaviours the reference's own tests pin (dpnp/tests/tensor/test_tensor_clip.py)."""
import numpy as np
import pytest

import dpnp_amd as dpnp
import dpnp_amd.tensor as dpt
from oracle import oracle as orc
from tests.helpers import ALL, assert_same, dev, host, random_array

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("dt", ALL, ids=str)
def test_clip_against_oracle_all_layouts(dt):
    rng = np.random.default_rng(31)
    for shape in [(1,), (1023,), (70001,), (37, 129), (5, 7, 33)]:
        x, lo, hi = (random_array(rng, shape, dt) for _ in range(3))
        if dt.kind == "f":
            x.ravel()[::17] = np.nan
            lo.ravel()[5::29] = np.nan
            hi.ravel()[7::31] = np.nan
        assert_same(host(dpt.clip(dev(x), dev(lo), dev(hi))), orc.clip(x, lo, hi))
        assert_same(host(dpt.clip(dev(x), dev(lo))), orc.binary("maximum", x, lo))
        assert_same(host(dpt.clip(dev(x), None, dev(hi))), orc.binary("minimum", x, hi))
    # broadcast bounds, transposed and strided operands
    x = random_array(rng, (64, 96), dt)
    lo_row, hi_col = random_array(rng, (96,), dt), random_array(rng, (64, 1), dt)
    assert_same(host(dpt.clip(dev(x), dev(lo_row), dev(hi_col))), orc.clip(x, lo_row, hi_col))
    xt = np.ascontiguousarray(x.T)
    assert_same(host(dpt.clip(dev(xt).mT, dev(lo_row), dev(hi_col))), orc.clip(x, lo_row, hi_col))
    assert_same(host(dpt.clip(dev(x)[::2, 1::3], dev(lo_row)[1::3], dev(hi_col)[::2])),
                orc.clip(x[::2, 1::3], lo_row[1::3], hi_col[::2]))


def test_clip_dtype_matrix():
    # test_tensor_clip.py:66-110: bounds must cast safely to the dtype of x, the result keeps it
    for d1 in ALL:
        for d2 in ALL:
            a, b, c = dpt.ones(127, dtype=d1), dpt.ones(127, dtype=d1), dpt.ones(127, dtype=d2)
            if np.can_cast(d2, d1, "safe"):
                for r in (dpt.clip(a, b, c), dpt.clip(a, min=c, max=None), dpt.clip(a, min=None, max=c)):
                    assert isinstance(r, dpt.usm_ndarray) and r.dtype == d1 and r.shape == a.shape
                    assert bool(dpt.all(r == a))
            else:
                for kw in (dict(min=b, max=c), dict(min=c, max=None), dict(min=None, max=c)):
                    with pytest.raises(ValueError):
                        dpt.clip(a, **kw)


def test_clip_python_scalars_and_weak_types():
    # test_tensor_clip.py:125-153, 646-699
    kinds = ["?", "i4", "f4", "c8"]
    zeros, ones = [False, 0, 0.0, 0j], [True, 1, 1.0, 1 + 0j]
    for ia, dt in enumerate(kinds):
        x = dpt.zeros(10, dtype=dt)
        for ib, (z, o) in enumerate(zip(zeros, ones)):
            if ia >= ib:
                for r in (dpt.clip(x, z, o), dpt.clip(x, z), dpt.clip(x, None, z)):
                    assert isinstance(r, dpt.usm_ndarray) and r.dtype == x.dtype
            else:
                for args in ((z, o), (z,), (None, o)):
                    with pytest.raises(ValueError):
                        dpt.clip(x, *args)
    x, m = dpt.zeros(10, dtype="i4"), dpt.ones(10, dtype="i4")
    for args in ((m, 2.5), (2.5, m), (2.5,)):
        with pytest.raises(ValueError):
            dpt.clip(x, *args)
    with pytest.raises(ValueError):
        dpt.clip(dpt.astype(x, "?"), 2)
    with pytest.raises(ValueError):
        dpt.clip(dpt.astype(x, "f4"), complex(2))
    # integer scalars beyond the range of the dtype do nothing (test_tensor_clip.py:787-792)
    u = dev(np.array([0, 255], "u1"))
    assert_same(host(dpt.clip(u, -300, 300)), np.array([0, 255], "u1"))
    assert_same(host(dpt.clip(u, 1, 300)), np.array([1, 255], "u1"))


def test_clip_special_values_and_order_of_bounds():
    # test_tensor_clip.py:178-187, 638-644
    x = dpt.arange(10, dtype="f4")
    assert_same(host(dpt.clip(x, -dpt.inf, dpt.inf)), np.arange(10, dtype="f4"))
    assert np.isnan(host(dpt.clip(x, dpt.nan, dpt.inf))).all()
    assert np.isnan(host(dpt.clip(x, -dpt.inf, dpt.nan))).all()
    assert (host(dpt.clip(dpt.ones(10, dtype="i4"), 5, 0)) == 0).all()
    r = dpt.clip(dpt.arange(10, dtype="i4"))
    assert_same(host(r), np.arange(10, dtype="i4"))
    xs = dpt.full(513, 5, dtype="i4")
    assert (host(dpt.clip(xs[1:], dpt.zeros(512, dtype="i4"), dpt.full(512, 2, dtype="i4"))) == 2).all()
    e = dpt.empty((0,), dtype="i4")
    assert dpt.clip(e, 1, 2).shape == (0,) and dpt.clip(e).shape == (0,) and dpt.clip(e, 1).shape == (0,)


def test_clip_out_in_place_and_overlapping():
    # test_tensor_clip.py:156-246
    x = dpt.arange(10, dtype="i4")
    a_min, a_max = dpt.arange(1, 11, dtype="i4"), dpt.arange(2, 12, dtype="i4")
    r = dpt.clip(x, a_min, a_max, out=x)
    assert r is x and (host(x) == host(a_min)).all()
    x = dpt.arange(10, dtype="i4")
    dpt.clip(x, min=a_min, max=None, out=x)
    assert (host(x) == host(a_min)).all()
    x = dpt.arange(10, dtype="i4")
    dpt.clip(x, a_min, a_max, out=a_max)
    assert (host(a_max) == host(a_min)).all()
    a_min = dpt.arange(1, 11, dtype="i4")
    dpt.clip(x, min=a_min, max=None, out=a_min[::-1])
    assert_same(host(a_min), (np.arange(10, dtype="i4") + 1)[::-1])
    for lo_dt, hi_dt in (("i4", "i4"), ("i4", "i2"), ("i2", "i4"), ("i2", "i1")):
        x = dpt.ones(10, dtype="i4")
        dpt.clip(x[:6], dpt.asarray(2, dtype=lo_dt), dpt.asarray(3, dtype=hi_dt), out=x[-6:])
        assert_same(host(x), np.array([1, 1, 1, 1, 2, 2, 2, 2, 2, 2], "i4"))
    x = dpt.arange(12, dtype="i4")
    dpt.clip(x[:6], out=x[-6:])
    assert_same(host(x), np.tile(np.arange(6, dtype="i4"), 2))
    x = dpt.ones(10, dtype="i4")
    assert dpt.clip(x, out=x) is x and (host(x) == 1).all()
    for hi_dt in ("i4", "i2"):
        x, a_min = dpt.full(6, 3, dtype="i4"), dpt.full(10, 2, dtype="i4")
        dpt.clip(x, min=a_min[:6], max=dpt.asarray(4, dtype=hi_dt), out=a_min[-6:])
        assert_same(host(a_min), np.array([2, 2, 2, 2, 3, 3, 3, 3, 3, 3], "i4"))
    x, a_min = dpt.full(6, 3, dtype="i4"), dpt.full(10, 2, dtype="i4")
    dpt.clip(x, min=a_min[:6], max=None, out=a_min[-6:])
    assert_same(host(a_min), np.array([2, 2, 2, 2, 3, 3, 3, 3, 3, 3], "i4"))


def test_clip_argument_validation():
    # test_tensor_clip.py:249-272, 415-440, 583-594, 720-740, 768-784
    bad = {}
    x1, x2 = dpt.empty((1,), dtype="i4"), dpt.empty((1,), dtype="i4")
    with pytest.raises(TypeError):
        dpt.clip(bad, x1, x2)
    with pytest.raises(ValueError):
        dpt.clip(x1, bad, x2)
    with pytest.raises(ValueError):
        dpt.clip(x1, bad)
    for args in ((x1, x1, x2), (x1, x2), (x1,)):
        with pytest.raises(TypeError):
            dpt.clip(*args, out=bad)
    a = dpt.ones(1, dtype="i4")
    with pytest.raises(ValueError, match="Output array of type.*is needed"):
        dpt.clip(a, a, a, dpt.empty_like(a, dtype="f4"))
    with pytest.raises(ValueError, match="Output array of type.*is needed"):
        dpt.clip(a, a, None, dpt.empty_like(a, dtype="f4"))
    with pytest.raises(ValueError, match="Output array of type.*is needed"):
        dpt.clip(a, out=dpt.empty_like(a, dtype="f4"))
    x = dpt.ones((4, 5), dtype="i4")
    with pytest.raises(ValueError):
        dpt.clip(x, dpt.ones((3,), dtype="i4"), 2)
    with pytest.raises(ValueError):
        dpt.clip(x, 0, 2, out=dpt.empty((5, 4), dtype="i4"))
    with pytest.raises(ValueError):
        dpt.clip(x, 0, out=dpt.empty((5, 4), dtype="i4"))
    ro = dpt.empty((4, 5), dtype="i4")
    ro.flags["W"] = False
    for args in ((0, 2), (0,), ()):
        with pytest.raises(ValueError):
            dpt.clip(x, *args, out=ro)


@pytest.mark.parametrize("dts", [("i4", "i4"), ("i4", "i2"), ("i2", "i4"), ("i1", "i2")])
def test_clip_result_layout(dts):
    # test_tensor_clip.py:275-381
    d1, d2 = dts
    n = 20
    for order_in, flag in (("C", "c_contiguous"), ("F", "f_contiguous")):
        a, b, c = (dpt.ones((n, n), dtype=d, order=order_in) for d in ("i4", d1, d2))
        assert dpt.clip(a, b, c, order="C").flags.c_contiguous
        assert dpt.clip(a, b, c, order="F").flags.f_contiguous
        assert getattr(dpt.clip(a, b, c, order="A").flags, flag)
        assert getattr(dpt.clip(a, b, c, order="K").flags, flag)
        assert getattr(dpt.clip(a, min=None, max=c, order="K").flags, flag)
        assert dpt.clip(a, min=None, max=c, order="F").flags.f_contiguous
    a, b, c = (dpt.ones((2 * n, 2 * n), dtype=d)[:n, ::-2] for d in ("i4", d1, d2))
    assert dpt.clip(a, b, c, order="K").strides == (n, -1)
    assert dpt.clip(a, b, c, order="C").strides == (n, 1)
    assert dpt.clip(a, None, c, order="K").strides == (n, -1)
    assert dpt.clip(a.mT, b.mT, c.mT, order="K").strides == (-1, n)
    assert dpt.clip(a.mT, b.mT, c.mT, order="C").strides == (n, 1)


def test_dpnp_clip_function_and_method():
    # dpnp/tests/test_mathematical.py (TestClip)
    a = np.arange(10)
    x = dpnp.asarray(a)
    assert_same(dpnp.clip(x, 1, 8).asnumpy(), np.clip(a, 1, 8))
    assert_same(dpnp.clip(x, 8, 1).asnumpy(), np.clip(a, 8, 1))
    assert_same(dpnp.clip(x, 3, None).asnumpy(), np.clip(a, 3, None))
    assert_same(dpnp.clip(x, max=6).asnumpy(), np.clip(a, None, 6))
    lo = np.array([3, 4, 1, 1, 1, 4, 4, 4, 4, 4])
    assert_same(dpnp.clip(x, dpnp.asarray(lo), 8).asnumpy(), np.clip(a, lo, 8))
    assert_same(x.clip(2, 5).asnumpy(), a.clip(2, 5))
    o = dpnp.empty(10, dtype=a.dtype)
    r = dpnp.clip(x, 3, 6, out=o)
    assert r is o
    assert_same(o.asnumpy(), np.clip(a, 3, 6))
    f = np.linspace(-2, 2, 101, dtype="f4")
    assert_same(dpnp.clip(dpnp.asarray(f), -0.5, 0.75).asnumpy(), np.clip(f, np.float32(-0.5), np.float32(0.75)))
    with pytest.raises(NotImplementedError):
        dpnp.clip(x, 1, 2, where=False)
