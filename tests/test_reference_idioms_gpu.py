"""Behaviours the reference's own elementwise tests exercise (dpnp/tests/tensor/elementwise/
test_add.py, test_bitwise_and.py, test_exp.py, test_sqrt.py, test_greater.py), restated for
this package's surface."""
import ctypes

import numpy as np
import pytest

import dpnp_amd.tensor as dpt
from tests.helpers import ALL, assert_same, dev, host

pytestmark = pytest.mark.gpu


def test_add_order():
    # test_add.py:90-134
    n = 20
    for dt1, dt2 in zip(["i4", "i4", "f4"], ["i4", "f4", "i4"]):
        a1, a2 = dpt.ones((n, n), dtype=dt1, order="C"), dpt.ones((n, n), dtype=dt2, order="C")
        assert dpt.add(a1, a2, order="C").flags.c_contiguous
        assert dpt.add(a1, a2, order="F").flags.f_contiguous
        assert dpt.add(a1, a2, order="A").flags.c_contiguous
        assert dpt.add(a1, a2, order="K").flags.c_contiguous
        a1, a2 = dpt.ones((n, n), dtype=dt1, order="F"), dpt.ones((n, n), dtype=dt2, order="F")
        assert dpt.add(a1, a2, order="C").flags.c_contiguous
        assert dpt.add(a1, a2, order="F").flags.f_contiguous
        assert dpt.add(a1, a2, order="A").flags.f_contiguous
        assert dpt.add(a1, a2, order="K").flags.f_contiguous
        a1 = dpt.ones((2 * n, 2 * n), dtype=dt1)[:n, ::-2]
        a2 = dpt.ones((2 * n, 2 * n), dtype=dt2)[:n, ::-2]
        assert dpt.add(a1, a2, order="K").strides == (n, -1)
        assert dpt.add(a1, a2, order="C").strides == (n, 1)
        assert dpt.add(a1.mT, a2.mT, order="K").strides == (-1, n)
        assert dpt.add(a1.mT, a2.mT, order="C").strides == (n, 1)
        assert (host(dpt.add(a1.mT, a2.mT)) == 2).all()


def test_add_broadcasting():
    # test_add.py:137-195
    m, v = dpt.ones((100, 5), dtype="i4"), dpt.arange(5, dtype="i4")
    want = np.arange(1, 6, dtype="i4")[np.newaxis, :]
    assert (host(dpt.add(m, v)) == want).all() and (host(dpt.add(v, m)) == want).all()
    r3 = dpt.empty_like(m)
    dpt.add(m, v, out=r3)
    assert (host(r3) == want).all()
    r4 = dpt.empty_like(m)
    dpt.add(v, m, out=r4)
    assert (host(r4) == want).all()
    a1, a2 = dpt.ones((6, 1), dtype="i4"), dpt.arange(6, dtype="i4")
    want = np.arange(1, 7, dtype="i4")[np.newaxis, :]
    assert (host(dpt.add(a1, a2)) == want).all() and (host(dpt.add(a2, a1)) == want).all()
    assert (host(dpt.add(a1[::2], a2[::2])) == want[:, ::2]).all()
    with pytest.raises(ValueError):
        dpt.add(a1, a2, out=dpt.empty_like(a1))
    a3, a4 = dpt.ones((6, 1), dtype="i4"), dpt.ones((1, 6), dtype="i4")
    assert (host(dpt.add(a3, a4)) == np.full((6, 6), 2)).all()
    assert (host(dpt.add(a3[::2], a4[:, ::2])) == np.full((3, 3), 2)).all()
    assert (host(dpt.add(a3[::2], a4)) == np.full((3, 6), 2)).all()
    with pytest.raises(ValueError):
        dpt.add(dpt.ones((10, 10), dtype="i4"), dpt.ones((3,), dtype="i4"))


@pytest.mark.parametrize("dt", ALL, ids=str)
def test_python_scalars_of_every_kind(dt):
    # test_add.py:198-214,309-330
    x = dpt.zeros((10, 10), dtype=dt)
    for sc in (bool(0), int(0), float(0), complex(0), np.float32(0), ctypes.c_int(0)):
        assert isinstance(dpt.add(x, sc), dpt.usm_ndarray)
        assert isinstance(dpt.add(sc, x), dpt.usm_ndarray)
    k = x.dtype.kind
    x += {"b": bool(0), "i": int(0), "u": int(0), "f": float(0), "c": complex(0)}[k]
    assert (host(x) == 0).all()


def test_types_property_and_errors():
    # test_add.py:244-306
    assert isinstance(dpt.add.types, list) and len(dpt.add.types) > 0 and dpt.add.types == dpt.add.types_
    a1, a2 = dpt.ones(2, dtype="f4"), dpt.ones(2, dtype="i4")
    with pytest.raises(ValueError, match="The shape of input and output arrays are inconsistent"):
        dpt.add(a1, a2, out=dpt.empty(3))
    with pytest.raises(dpt.ExecutionPlacementError, match="Execution placement can not be unambiguously inferred"):
        dpt.add(np.ones(2, dtype="f4"), np.ones(2, dtype="i4"))
    with pytest.raises(TypeError, match="output array must be of usm_ndarray type"):
        dpt.add(a1, a2, out=np.empty(2, dtype="f4"))
    with pytest.raises(ValueError, match="Output array of type.*is needed"):
        dpt.add(dpt.ones(5, dtype="f4"), dpt.ones(5, dtype="f4"), out=dpt.zeros(5, dtype="i1"))


def test_inplace_dtype_matrix():
    # test_add.py (in-place dtype matrix): x += y works iff y casts to x's dtype "same_kind"
    for d1 in ALL:
        for d2 in ALL:
            x, y = dpt.zeros(17, dtype=d1), dpt.ones(17, dtype=d2)
            if np.can_cast(d2, d1, casting="same_kind"):
                x += y
                assert x.dtype == d1 and (host(x) == 1).all()
                x2 = dpt.zeros(34, dtype=d1)[::2]
                x2 += y
                assert (host(x2) == 1).all()
            else:
                with pytest.raises(ValueError):
                    x += y


def test_inplace_broadcasting_and_overlap():
    m, v = dpt.ones((100, 5), dtype="i4"), dpt.arange(5, dtype="i4")
    m += v
    assert (host(m) == np.arange(1, 6, dtype="i4")[np.newaxis, :]).all()
    with pytest.raises(ValueError):
        v += m  # left-hand side cannot grow
    x = dpt.ones(10, dtype="i4")
    dpt.add(x, 1, out=x)
    assert (host(x) == 2).all()
    dpt.add(1, x, out=x)  # out is the second operand
    assert (host(x) == 3).all()
    y = dev(np.arange(10, dtype="i4"))
    y[1:] += y[:-1]  # overlapping operand is buffered first
    assert_same(host(y), np.concatenate([[0], np.arange(1, 10) + np.arange(0, 9)]).astype("i4"))


def test_bitwise_and_bool_and_ints():
    # test_bitwise_and.py:43-94
    rng = np.random.default_rng(5)
    for dt in [d for d in ALL if d.kind in "biu"]:
        lo, hi = (0, 2) if dt.kind == "b" else (np.iinfo(dt).min, np.iinfo(dt).max)
        a = rng.integers(lo, hi, 1000, dtype=np.int64 if dt.kind != "u" or dt.itemsize < 8 else np.uint64).astype(dt)
        b = rng.integers(lo, hi, 1000, dtype=np.int64 if dt.kind != "u" or dt.itemsize < 8 else np.uint64).astype(dt)
        r = dpt.bitwise_and(dev(a), dev(b))
        assert r.dtype == dt
        assert_same(host(r), np.bitwise_and(a, b))
        assert_same(host(dpt.bitwise_and(dev(a)[::-1], dev(b)[::-1])), np.bitwise_and(a[::-1], b[::-1]))
    with pytest.raises(ValueError):
        dpt.bitwise_and(dpt.ones(3, dtype="f4"), dpt.ones(3, dtype="f4"))


def test_sqrt_and_log_special_cases():
    # test_sqrt.py:94-129, test_log.py:88
    x = np.array([np.nan, np.inf, -np.inf, 0.0, -0.0, -1.0, 4.0], dtype="f4")
    with np.errstate(all="ignore"):
        for f, g in ((dpt.sqrt, np.sqrt), (dpt.log, np.log), (dpt.exp, np.exp)):
            got, want = host(f(dev(x))), g(x)
            special = ~np.isfinite(want) | (want == 0) | (want == 1)
            np.testing.assert_array_equal(got[special], want[special])
            np.testing.assert_allclose(got[~special], want[~special], rtol=4 * np.finfo("f4").eps)
            np.testing.assert_array_equal(np.signbit(got[~np.isnan(got)]), np.signbit(want[~np.isnan(want)]))
    assert dpt.sqrt(dpt.ones(3, dtype="i4")).dtype == np.dtype("f8")
    assert dpt.sqrt(dpt.ones(3, dtype="u1")).dtype == np.dtype("f2")


def test_comparison_of_mixed_signedness():
    # test_greater.py / test_less.py: int64 vs uint64 compare exactly
    a = dev(np.array([-1, 0, 2**62], dtype="i8"))
    b = dev(np.array([2**64 - 1, 0, 2**62], dtype="u8"))
    assert_same(host(dpt.less(a, b)), np.array([True, False, False]))
    assert_same(host(dpt.greater(b, a)), np.array([True, False, False]))
    assert_same(host(dpt.equal(a, b)), np.array([False, True, True]))
    u = dev(np.array([200, 5], dtype="u1"))
    assert_same(host(dpt.greater(u, -1)), np.array([True, True]))
    assert_same(host(dpt.less(u, 1000)), np.array([True, True]))
