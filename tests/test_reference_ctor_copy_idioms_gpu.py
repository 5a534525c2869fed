"""Construction, conversion, copy and assignment behaviours that the reference's own tests pin
(dpnp/tests/tensor/test_usm_ndarray_utility_functions.py, test_tensor_copy_utils.py,
test_tensor_asarray.py, test_usm_ndarray_ctor.py), restated against this library's arrays."""
import ctypes
from random import randrange

import numpy as np
import pytest

import dpnp_amd.tensor as dpt
import dpnp_amd.tensor._copy_utils as cu
from tests.helpers import ALL, assert_same, host

pytestmark = pytest.mark.gpu


# ---- all / any: test_usm_ndarray_utility_functions.py:61-204 ------------------------------------
@pytest.mark.parametrize("func,identity", [(dpt.all, True), (dpt.any, False)])
@pytest.mark.parametrize("dt", ALL, ids=str)
def test_boolean_reduction_every_dtype(func, identity, dt):
    for n in (10, 4 * 32 + 1):
        x = dpt.full(n, identity, dtype=dt)
        assert bool(host(func(x))) is identity
        x[randrange(n)] = not identity
        assert bool(host(func(x))) is (not identity)
    x = dpt.full(20, identity, dtype=dt)[::-2]
    assert bool(host(func(x))) is identity
    x[randrange(x.size)] = not identity
    assert bool(host(func(x))) is (not identity)


@pytest.mark.parametrize("func,identity", [(dpt.all, True), (dpt.any, False)])
def test_boolean_reduction_axes_keepdims_empty(func, identity):
    x = dpt.full((2, 3, 4, 5, 6), identity, dtype="i4")
    r = func(x, axis=(1, 2, -1))
    assert r.shape == (2, 5) and (host(r) == identity).all()
    x[0, 0, 0, ...] = not identity
    r = func(x, axis=(1, 2, -1))
    assert (host(r[0]) == (not identity)).all()
    o = dpt.ones((2, 3, 4, 5, 6), dtype="i4")
    r = func(o, axis=(1, 2, -1), keepdims=True)
    assert r.shape == (2, 1, 1, 5, 1) and host(r).all()
    assert func(o, axis=None, keepdims=True).shape == (1,) * 5
    assert bool(host(func(dpt.empty((0,), dtype="i4")))) is identity
    nan_inf = dpt.asarray([dpt.nan, dpt.inf, -dpt.inf], dtype="f4")[:, dpt.newaxis]
    assert_same(host(func(nan_inf, axis=1)), np.array([True, True, True]))
    assert bool(host(func(dpt.ones((), dtype="i4")))) and not bool(host(func(dpt.zeros((), dtype="i4"))))
    v = dpt.ones((5,), dtype="i4")
    assert_same(host(func(v, axis=())), np.ones(5, dtype=bool))
    with pytest.raises(TypeError):
        func({})
    with pytest.raises(np.exceptions.AxisError):
        func(dpt.ones((4, 5), dtype="i4"), axis=-3)


def test_boolean_reductions_3d():
    x = dpt.reshape(dpt.arange(-10, 14, 1, dtype="i4"), (2, 3, 4))
    want = np.full((3, 4), True)
    want[2, 2] = False
    assert_same(host(dpt.all(x, axis=0)), want)
    assert host(dpt.any(dpt.ones((2, 3, 4, 5), dtype="i4"), axis=0)).all()


# ---- order-K helpers: test_tensor_copy_utils.py:38-120 --------------------------------------------
def test_order_k_allocation_helpers():
    a = dpt.empty((10, 10), dtype="i4", order="F")
    assert cu._empty_like_orderK(a, dpt.int32).flags["F"]
    with pytest.raises(TypeError):
        cu._empty_like_orderK([1, 2, 3], dpt.int32)
    with pytest.raises(TypeError):
        cu._empty_like_pair_orderK([1, 2, 3], (1, 2, 3), dpt.int32, (3,))
    with pytest.raises(TypeError):
        cu._empty_like_pair_orderK(dpt.empty(10, dtype="i4"), (1, 2, 3), dpt.int32, (10,))
    a = np.ones((2, 3, 4), dtype="i4")
    for perm in ((1, 0, 2), (2, 0, 1), (0, 2, 1)):
        v = np.transpose(a, perm)
        d = dpt.asarray(v, order="K")
        assert d.shape == v.shape and d.strides == tuple(s // 4 for s in v.strides)
        assert_same(host(d), v)


# ---- asarray: test_tensor_asarray.py:81-470 ---------------------------------------------------------
def test_asarray_sources():
    x = np.arange(10)
    y = dpt.asarray(x)
    assert type(y) is dpt.usm_ndarray and y.shape == x.shape and y.dtype == x.dtype
    xf = np.array([[1, 2, 3], [4, 5, 6]], dtype="f4", order="F")
    assert_same(host(dpt.asarray(xf)), xf)
    xs = np.array([[1, 2, 3], [4, 5, 6]], dtype="i8")[::-1, ::-1]
    assert_same(host(dpt.asarray(xs)), xs)
    assert type(dpt.asarray([1, 2, 3])) is dpt.usm_ndarray
    y = dpt.asarray([(1, 1), (2.0, 2.0 + 1.0j), range(4, 6), np.array([3, 4], dtype="c16")])
    assert y.ndim == 2 and y.shape == (4, 2) and y.dtype == np.complex128
    assert dpt.asarray([]).shape == (0,) and dpt.asarray([[], []]).shape == (2, 0)
    assert dpt.asarray([True, False]).dtype.kind == "b"
    assert dpt.asarray(5).dtype == np.dtype(int) and dpt.asarray(5.2).dtype == np.dtype(float)
    assert dpt.asarray(np.float32(2.3)).dtype == np.float32 and dpt.asarray(1.0j).dtype == np.dtype(complex)
    assert dpt.asarray(ctypes.c_int(8)).dtype == np.dtype(ctypes.c_int)
    assert dpt.asarray(9223372036854775807, dtype="u8").dtype == np.uint64
    assert int(dpt.asarray(9223372036854775808, dtype="u8")) == 9223372036854775808
    r = dpt.arange(10)
    m = dpt.asarray([r] * 4)
    assert m.shape == (4, 10) and m.dtype == r.dtype
    assert_same(host(m), np.tile(np.arange(10), (4, 1)))
    ar = dpt.asarray([dpt.ones((2, 4), dtype="i4"), [dpt.zeros(4), dpt.full(4, -1)]])
    assert ar.shape == (2, 2, 4)
    assert_same(host(ar)[1], np.array([[0, 0, 0, 0], [-1, -1, -1, -1]], dtype=host(ar).dtype))


def test_asarray_argument_validation():
    with pytest.raises(TypeError):
        dpt.asarray([1], copy="invalid")
    with pytest.raises(TypeError):
        dpt.asarray([1], order=1)
    with pytest.raises(TypeError):
        dpt.asarray([1], dtype="invalid")
    with pytest.raises(ValueError):
        dpt.asarray([1], order="Z")
    with pytest.raises(ValueError):
        dpt.asarray([[1], 2])
    with pytest.raises(OverflowError):
        dpt.asarray(-9223372036854775809, dtype="i4")
    for src in (memoryview(np.arange(5)), np.arange(5), [1, 2, 3], 5):
        with pytest.raises(ValueError):
            dpt.asarray(src, copy=False)
    with pytest.raises(TypeError):
        dpt.asarray(np.array([1, 2, 3], dtype=object))


def test_asarray_copy_false_and_order():
    xnp = np.random.default_rng(1).integers(-255, 255, size=(10, 4))
    x = dpt.from_numpy(xnp)
    assert dpt.asarray(x, copy=False, order="K") is x
    assert dpt.asarray(x, copy=True, order="K") is not x
    assert dpt.asarray(x, copy=False, order="C") is x and dpt.asarray(x, copy=False, order="A") is x
    with pytest.raises(ValueError):
        dpt.asarray(x, copy=False, order="F")
    xf = dpt.empty(x.shape, dtype=x.dtype, order="F")
    xf[:] = x
    for order in "KFA":
        assert dpt.asarray(xf, copy=False, order=order) is xf
    with pytest.raises(ValueError):
        dpt.asarray(xf, copy=False, order="C")
    a = dpt.empty((2, 3, 4), dtype="u1")
    b = dpt.permute_dims(a, (2, 0, 1))
    c = dpt.asarray(b, copy=True, order="K")
    assert c.shape == b.shape and c.strides == b.strides and c._element_offset == 0 and c._pointer != b._pointer


def _typesafe_arange(n, dt):
    dt = np.dtype(dt)
    if dt.kind in "ui":
        ii = np.iinfo(dt)
        m0 = max(ii.min, -(n // 2))
        m1 = min(m0 + n, ii.max)
        base = np.arange(m0, m1, dtype=dt)
        return dpt.asarray(np.resize(base, n))
    if dt.kind == "b":
        return dpt.asarray(np.resize(np.array([False, True]), n))
    return dpt.asarray(np.linspace(-(n // 2), -(n // 2) + n, num=n).astype(dt))


@pytest.mark.parametrize("dt", ALL, ids=str)
def test_contiguous_copies_of_permuted_arrays(dt):
    # test_tensor_asarray.py:470-610 (copy_as_contiguous kernels)
    n0, n1, n2 = 6, 35, 37
    flat = _typesafe_arange(n0 * n1 * n2, dt)
    hflat = host(flat)
    x = dpt.reshape(flat, (n0, n1, n2)).mT
    hx = np.swapaxes(hflat.reshape(n0, n1, n2), -1, -2)
    for view, hview in ((x, hx), (x[0], hx[0]), (dpt.flip(x, axis=1), np.flip(hx, axis=1))):
        y = dpt.asarray(view, order="C")
        assert y.flags.c_contiguous
        assert_same(host(y), hview)
    x4 = dpt.reshape(flat, (2, 3, n1, n2)).mT[:, :2]
    assert_same(host(dpt.asarray(x4, order="C")), np.swapaxes(hflat.reshape(2, 3, n1, n2), -1, -2)[:, :2])
    x6 = dpt.reshape(flat, (n0, n1, n2), order="F")
    assert_same(host(dpt.asarray(x6, order="C")), hflat.reshape((n0, n1, n2), order="F"))
    x = dpt.reshape(flat, (n0, n1, n2))
    hx = hflat.reshape(n0, n1, n2)
    for view, hview in ((x, hx), (x[0], hx[0]), (dpt.flip(x, axis=1), np.flip(hx, axis=1))):
        y = dpt.asarray(view, order="F")
        assert y.flags.f_contiguous
        assert_same(host(y), hview)
    m0, m1 = 4, 53
    sq = dpt.reshape(_typesafe_arange(m0 * m1 * m1, dt), (m0, m1, m1))
    hsq = host(sq)
    assert_same(host(dpt.asarray(sq.mT, order="C")), np.swapaxes(hsq, -1, -2))
    assert_same(host(dpt.asarray(dpt.flip(sq.mT, axis=1), order="C")), np.flip(np.swapaxes(hsq, -1, -2), axis=1))
    assert_same(host(dpt.asarray(sq, order="F")), hsq)


# ---- astype / copy: test_usm_ndarray_ctor.py:967-1072 ----------------------------------------------
def test_astype_and_copy():
    x = dpt.empty((5, 5), dtype="i4")
    x[:] = np.full((5, 5), 7, dtype="i4")
    assert_same(host(dpt.astype(x, "c8", order="C")), np.full((5, 5), 7, dtype="c8"))
    for dt in ("f2", "f4"):
        y = dpt.astype(x[::2, ::-1], dt, order="K")
        assert_same(host(y), np.full(y.shape, 7, dtype=dt))
    y = dpt.astype(x[::2, ::-1], "i4", order="K", copy=False)
    assert y.usm_data is x.usm_data
    assert dpt.astype(x, None, order="K").dtype == np.float64
    with pytest.raises(ValueError):
        dpt.astype(x, "i4", order="WRONG")
    o = dpt.ones(64)
    assert dpt.astype(o, o.dtype, copy=False, order="C") is o and dpt.astype(o, o.dtype, copy=False, order="F") is o
    b = dpt.asarray(np.asarray([0, 3, 1, 2, 0, 1], dtype="u1").view("?"))  # truth values that are not 0 / 1
    assert_same(host(dpt.astype(b, dpt.uint8)), np.array([0, 1, 1, 1, 0, 1], dtype="u1"))
    assert_same(host(dpt.astype(dpt.asarray([160.0, 120.0], dtype="f4"), dpt.uint8)), np.array([160, 120], dtype="u1"))
    assert (host(dpt.astype(dpt.ones(513, dtype="i4")[1:], "f4")) == 1).all()
    v = dpt.usm_ndarray((5, 5), "i4")[2:4, 1:4]
    v[:] = 42
    copies = {o: dpt.copy(v, order=o) for o in "CFAK"}
    assert all(c.usm_data is not v.usm_data for c in copies.values())
    assert copies["C"].strides == (3, 1) and copies["F"].strides == (1, 2)
    assert copies["A"].strides == (3, 1) and copies["K"].strides == (3, 1)
    for c in copies.values():
        assert_same(host(c), np.full((2, 3), 42, dtype="i4"))


# ---- assignment: test_usm_ndarray_ctor.py:649-810 ---------------------------------------------------
@pytest.mark.parametrize("dt", ALL, ids=str)
def test_setitem_same_dtype_views(dt):
    shape = (2, 4, 3)
    xnp = np.random.default_rng(3).integers(-10, 10, size=24).astype(dt).reshape(shape)
    x = dpt.from_numpy(xnp)
    z = dpt.zeros(shape, dtype=dt)
    z0 = dpt.copy(z[0, 0, 0])
    z0[Ellipsis] = x[-1, -1, -1]
    assert_same(host(z0), xnp[-1, -1, -1])
    z1 = dpt.copy(z[0, 1:3, 0])
    z1[Ellipsis] = x[-1, 0:2, -1]
    assert_same(host(z1), xnp[-1, 0:2, -1])
    z2 = dpt.copy(z[:, 1:3, 0])[::-1]
    z2[:] = x[:, 1:4, -1][:, 0:2]
    assert_same(host(z2), xnp[:, 1:3, -1])
    z3 = dpt.copy(z)
    z3[:] = x
    assert_same(host(z3), xnp)
    z3[::-1] = x[::-1]
    assert_same(host(z3), xnp)
    z3[:] = x[0]
    assert_same(host(z3), np.broadcast_to(xnp[0], shape))
    z1[0:0][Ellipsis] = z3[0, 0, 0:0]


def test_setitem_broadcasting_scalars_and_errors():
    dst = dpt.ones((2, 3, 4), dtype="u4")
    dst[...] = dpt.zeros((3, 1), dtype="u4")
    assert (host(dst) == 0).all()
    x = dpt.asarray([[1, 2, 3], [6, 7, 8]], dtype="i4")
    x[0] = dpt.asarray([4, 5], dtype="i4")[1]
    assert_same(host(x), np.array([[5, 5, 5], [6, 7, 8]], dtype="i4"))
    with pytest.raises(ValueError):
        dpt.ones((2, 0, 5, 4), dtype="i8")[...] = dpt.ones((2, 0, 3, 4), dtype="i8")
    dpt.ones(1, dtype="i8")[0:0][...] = dpt.ones((), dtype="i8")
    for src_shape in ((2, 1, 4), (1, 2, 1, 4)):
        dst = dpt.ones((2, 3, 4), dtype="i4")
        dst[...] = dpt.zeros(src_shape, dtype="i4")
        assert (host(dst) == 0).all()
    for dt in ALL:
        a = dpt.usm_ndarray((6, 6), dtype=dt)
        for i in range(a.size):
            a[np.unravel_index(i, a.shape)] = np.asarray(i, dtype=dt)
        assert_same(host(a), np.arange(36).astype(dt).reshape(6, 6))
        b = dpt.usm_ndarray((2, 3), dtype=dt)
        for i in range(b.size):
            b[np.unravel_index(i, b.shape)] = i
        assert_same(host(b), np.arange(6).astype(dt).reshape(2, 3))
    xx, yy = dpt.empty((4,), dtype="u1"), dpt.empty((4, 2), dtype="u1")
    with pytest.raises(ValueError):
        xx[:] = yy
    with pytest.raises(ValueError):
        xx[:] = yy[:, 0:1]
    xx[:] = yy[None, :, 0]
    for src_dt, dst_dt in (("i4", "i8"), ("f4", "f8")):
        z = dpt.empty((20,), dtype=dst_dt)
        z[::2] = dpt.ones(10, dtype=src_dt)
        z[1::2] = dpt.zeros(10, dtype=src_dt)
        assert_same(host(z), np.tile(np.array([1, 0], dst_dt), 10))
    d = dpt.empty(4, dtype="int32")
    d[:] = np.arange(4, dtype="intc")
    assert_same(host(d), np.arange(4, dtype="i4"))


# ---- zeros / ones / full / arange / linspace / *_like: test_usm_ndarray_ctor.py:1278-1720, 2100-2215 ----
@pytest.mark.parametrize("dt", ALL, ids=str)
def test_filled_constructors_every_dtype(dt):
    assert_same(host(dpt.zeros(10, dtype=dt)), np.zeros(10, dtype=dt))
    assert_same(host(dpt.ones(10, dtype=dt)), np.ones(10, dtype=dt))
    assert_same(host(dpt.full(10, 4, dtype=dt)), np.full(10, 4, dtype=dt))
    np.testing.assert_allclose(host(dpt.linspace(0, 1, num=2, dtype=dt)), np.linspace(0, 1, num=2, dtype=dt))
    for shape in ((4, 5), ()):
        x = dpt.empty(shape, dtype=dt)
        e = dpt.empty_like(x)
        assert e.shape == x.shape and e.dtype == x.dtype
        assert_same(host(dpt.zeros_like(x)), np.zeros(shape, dtype=dt))
        assert_same(host(dpt.ones_like(x)), np.ones(shape, dtype=dt))
        assert_same(host(dpt.full_like(x, np.dtype(dt).type(1))), np.ones(shape, dtype=dt))
    if dt != np.dtype("?"):
        x = dpt.arange(0, 123, dtype=dt)
        assert complex(x[47]) == 47
        assert dpt.arange(128, dtype=dt).shape == (128,) and dpt.arange(127, 0, -1, dtype=dt).shape == (127,)


def test_full_inference_special_values_and_array_fill():
    for v in (1 + 1j, 0 + 1j, 0 + 0j):
        assert_same(host(dpt.full((), fill_value=v, dtype="c16")), np.full((), v, dtype="c16"))
    assert np.issubdtype(dpt.full(10, 4).dtype, np.integer)
    assert dpt.full(10, True).dtype == np.dtype(bool)
    assert np.issubdtype(dpt.full(10, 12.3).dtype, np.floating)
    assert np.issubdtype(dpt.full(10, 0.3 - 2j).dtype, np.complexfloating)
    assert np.issubdtype(dpt.full(10, 12.3, dtype=int).dtype, np.integer)
    assert np.issubdtype(dpt.full(10, 0.3 - 2j, dtype=int).dtype, np.integer)
    assert np.issubdtype(dpt.full(10, 0.3 - 2j, dtype="f8").dtype, np.floating)
    for dt in ("f2", "f4", "f8"):
        assert bool(dpt.isnan(dpt.full(10, fill_value=dpt.nan, dtype=dt)[0]))
        hi, lo = dpt.full(10, fill_value=dpt.inf, dtype=dt)[0], dpt.full(10, fill_value=-dpt.inf, dtype=dt)[0]
        assert bool(dpt.isinf(hi)) and bool(dpt.greater(hi, 0)) and bool(dpt.isinf(lo)) and bool(dpt.less(lo, 0))
        ar = dpt.full(10, fill_value=dpt.pi, dtype=dt)
        assert abs(float(ar[0]) - dpt.pi) < 16 * dpt.finfo(ar.dtype).eps
    xnp = np.array([1, 2, 3], dtype="i4")
    y = dpt.full((3, 3), dpt.asarray(xnp))
    assert y.dtype == np.int32
    assert_same(host(y), np.full((3, 3), xnp))
    x = dpt.arange(10, dtype="i4")
    y = dpt.full(10, x[3])
    assert y.dtype == x.dtype
    assert_same(host(y), np.full(10, 3, dtype="i4"))
    assert_same(host(dpt.full(10, x[3], dtype="f4")), np.full(10, 3, dtype="f4"))
    for o1 in "FC":
        for o2 in "FC":
            src = np.array([1, 2, 3], order=o1)
            want = np.full((3, 3), src, order=o2)
            got = dpt.full((3, 3), src, order=o2)
            assert got.flags.c_contiguous == want.flags.c_contiguous and got.flags.f_contiguous == want.flags.f_contiguous
            assert_same(host(got), want)
    for fill in (dpt.arange(3, dtype="i4"), dpt.arange(6, dtype="i4")[::2]):
        got = dpt.full((3, 3), fill)
        assert got.strides == (3, 1)
        assert_same(host(got), np.full((3, 3), host(fill)))
    for dt in ("i1", "u1", "i2", "u2", "i4", "u4", "i8", "u8"):
        with pytest.raises(OverflowError):
            dpt.full(1, int(np.iinfo(dt).max) + 1, dtype=dt)
    with pytest.raises(TypeError):
        dpt.empty(1, dtype=np.object_)


def test_arange_and_linspace_rules():
    assert dpt.arange(7, 0, -2, dtype="f4").shape == (4,) and dpt.arange(0, 1, 0.25, dtype="f4").shape == (4,)
    assert dpt.arange(7, 0, -2, dtype="f8").shape == (4,)
    x = dpt.arange(9.7, stop=10)
    assert x.shape == (1,) and x.dtype == np.float64
    assert dpt.arange(0, stop=10, step=None, dtype="int32").shape == (10,)
    b = dpt.arange(0, stop=2, dtype="bool")
    assert b.shape == (2,) and b.dtype == np.dtype(bool)
    x = dpt.arange(-2.5, stop=200, step=100, dtype="int32")
    assert x.shape[0] == 3 and int(x[1]) == 99 + int(x[0])
    x = dpt.arange(+2.5, stop=200, step=100, dtype="int32")
    assert x.shape[0] == 2 and int(x[1]) == 100 + int(x[0])
    assert dpt.arange(0, stop=np.float32(504), step=100, dtype="f4").shape == (6,)
    assert dpt.arange(-5, stop=10**2, step=2.7, dtype="int64").shape == (39,)  # length from the uncast arguments
    x = dpt.linspace(0, 15, num=16)
    assert x.dtype == np.float64 and x.shape == (16,) and x.strides == (1,)
    for dt in ("f2", "f4", "f8"):
        mx = np.finfo(dt).max
        x = dpt.linspace(mx, mx, endpoint=True, num=16, dtype=dt)
        assert x.shape == (16,)
        np.testing.assert_allclose(host(x), np.linspace(mx, mx, endpoint=True, num=16, dtype=dt))
    assert_same(host(dpt.linspace(0.1, 9.1, 11, endpoint=True, dtype=int)), np.linspace(0.1, 9.1, 11, endpoint=True, dtype=int))


def test_like_constructors_layout():
    sh = (10, 10)
    likes = (lambda x, o: dpt.full_like(x, 2, order=o), lambda x, o: dpt.empty_like(x, order=o),
             lambda x, o: dpt.ones_like(x, order=o), lambda x, o: dpt.zeros_like(x, order=o))
    values = (2, None, 1, 0)
    for order in "KA":
        for src_order, flag in (("C", "c_contiguous"), ("F", "f_contiguous")):
            x = dpt.zeros(sh, dtype="i4", order=src_order)
            for mk, v in zip(likes, values):
                r = mk(x, order)
                assert getattr(r.flags, flag)
                assert v is None or (host(r) == v).all()
        x3 = dpt.zeros(sh, dtype="i4", order="C")[::-2, :5]
        for mk, v in zip(likes, values):
            r = mk(x3, order)
            if order == "K":
                assert r.strides == (-5, 1) and not r.flags.forc
            else:
                assert r.flags.c_contiguous
            assert v is None or (host(r) == v).all()
    x = dpt.zeros(sh, dtype="i4")
    assert (host(dpt.full_like(x, dpt.asarray(2, dtype="i4"), order="K")) == 2).all()
    col = dpt.arange(10, dtype="i4")[:, dpt.newaxis]
    assert_same(host(dpt.full_like(x, col, order="K")), np.tile(np.arange(10, dtype="i4")[:, None], (1, 10)))


# ---- dtype routines: test_tensor_dtype_routines.py:73-172 ---------------------------------------------
def test_isdtype_finfo_iinfo():
    names = ["bool", "int8", "int16", "int32", "int64", "uint8", "uint16", "uint32", "uint64",
             "float16", "float32", "float64", "complex64", "complex128"]
    cats = {
        "bool": ["bool"],
        "signed integer": ["int8", "int16", "int32", "int64"],
        "unsigned integer": ["uint8", "uint16", "uint32", "uint64"],
        "integral": ["int8", "int16", "int32", "int64", "uint8", "uint16", "uint32", "uint64"],
        "real floating": ["float16", "float32", "float64"],
        "complex floating": ["complex64", "complex128"],
        "numeric": [d for d in names if d != "bool"],
    }
    for name in names:
        dt = dpt.dtype(name)
        for kind, members in cats.items():
            assert dpt.isdtype(dt, kind) == (name in members)
    assert dpt.isdtype(dpt.bool, ("real floating", "bool")) and not dpt.isdtype(dpt.bool, ("integral", "real floating"))
    assert dpt.isdtype(dpt.int16, ("real floating", "signed integer"))
    assert not dpt.isdtype(dpt.int16, ("bool", "unsigned integer", "real floating"))
    assert dpt.isdtype(dpt.uint8, (dpt.uint8, dpt.uint16)) and not dpt.isdtype(dpt.uint8, (dpt.bool, dpt.int32, dpt.float32))
    assert dpt.isdtype(dpt.float32, (dpt.float16, dpt.float32, dpt.float64))
    assert dpt.isdtype(dpt.complex64, ("integral", "complex floating"))
    for bad in ([dpt.int32, dpt.bool], "f4", float, 123, "complex"):
        with pytest.raises((TypeError, ValueError)):
            dpt.isdtype(dpt.int32, bad)
    assert dpt.finfo(dpt.empty((), dtype="f4")).dtype == np.float32
    assert dpt.iinfo(dpt.empty((), dtype="i4")).dtype == np.int32
    with pytest.raises(ValueError):
        dpt.iinfo("O")
    with pytest.raises(ValueError):
        dpt.finfo("O")
