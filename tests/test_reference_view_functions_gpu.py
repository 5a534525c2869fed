"""Views and shape queries around the hot path, against NumPy on the same arrays (the cases of
dpnp/tests/test_manipulation.py and dpnp/tests/tensor/test_usm_ndarray_manipulation.py for moveaxis, swapaxes,
expand_dims, squeeze, flip, broadcast_arrays, atleast_nd, ravel, rollaxis, ndim / shape / size).  A view must share
the memory of its base: each case also writes through the view and reads the base."""
import numpy as np
import pytest

import dpnp_amd as dpnp
import dpnp_amd.tensor as dpt

pytestmark = pytest.mark.gpu


def pair(shape, dt="f4"):
    a = np.arange(int(np.prod(shape)), dtype=dt).reshape(shape)
    return a, dpnp.array(a)


def same(result, expected):
    got = result.asnumpy()
    assert got.shape == expected.shape and got.dtype == expected.dtype
    np.testing.assert_array_equal(got, expected)


def is_view_of(view, base):
    return view.get_array().usm_data is base.get_array().usm_data


@pytest.mark.parametrize("source, destination", [(0, 2), (-1, 0), ([0, 1], [2, 3]), ((3, 0), (0, 1)), (1, 1)])
def test_moveaxis(source, destination):
    a, d = pair((2, 3, 4, 5))
    r = dpnp.moveaxis(d, source, destination)
    same(r, np.moveaxis(a, source, destination))
    assert is_view_of(r, d)
    same(dpnp.square(r), np.square(np.moveaxis(a, source, destination)))
    with pytest.raises(np.exceptions.AxisError):
        dpnp.moveaxis(d, 4, 0)
    with pytest.raises(ValueError):
        dpnp.moveaxis(d, [0, 1], [2])
    with pytest.raises(ValueError):
        dpnp.moveaxis(d, [0, 0], [1, 2])


@pytest.mark.parametrize("axes", [(0, 1), (2, 0), (-1, -3), (1, 1)])
def test_swapaxes_and_rollaxis(axes):
    a, d = pair((2, 3, 4))
    same(dpnp.swapaxes(d, *axes), np.swapaxes(a, *axes))
    same(d.swapaxes(*axes), a.swapaxes(*axes))
    same(dpnp.sum(dpnp.swapaxes(d, *axes), axis=0), np.sum(np.swapaxes(a, *axes), axis=0))
    for axis, start in ((2, 0), (0, 3), (1, -1), (1, 1)):
        same(dpnp.rollaxis(d, axis, start), np.rollaxis(a, axis, start))
    with pytest.raises(ValueError):
        dpnp.rollaxis(d, 0, 5)
    with pytest.raises(np.exceptions.AxisError):
        dpnp.swapaxes(d, 3, 0)


def test_expand_dims_squeeze_flip_transposes():
    a, d = pair((3, 1, 4))
    for axis in (0, 1, -1, (0, 2), (-1, -2)):
        same(dpnp.expand_dims(d, axis), np.expand_dims(a, axis))
    same(dpnp.squeeze(d), np.squeeze(a))
    same(dpnp.squeeze(d, axis=1), np.squeeze(a, axis=1))
    with pytest.raises(ValueError):
        dpnp.squeeze(d, axis=0)
    for axis in (None, 0, 2, (0, 2), -1):
        r = dpnp.flip(d, axis)
        same(r, np.flip(a, axis))
        assert is_view_of(r, d)
        same(dpnp.add(r, d), np.flip(a, axis) + a)
    same(dpnp.fliplr(d), np.fliplr(a))
    same(dpnp.flipud(d), np.flipud(a))
    with pytest.raises(ValueError):
        dpnp.fliplr(dpnp.ones(3))
    same(dpnp.matrix_transpose(d), np.matrix_transpose(a))
    same(dpnp.permute_dims(d, (2, 0, 1)), np.transpose(a, (2, 0, 1)))
    same(dpnp.permute_dims(d), a.T)
    with pytest.raises(ValueError):
        dpnp.matrix_transpose(dpnp.ones(3))
    v = dpnp.expand_dims(d, 0)
    v[...] = 7
    assert (d.asnumpy() == 7).all()


def test_broadcast_arrays_and_shapes():
    a, d = pair((3, 1))
    b, e = pair((4,), "i4")
    got = dpnp.broadcast_arrays(d, e)
    want = np.broadcast_arrays(a, b)
    assert isinstance(got, tuple) and len(got) == 2
    for g, w in zip(got, want):
        same(g, w)
    assert is_view_of(got[0], d) and got[0].strides == (4, 0) and got[0].get_array().strides == (1, 0)
    same(dpnp.multiply(*got), a * b)
    assert dpnp.broadcast_arrays() == ()
    with pytest.raises(ValueError):
        dpnp.broadcast_arrays(dpnp.ones((2, 3)), dpnp.ones((4,)))
    with pytest.raises(NotImplementedError):
        dpnp.broadcast_arrays(d, subok=True)
    assert dpnp.broadcast_shapes((3, 1), (4,), ()) == (3, 4)
    assert [t.shape for t in dpt.broadcast_arrays(d.get_array(), e.get_array())] == [(3, 4), (3, 4)]


def test_atleast_nd():
    s, v, m = dpnp.array(3.0), dpnp.arange(4), dpnp.ones((2, 3))
    hs, hv, hm = s.asnumpy(), v.asnumpy(), m.asnumpy()
    for name in ("atleast_1d", "atleast_2d", "atleast_3d"):
        got = getattr(dpnp, name)(s, v, m)
        want = getattr(np, name)(hs, hv, hm)
        assert isinstance(got, tuple)
        for g, w in zip(got, want):
            same(g, w)
        same(getattr(dpnp, name)(v), getattr(np, name)(hv))
        with pytest.raises(TypeError):
            getattr(dpnp, name)([1, 2])
    assert dpnp.atleast_1d(v) is v and dpnp.atleast_3d(dpnp.ones((2, 2, 2, 2))).ndim == 4


@pytest.mark.parametrize("order", ["C", "F", "A"])
def test_ravel_and_flatten(order):
    a, d = pair((3, 4, 5))
    for src, hsrc in ((d, a), (d.T, a.T), (d[:, ::2], a[:, ::2]), (d[1], a[1])):
        same(dpnp.ravel(src, order=order), np.ravel(hsrc, order=order))
        same(src.ravel(order), hsrc.ravel(order))
        if order != "A":
            f = src.flatten(order)
            same(f, hsrc.flatten(order))
            assert not is_view_of(f, d)
    assert is_view_of(dpnp.ravel(d), d)
    with pytest.raises(NotImplementedError):
        dpnp.ravel(d, order="K")


def test_ndim_shape_size():
    a, d = pair((2, 3, 4))
    assert dpnp.ndim(d) == 3 and dpnp.ndim([[1, 2]]) == 2 and dpnp.ndim(d.get_array()) == 3
    assert dpnp.shape(d) == (2, 3, 4) and dpnp.shape([[1, 2]]) == (1, 2)
    assert dpnp.size(d) == 24 and dpnp.size(d, 1) == 3 and dpnp.size(d, (0, 2)) == 8 and dpnp.size([[1, 2]]) == 2
    with pytest.raises(np.exceptions.AxisError):
        dpnp.size(d, 3)
