"""dpnp.var / dpnp.std of complex input and with the caller's `mean=`
(dpnp/dpnp_iface_statistics.py:1644-1660,1832-1869; dpnp/tests/test_statistics.py:1065-1150) against the
oracle's restatement, over every reduction kernel family, and the C-ABI op under them
(DPX_R_SUMSQDEV of complex input)."""
import numpy as np
import pytest

import dpnp_amd as dpnp
import dpnp_amd.tensor as dpt
from dpnp_amd import _lib
from helpers import dev, host, random_array
from oracle import oracle as orc

pytestmark = pytest.mark.gpu

RTOL = {"f2": 2e-3, "f4": 1e-5, "f8": 1e-12}


def _oracle(a, axis, mean, ddof, out_dtype=None):
    """orc.var_around_mean on the axes moved last; `mean` in its keepdims shape."""
    nd = a.ndim
    axes = tuple(range(nd)) if axis is None else tuple(ax % nd for ax in (axis if isinstance(axis, tuple) else (axis,)))
    keep = [d for d in range(nd) if d not in axes]
    moved = np.ascontiguousarray(np.transpose(a, keep + list(axes)))
    m = None
    if mean is not None:
        m = np.broadcast_to(mean, [1 if d in axes else a.shape[d] for d in range(nd)])
        m = m.reshape([a.shape[d] for d in keep])
    return orc.var_around_mean(moved, len(axes), mean=m, ddof=ddof, out_dtype=out_dtype)


# shapes chosen to land in each kernel family: long rows (row kernel, split), many short rows (staged rows),
# columns (column kernel and its split), few columns (flat kernel), reduced dims that stay apart (walked rows
# and columns), a full reduction
LAYOUTS = [
    ((7, 5000), 1), ((3, 70000), 1), ((4000, 9), 1), ((3000, 40), 0), ((70000, 5), 0), ((600, 1100), 0),
    ((12, 50, 33), (0, 2)), ((9, 40, 16, 5), (1, 3)), ((300, 700), None), ((5, 6, 7), -1), ((2, 3), (0, 1)),
]


@pytest.mark.parametrize("shape,axis", LAYOUTS)
@pytest.mark.parametrize("dt", ["c8", "c16"])
def test_complex_var_std_every_kernel_family(shape, axis, dt):
    rng = np.random.default_rng(hash((shape, str(axis), dt)) % 2**32)
    a = random_array(rng, shape, dt, -3, 5)
    x = dpnp.array(a)
    for keepdims in (False, True):
        for ddof in (0, 1):
            want = _oracle(a, axis, None, ddof)
            got = dpnp.var(x, axis=axis, ddof=ddof, keepdims=keepdims)
            assert got.dtype == want.dtype
            g = got.asnumpy()
            if keepdims:
                assert g.shape == np.var(a, axis=axis, keepdims=True).shape
                g = g.reshape(want.shape)
            np.testing.assert_allclose(g, want, rtol=RTOL[want.dtype.str[1:]])
    s = dpnp.std(x, axis=axis).asnumpy()
    np.testing.assert_allclose(s, np.sqrt(_oracle(a, axis, None, 0).astype("f8")), rtol=RTOL[s.dtype.str[1:]])
    # var(z) = var(Re z) + var(Im z), each part through the real kernels (stride-2 views of the same memory)
    parts = (dpnp.var(x.real, axis=axis) + dpnp.var(x.imag, axis=axis)).asnumpy()
    np.testing.assert_allclose(dpnp.var(x, axis=axis).asnumpy(), parts, rtol=10 * RTOL[parts.dtype.str[1:]])


@pytest.mark.parametrize("shape,axis", LAYOUTS)
@pytest.mark.parametrize("dt", ["f4", "f8", "f2", "i4", "u1", "?", "c8", "c16"])
def test_var_std_with_given_mean(shape, axis, dt):
    rng = np.random.default_rng(hash((shape, str(axis), dt, 1)) % 2**32)
    a = random_array(rng, shape, dt, -3, 5)
    if dt == "f2":
        # runs of more than a few thousand elements: the sum of squares and the count leave float16's range (in
        # the reference as well); keep the layout, shorten the reduced axes
        red = range(a.ndim) if axis is None else [ax % a.ndim for ax in (axis if isinstance(axis, tuple) else (axis,))]
        a = np.ascontiguousarray(a[tuple(slice(0, 60) if d in red else slice(None) for d in range(a.ndim))])
    x = dpnp.array(a)
    exact = np.mean(a.astype("c16" if a.dtype.kind == "c" else "f8"), axis=axis, keepdims=True)
    # the mean as dpnp.mean gives it (the documented use), and a mean that is off (nothing checks that it is the mean)
    for m_host in (None, exact + (0.25 if a.dtype.kind != "c" else 0.25 - 0.5j)):
        if m_host is None:
            m_dev = dpnp.mean(x, axis=axis, keepdims=True)
            m_host = m_dev.asnumpy()
        else:
            m_host = m_host.astype(dpnp.mean(x, axis=axis).dtype)
            m_dev = dpnp.array(m_host)
        for keepdims in (False, True):
            want = _oracle(a, axis, m_host, 0)
            got = dpnp.var(x, axis=axis, keepdims=keepdims, mean=m_dev)
            assert got.dtype == want.dtype, (got.dtype, want.dtype)
            g = got.asnumpy().reshape(want.shape)
            np.testing.assert_allclose(g, want, rtol=RTOL[want.dtype.str[1:]], atol=1e-30)
        want = _oracle(a, axis, m_host, 1)
        got = x.std(axis=axis, mean=m_dev, ddof=1)
        np.testing.assert_allclose(got.asnumpy(), np.sqrt(want.astype("f8")), rtol=RTOL[want.dtype.str[1:]], atol=1e-30)


def test_reference_docstring_values_and_shift_identity():
    # dpnp_iface_statistics.py:1821-1826, 1629-1634
    a = dpnp.array([[14, 8, 11, 10], [7, 9, 10, 11], [10, 15, 5, 10]])
    mean = dpnp.mean(a, axis=1, keepdims=True)
    assert np.array_equal(dpnp.var(a, axis=1, mean=mean).asnumpy(), [4.6875, 2.1875, 12.5])
    np.testing.assert_allclose(dpnp.std(a, axis=1, mean=mean).asnumpy(), [2.16506351, 1.47901995, 3.53553391], rtol=1e-8)
    rng = np.random.default_rng(3)
    h = rng.normal(2, 3, (64, 4096))
    x = dpnp.array(h)
    shift = rng.normal(0, 1, (64, 1))
    got = dpnp.var(x, axis=1, mean=dpnp.array(h.mean(axis=1, keepdims=True) + shift)).asnumpy()
    np.testing.assert_allclose(got, dpnp.var(x, axis=1).asnumpy() + shift[:, 0] ** 2, rtol=1e-12)


def test_mean_shapes_dtypes_out_and_divisor():
    rng = np.random.default_rng(11)
    h = rng.normal(0, 1, (6, 50, 8)).astype("f4")
    x = dpnp.array(h)
    # a scalar mean, a mean with fewer dims, a float64 mean for float32 data (the deviations are then float64)
    for m in (np.float32(0.5), np.full((1,), 0.5, "f4"), np.full((50, 1), 0.5, "f4"), np.full((6, 50, 1), 0.5, "f8")):
        got = dpnp.var(x, axis=2, mean=dpnp.array(m))
        want = _oracle(h, 2, np.asarray(m), 0)
        assert got.dtype == want.dtype
        np.testing.assert_allclose(got.asnumpy(), want, rtol=RTOL[want.dtype.str[1:]])
    # a mean that varies along the reduced axis (full shape): the reference's sequence of calls
    full = rng.normal(0, 1, h.shape).astype("f4")
    got = dpnp.var(x, axis=2, mean=dpnp.array(full)).asnumpy()
    np.testing.assert_allclose(got, ((h - full).astype("f8") ** 2).sum(axis=2) / 8, rtol=1e-5)
    # a complex mean of real data
    got = dpnp.var(x, axis=2, mean=dpnp.array(np.complex64(0.5 + 1j))).asnumpy()
    np.testing.assert_allclose(got, (np.abs(h - (0.5 + 1j)).astype("f8") ** 2).sum(axis=2) / 8, rtol=1e-5)
    # dtype= and out=
    m = dpnp.mean(x, axis=2, keepdims=True)
    got = dpnp.var(x, axis=2, mean=m, dtype="f8")
    assert got.dtype == np.dtype("f8")
    np.testing.assert_allclose(got.asnumpy(), _oracle(h, 2, m.asnumpy(), 0, "f8"), rtol=1e-6)
    out = dpnp.empty((6, 50), dtype="f4")
    assert dpnp.var(x, axis=2, mean=m, out=out) is out
    np.testing.assert_allclose(out.asnumpy(), _oracle(h, 2, m.asnumpy(), 0), rtol=1e-5)
    z = dpnp.array((h + 1j * full).astype("c8"))
    out = dpnp.empty((6, 8), dtype="f4")
    assert dpnp.std(z, axis=1, out=out) is out
    np.testing.assert_allclose(out.asnumpy(), np.std((h + 1j * full).astype("c16"), axis=1), rtol=1e-5)
    # complex data with a real dtype=: the reference's mean drops the imaginary part (as NumPy's does)
    with np.testing.suppress_warnings() as sup:
        sup.filter(np.exceptions.ComplexWarning)
        want = np.var((h + 1j * full).astype("c8"), axis=1, dtype="f8")
        got = dpnp.var(z, axis=1, dtype="f8").asnumpy()
    np.testing.assert_allclose(got, want, rtol=1e-5)
    # N - ddof: zero gives NaN, a negative one is kept as the reference keeps it
    assert np.isnan(dpnp.var(z, axis=1, ddof=50).asnumpy()).all()
    np.testing.assert_allclose(dpnp.var(z, axis=1, ddof=52).asnumpy(), -25 * dpnp.var(z, axis=1).asnumpy(), rtol=1e-5)
    np.testing.assert_allclose(dpnp.var(z, axis=1, correction=1).asnumpy(), dpnp.var(z, axis=1, ddof=1).asnumpy())
    with pytest.raises(ValueError):
        dpnp.var(z, ddof=1, correction=1)
    with pytest.raises(TypeError):
        dpnp.std(z, ddof="1")
    # empty reduced axis and empty result
    e = dpnp.array(np.zeros((3, 0), "c8"))
    assert np.isnan(dpnp.var(e, axis=1).asnumpy()).all() and dpnp.var(e, axis=0).shape == (0,)
    # tensor level: var / std of complex input stay refused there (dpnp/tensor/_statistical_functions.py:233-235)
    with pytest.raises(ValueError):
        dpt.var(z.get_array())


def test_non_finite_values_propagate():
    h = np.ones((5, 300), "c16")
    h[1, 7] = np.nan
    h[2, 200] = complex(np.inf, 0)
    h[3, 0] = complex(0, -np.inf)
    got = dpnp.var(dpnp.array(h), axis=1).asnumpy()
    assert got[0] == 0 and got[4] == 0 and np.isnan(got[1:4]).all()
    r = np.ones((5, 300))
    r[1, 299] = np.inf
    got = dpnp.var(dpnp.array(r), axis=1, mean=dpnp.array(np.ones((5, 1)))).asnumpy()
    assert got[0] == 0 and got[1] == np.inf


@pytest.mark.parametrize("src_dt,dst_dt,aux_dt", [("c8", "f4", "c8"), ("c8", "f8", "c16"), ("c16", "f8", "c16")])
def test_c_abi_sumsqdev_complex(src_dt, dst_dt, aux_dt):
    rng = np.random.default_rng(7)
    op = _lib.REDUCE_ID["sumsqdev"]
    assert _lib.lib.dpx_reduce_dtype_supported(op, dpt._dtypes.dtype_id(np.dtype(src_dt)), dpt._dtypes.dtype_id(np.dtype(dst_dt)))
    assert not _lib.lib.dpx_reduce_dtype_supported(op, dpt._dtypes.dtype_id(np.dtype("c16")), dpt._dtypes.dtype_id(np.dtype("f4")))
    for shape, trailing in (((33, 2000), 1), ((2, 1 << 20), 1), ((2000, 33), 1), ((1 << 18,), 1), ((40, 30, 20), 2)):
        a = random_array(rng, shape, src_dt, -2, 2)
        lead = shape[: len(shape) - trailing]
        m = random_array(rng, lead, aux_dt, -1, 1)
        x, aux, dst = dev(a), dev(m), dpt.empty(lead, dtype=dst_dt)
        _lib.check(_lib.lib.dpx_reduce(op, x._as_view(), trailing, dst._as_view(), aux._as_view(), _stream()))
        n = int(np.prod(shape[len(lead):]))
        want = orc.var_around_mean(a, trailing, mean=m, out_dtype=dst_dt).astype("f8") * n
        np.testing.assert_allclose(host(dst), want, rtol=RTOL[dst_dt])
    # an aux of the wrong type is refused
    a, bad = dev(np.zeros((4, 8), src_dt)), dev(np.zeros(4, dst_dt))
    dst = dpt.empty((4,), dtype=dst_dt)
    rc = _lib.lib.dpx_reduce(op, a._as_view(), 1, dst._as_view(), bad._as_view(), _stream())
    assert rc == _lib.ERR_BAD_DTYPE


def _stream():
    from dpnp_amd.tensor._tensor_impl import _stream as s

    return s(None)
