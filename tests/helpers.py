"""Shared helpers of the GPU parity tests."""
import numpy as np

import dpnp_amd.tensor as dpt
from oracle import oracle as orc

ALL = list(dpt._dtypes.ALL_DTYPES)
REAL = [d for d in ALL if d.kind in "iuf"]
INTS = [d for d in ALL if d.kind in "iu"]
FLOATS = [d for d in ALL if d.kind == "f"]


def dev(a, **kw):
    return dpt.asarray(np.asarray(a), **kw)


def host(x):
    return dpt.asnumpy(x)


def random_array(rng, shape, dtype, lo=-100, hi=100):
    dtype = np.dtype(dtype)
    if dtype.kind == "b":
        return rng.integers(0, 2, shape).astype(bool)
    if dtype.kind in "iu":
        info = np.iinfo(dtype)
        return rng.integers(max(lo, info.min), min(hi, info.max) + 1, shape).astype(dtype)
    if dtype.kind == "f":
        return rng.uniform(lo, hi, shape).astype(dtype)
    return (rng.uniform(lo, hi, shape) + 1j * rng.uniform(lo, hi, shape)).astype(dtype)


def assert_same(got, want):
    """Bit-level agreement (NaNs in the same places)."""
    got, want = np.asarray(got), np.asarray(want)
    assert got.dtype == want.dtype, (got.dtype, want.dtype)
    assert got.shape == want.shape, (got.shape, want.shape)
    np.testing.assert_array_equal(got, want)
    if got.dtype.kind == "f":  # -0.0 and +0.0 compare equal: check the sign bit as well
        ok = ~np.isnan(want)
        np.testing.assert_array_equal(np.signbit(got[ok]), np.signbit(want[ok]))


def assert_ulp(got, exact_hi, max_ulp=4.0):
    got = np.asarray(got)
    err = orc.ulp_error(got, exact_hi)
    worst = float(np.max(err)) if err.size else 0.0
    assert worst <= max_ulp, f"{worst} ULP"


def strided_views(a):
    """(description, numpy view) variants of a 1-D or 2-D host array as in the reference's tests:
    reversed, every other element, transposed."""
    out = [("contig", a)]
    if a.ndim == 1:
        out += [("rev", a[::-1]), ("step2", a[::2]), ("rev_step2", a[::-2]), ("offset1", a[1:])]
    else:
        out += [("T", a.T), ("cols2", a[:, ::2]), ("rows_rev", a[::-1]), ("both_rev2", a[::-2, ::-2])]
    return out


def dev_view_like(np_view, np_base):
    """Device array with the same layout as `np_view` inside a device copy of `np_base`."""
    d = dev(np_base)
    off = (np_view.__array_interface__["data"][0] - np_base.__array_interface__["data"][0]) // np_base.itemsize
    from dpnp_amd.tensor._usmarray import usm_ndarray

    return usm_ndarray(np_view.shape, dtype=np_view.dtype, buffer=d, offset=d._offset + off,
                       strides=[s // np_base.itemsize for s in np_view.strides])
