"""Calls with a stride-2 input whose rows are whole waves of packs take the two-rows kernel
(ew_rows2): every pattern it is instantiated for, against NumPy (exact operations) through the
Python layer and the C ABI.  A[:, ::2], real / imaginary parts of complex arrays, batch dims, the
one-dimensional form the collapse produces, and shapes next to the kernel's conditions that must
stay on the generic kernel."""
import numpy as np
import pytest

import dpnp_amd as dpnp
import dpnp_amd._lib as L
import dpnp_amd.tensor as dpt
from tests.helpers import assert_same, dev, host, random_array

pytestmark = pytest.mark.gpu


def _path(fn_name, *arrays):
    p = L.Plan()
    views = [dpt.broadcast_to(a, arrays[-1].shape)._as_view() for a in arrays]
    if len(arrays) == 2:
        L.check(L.lib.dpx_unary_plan(L.UNARY_ID[fn_name], views[0], views[1], p))
    elif len(arrays) == 3:
        L.check(L.lib.dpx_binary_plan(L.BINARY_ID[fn_name], views[0], views[1], views[2], p))
    else:
        L.check(L.lib.dpx_where_plan(views[0], views[1], views[2], views[3], p))
    return L.PATH_NAMES[p.path]


@pytest.mark.parametrize("dt", ["f4", "i4", "u4", "f8", "i8", "c8"])
@pytest.mark.parametrize("shape", [(6, 512), (64, 1024), (2, 3, 4, 256), (130, 2048)])
def test_stride2_patterns(dt, shape):
    rng = np.random.default_rng(71)
    E = 16 // np.dtype(dt).itemsize
    cols = shape[-1] * (E // 4 if E > 4 else 1)
    shape = shape[:-1] + (cols,)
    assert cols % (64 * E) == 0
    base = shape[:-1] + (2 * cols,)
    a, b = random_array(rng, base, dt, -9, 9), random_array(rng, base, dt, -9, 9)
    row = random_array(rng, (1,) * (len(shape) - 1) + (cols,), dt, -9, 9)
    da, db, drow = dev(a), dev(b), dev(row)
    va, vb = da[..., ::2], db[..., ::2]
    ha, hb = a[..., ::2], b[..., ::2]
    out = dpt.empty(shape, dtype=dt)
    assert _path("negative", va, out) == "ew_rows2"
    assert _path("subtract", va, vb, out) == "ew_rows2"
    assert _path("subtract", va, drow, out) == "ew_rows2"
    assert _path("subtract", drow, va, out) == "ew_rows2"
    assert_same(host(dpt.negative(va)), -ha)
    assert_same(host(dpt.subtract(va, vb)), ha - hb)
    assert_same(host(dpt.subtract(va, drow)), ha - row)      # operand order matters: both ways
    assert_same(host(dpt.subtract(drow, va)), row - ha)
    assert_same(host(dpt.subtract(va, 3)), ha - np.asarray(3, dtype=dt))          # scalar second
    assert_same(host(dpt.subtract(3, va)), np.asarray(3, dtype=dt) - ha)
    assert_same(host(dpt.subtract(va[..., 1:2, :] if len(shape) > 1 else va, vb)), (ha[..., 1:2, :] if len(shape) > 1 else ha) - hb)
    # odd columns: the view starts one element in, and its last read ends at the allocation's end
    assert_same(host(dpt.negative(da[..., 1::2])), -a[..., 1::2])
    assert_same(host(dpt.add(da[..., 1::2], db[..., 1::2])), a[..., 1::2] + b[..., 1::2])
    if np.dtype(dt).kind != "c":
        assert_same(host(dpt.greater(va, 0)), ha > 0)
        mask = dev(ha > hb)
        assert _path("where", mask, va, drow, out) == "ew_rows2"
        assert_same(host(dpt.where(mask, va, drow)), np.where(ha > hb, ha, row))
    if dt in ("f4", "f8", "i4"):
        w = dpnp.where_compare("greater", dpnp.ndarray._create_from_usm_ndarray(va), 0,
                               dpnp.ndarray._create_from_usm_ndarray(va), dpnp.ndarray._create_from_usm_ndarray(drow))
        assert_same(w.asnumpy(), np.where(ha > 0, ha, row))
    # in place and into a view with the same layout
    o2 = dev(b)
    dpt.multiply(va, vb, out=o2[..., :cols])
    want = b.copy()
    want[..., :cols] = ha * hb
    if np.dtype(dt).kind != "c":
        assert_same(host(o2), want)


def test_real_and_imaginary_parts_are_stride2_views():
    rng = np.random.default_rng(73)
    z = (rng.standard_normal((40, 768)) + 1j * rng.standard_normal((40, 768))).astype("c8")
    dz = dev(z)
    out = dpt.empty((40, 768), dtype="f4")
    assert dz.real.strides == (2 * 768, 2) and dz.imag.strides == (2 * 768, 2)
    assert _path("add", dz.real, dz.imag, out) == "ew_rows2"
    assert_same(host(dpt.add(dz.real, dz.imag)), z.real + z.imag)
    assert_same(host(dpt.square(dz.imag)), z.imag * z.imag)
    z16 = z.astype("c16")
    dz16 = dev(z16)
    assert_same(host(dpt.subtract(dz16.imag, dz16.real)), z16.imag - z16.real)


def test_shapes_next_to_the_conditions_stay_generic():
    rng = np.random.default_rng(79)
    for shape in [(8, 250), (7, 256), (8, 260), (1, 256)]:
        a = random_array(rng, (shape[0], 2 * shape[1]), "f4")
        da = dev(a)
        row = random_array(rng, (1, shape[1]), "f4")
        out = dpt.empty(shape, dtype="f4")
        path = _path("add", da[:, ::2], dev(row), out)
        assert (path == "ew_rows2") == (shape[1] % 256 == 0 and shape[0] % 2 == 0), (shape, path)
        assert_same(host(dpt.add(da[:, ::2], dev(row))), a[:, ::2] + row)
        assert_same(host(dpt.exp(da[:, ::2]))[0, :3] > 0, np.ones(3, dtype=bool))
    # rows walked backwards: the highest row is not the last one, generic kernel
    a = random_array(rng, (16, 512), "f4")
    da = dev(a)
    out = dpt.empty((16, 256), dtype="f4")
    assert _path("negative", da[::-1, ::2], out) == "ew_rows"
    assert_same(host(dpt.negative(da[::-1, ::2])), -a[::-1, ::2])
    # overlapping windows (row stride smaller than a row's extent, explicit strides): rows interleave, so a
    # row's wave-wide read could end past the last element the view addresses; generic kernel
    from dpnp_amd.tensor._usmarray import usm_ndarray

    flat = random_array(rng, (4 * 100 + 2 * 256 - 1,), "f4")
    dflat = dev(flat)
    win = usm_ndarray((4, 256), dtype="f4", buffer=dflat, strides=(100, 2))
    out = dpt.empty((4, 256), dtype="f4")
    assert _path("negative", win, out) == "ew_rows"
    want = np.lib.stride_tricks.as_strided(flat, (4, 256), (400, 8))
    assert_same(host(dpt.negative(win)), -want)
    # rows exactly one extent apart (the closest that do not interleave) keep the two-rows kernel
    flat = random_array(rng, (4 * 511,), "f4")
    dflat = dev(flat)
    win = usm_ndarray((4, 256), dtype="f4", buffer=dflat, strides=(511, 2))
    assert _path("negative", win, out) == "ew_rows2"
    assert_same(host(dpt.negative(win)), -np.lib.stride_tricks.as_strided(flat, (4, 256), (2044, 8)))
    # narrow element types keep the generic kernel (two-byte packs of eight)
    h = random_array(rng, (8, 2048), "f2")
    assert_same(host(dpt.negative(dev(h)[:, ::2])), -h[:, ::2])


def test_full_size_cfg4_shapes():
    rng = np.random.default_rng(3)
    A = rng.standard_normal((8192, 8192)).astype("f4")
    B = rng.standard_normal((1, 4096)).astype("f4")
    dA, dB = dev(A), dev(B)
    V1 = dA[:, ::2]
    assert_same(host(dpt.multiply(V1, dB)), A[:, ::2] * B)
    assert_same(host(dpt.where(dpt.greater(V1, 0), V1, dB)), np.where(A[:, ::2] > 0, A[:, ::2], B))
    assert_same(host(dpt.negative(V1)), -A[:, ::2])
    I = rng.integers(-2**31, 2**31, (8192, 8192), dtype=np.int64).astype("i4")
    dI = dev(I)
    assert_same(host(dpt.bitwise_and(dI[:, ::2], dI[:, 1::2])), I[:, ::2] & I[:, 1::2])
