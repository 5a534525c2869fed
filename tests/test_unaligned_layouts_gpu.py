"""Layouts whose rows or base pointers are aligned to the element only: rows of odd length, views that
start at x[k:], transposed operands with odd extents.  The kernels read them with 16-byte accesses that
start at any element; results must equal the oracle bit for bit (integers, IEEE basic ops) and every
element outside the written view must keep its value."""
import numpy as np
import pytest

import dpnp_amd.tensor as dpt
from oracle import oracle as orc
from tests.helpers import assert_same, dev, host, random_array

pytestmark = pytest.mark.gpu


def oracle_sum(a, axis):
    if axis is None:
        return orc.reduce("sum", a.reshape(-1), 1)
    return orc.reduce("sum", np.moveaxis(a, axis, -1), 1)

DTYPES = ["?", "i1", "u2", "f2", "i4", "f4", "i8", "f8", "c8", "c16"]
ODD_SHAPES = [(37, 1001), (5, 4099), (1000, 3), (129, 17), (64, 1023), (3, 5, 257)]


@pytest.mark.parametrize("dt", DTYPES)
def test_contiguous_with_offsets_and_guard_elements(dt):
    rng = np.random.default_rng(3)
    n = 9001
    a, b = random_array(rng, n, dt), random_array(rng, n, dt)
    op = (lambda x, y: dpt.logical_xor(x, y)) if dt == "?" else (lambda x, y: dpt.add(x, y))
    ref = (lambda x, y: np.logical_xor(x, y)) if dt == "?" else (lambda x, y: x + y)
    for ka, kb, ko in [(1, 0, 0), (0, 1, 3), (3, 2, 1), (5, 5, 5), (7, 1, 2)]:
        m = n - 8
        fill = random_array(rng, n, dt)
        o = dev(fill)
        r = op(dev(a)[ka:ka + m], dev(b)[kb:kb + m])
        assert_same(host(r), ref(a[ka:ka + m], b[kb:kb + m]))
        if dt == "?":
            dpt.logical_xor(dev(a)[ka:ka + m], dev(b)[kb:kb + m], out=o[ko:ko + m])
        else:
            dpt.add(dev(a)[ka:ka + m], dev(b)[kb:kb + m], out=o[ko:ko + m])
        want = fill.copy()
        want[ko:ko + m] = ref(a[ka:ka + m], b[kb:kb + m])
        assert_same(host(o), want)


@pytest.mark.parametrize("src", ["i1", "f2", "i4", "f8"])
@pytest.mark.parametrize("dst", ["?", "u1", "i2", "f4", "f8", "c16"])
def test_casts_between_widths_at_offsets(src, dst):
    # the narrow side of a cast moves fewer than 16 bytes per pack; several packs per thread
    rng = np.random.default_rng(5)
    for n in (1, 63, 64, 127, 1000, 4096, 16384 + 3, 70001):
        a = random_array(rng, n + 3, src, lo=0)
        for k in (0, 1, 3):
            v = dev(a)[k:k + n]
            assert_same(host(dpt.astype(v, dst)), orc.cast(a[k:k + n], dst))
    for n in (255, 8192, 50001):  # predicates: wide in, one byte out
        a = random_array(rng, n, src)
        assert_same(host(dpt.less(dev(a), dev(a[::-1].copy()))), a < a[::-1])


@pytest.mark.parametrize("dt", ["i1", "f2", "f4", "f8", "c16"])
@pytest.mark.parametrize("shape", ODD_SHAPES)
def test_rows_of_odd_length(dt, shape):
    rng = np.random.default_rng(7)
    a, b = random_array(rng, shape, dt), random_array(rng, shape, dt)
    da, db = dev(a), dev(b)
    inner = shape[-1]
    # slices along the last dim make every row start at another alignment
    if inner > 4:
        sl = (Ellipsis, slice(1, inner - 1))
        assert_same(host(dpt.add(da[sl], db[sl])), a[sl] + b[sl])
        fill = random_array(rng, shape, dt)
        o = dev(fill)
        dpt.subtract(da[sl], db[sl], out=o[sl])
        want = fill.copy()
        want[sl] = a[sl] - b[sl]
        assert_same(host(o), want)
        # stride 2 along the inner dim
        s2 = (Ellipsis, slice(1, None, 2))
        assert_same(host(dpt.add(da[s2], db[s2])), a[s2] + b[s2])
    row = random_array(rng, (1,) * (len(shape) - 1) + (inner,), dt)
    col = random_array(rng, shape[:-1] + (1,), dt)
    assert_same(host(dpt.add(da, dev(row))), a + row)
    assert_same(host(dpt.add(da, dev(col))), a + col)
    if len(shape) == 2:
        assert_same(host(dpt.add(da.mT, db.mT)), a.T + b.T)
        assert_same(host(dpt.add(da.mT, dev(np.ascontiguousarray(b.T)))), a.T + b.T)
        assert_same(host(dpt.copy(da.mT, order="C")), np.ascontiguousarray(a.T))
        assert_same(host(dpt.where(da.mT != db.mT, da.mT, dev(np.ascontiguousarray(b.T)))), np.where(a.T != b.T, a.T, b.T))


@pytest.mark.parametrize("dt", ["i1", "u2", "i4", "f4", "f8"])
@pytest.mark.parametrize("shape", ODD_SHAPES + [(4097, 33), (2, 100003)])
def test_reductions_over_odd_shapes_and_offsets(dt, shape):
    rng = np.random.default_rng(11)
    a = random_array(rng, shape, dt, lo=-5, hi=5)
    da = dev(a)
    for axis in list(range(len(shape))) + [None]:
        assert_same(host(dpt.max(da, axis=axis)), np.max(a, axis=axis))
        assert_same(host(dpt.argmin(da, axis=axis)), np.argmin(a, axis=axis))
        got = host(dpt.sum(da, axis=axis))
        if np.dtype(dt).kind == "f":
            np.testing.assert_allclose(got, oracle_sum(a, axis), rtol=1e-5 if dt == "f4" else 1e-12, atol=1e-4 if dt == "f4" else 1e-10)
        else:
            assert_same(got, oracle_sum(a, axis))
    if shape[-1] > 4:
        sl = (Ellipsis, slice(1, shape[-1] - 2))
        for axis in range(len(shape)):
            assert_same(host(dpt.min(da[sl], axis=axis)), np.min(a[sl], axis=axis))
            assert_same(host(dpt.argmax(da[sl], axis=axis)), np.argmax(a[sl], axis=axis))
            assert_same(host(dpt.count_nonzero(da[sl], axis=axis)), np.count_nonzero(a[sl], axis=axis).astype(np.int64))


@pytest.mark.parametrize("dt", ["?", "i1", "u2", "f2", "i4", "f4", "f8", "c16"])
def test_short_rows_with_row_and_column_operands(dt):
    # x - mean(x, axis=0), x / norm(x, axis=1)[:, None]: rows shorter than 512 bytes are walked flat,
    # the small operands indexed by position modulo / divided by the row length
    rng = np.random.default_rng(13)
    itemsize = np.dtype(dt).itemsize
    for cols in (2, 3, 7, 16, 17, 33, 100, 127):
        if cols * itemsize >= 512:
            continue
        for rows in (1, 5, 1000, 20011):
            x = random_array(rng, (rows, cols), dt, lo=1, hi=9)
            row = random_array(rng, (cols,), dt, lo=1, hi=9)
            col = random_array(rng, (rows, 1), dt, lo=1, hi=9)
            dx, drow, dcol = dev(x), dev(row), dev(col)
            if dt == "?":
                assert_same(host(dpt.logical_xor(dx, drow)), np.logical_xor(x, row))
                assert_same(host(dpt.logical_and(dcol, dx)), np.logical_and(col, x))
                continue
            assert_same(host(dpt.subtract(dx, drow)), x - row)
            assert_same(host(dpt.subtract(drow, dx)), row - x)
            assert_same(host(dpt.add(dx, dcol)), x + col)
            assert_same(host(dpt.add(dcol, drow)), col + row)
            assert_same(host(dpt.less(dx, drow)), x < row)
            assert_same(host(dpt.where(dx > drow, dx, dcol)), np.where(x > row, x, np.broadcast_to(col, x.shape)))
            assert_same(host(dpt.clip(dx, drow, dcol)), orc.clip(x, np.broadcast_to(row, x.shape).copy(), np.broadcast_to(col, x.shape).copy()))
            fill = random_array(rng, (rows, cols), dt)
            o = dev(fill)
            dpt.multiply(dx, drow, out=o)
            if np.dtype(dt).kind != "c":
                assert_same(host(o), x * row)
            dpt.add(dx, drow, out=dx)  # in place
            assert_same(host(dx), x + row)


@pytest.mark.parametrize("dt", ["f4", "f8", "i2", "c8"])
def test_matrix_with_rows_of_megabytes_plus_a_row(dt):
    """Rows of 2 MiB and more combined with a broadcast row take the flat contiguous kernel, the row indexed by
    position modulo the (odd) row length; the same operands with a column stay with the row kernel."""
    rng = np.random.default_rng(41)
    ncols = (2 << 20) // np.dtype(dt).itemsize + 3
    a = rng.integers(-50, 50, (3, ncols)).astype(dt)
    row = rng.integers(-50, 50, (1, ncols)).astype(dt)
    col = rng.integers(-50, 50, (3, 1)).astype(dt)
    da, drow, dcol = dev(a), dev(row), dev(col)
    np.testing.assert_array_equal(host(dpt.add(da, drow)), a + row)
    np.testing.assert_array_equal(host(dpt.subtract(drow, da)), row - a)
    np.testing.assert_array_equal(host(dpt.multiply(da, dcol)), a * col)
    np.testing.assert_array_equal(host(dpt.where(dpt.greater(dpt.real(da) if dt == "c8" else da, 0), da, drow)),
                                  np.where(a.real > 0, a, row))


@pytest.mark.gpu
@pytest.mark.parametrize("dt", ["i1", "f2", "f4", "f8", "c16"])
def test_two_sliced_operands_every_alignment_of_the_output_rows(dt):
    # a + b over column slices of wider matrices: the rows kernel's straight-line form lays a row's packs so that the
    # stores are aligned, whatever the first column of the output slice; every offset of the three operands up to
    # two packs, row lengths around whole packs, result rows as rows of a wider matrix, every other row, reversed
    # rows, and a result type narrower than the operands (a comparison).  Guard columns stay untouched.
    rng = np.random.default_rng(67)
    per_pack = 16 // np.dtype(dt).itemsize
    wide = 4 * per_pack + 300
    a = random_array(rng, (37, wide), dt, -60, 60)
    b = random_array(rng, (37, wide), dt, -60, 60)
    da, db = dev(a), dev(b)
    for length in (1, per_pack - 1, per_pack, per_pack + 1, 5 * per_pack + 3, 256, 257):
        for oa, ob, oo in ((0, 0, 0), (1, 1, 1), (1, 2, 3), (per_pack - 1, 0, per_pack + 1), (3, per_pack, 2 * per_pack - 1),
                           (2, 2, 0), (0, 1, per_pack)):
            if max(oa, ob, oo) + length > wide:
                continue
            want = a[:, oa:oa + length] + b[:, ob:ob + length]
            out = dpt.full((37, wide), 7, dtype=dt)
            dpt.add(da[:, oa:oa + length], db[:, ob:ob + length], out=out[:, oo:oo + length])
            got = host(out)
            assert_same(got[:, oo:oo + length], want)
            assert (got[:, :oo] == 7).all() and (got[:, oo + length:] == 7).all()
    assert_same(host(dpt.subtract(da[:36:2, 1:-1], db[1::2, 2:])), a[:36:2, 1:-1] - b[1::2, 2:])
    assert_same(host(dpt.add(da[::-1, 3:-2], db[:, 1:-4])), a[::-1, 3:-2] + b[:, 1:-4])
    if dt != "c16":
        assert_same(host(dpt.less(da[:, 1:-1], db[:, 2:])), a[:, 1:-1] < b[:, 2:])
    # three dims, interior of a volume
    v = random_array(rng, (6, 9, 70), dt, -60, 60)
    dv = dev(v)
    assert_same(host(dpt.add(dv[1:-1, 1:-1, 1:-1], dv[:-2, 2:, 2:])), v[1:-1, 1:-1, 1:-1] + v[:-2, 2:, 2:])
