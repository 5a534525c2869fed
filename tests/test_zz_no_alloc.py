"""dpx_reduce_noalloc (static device scratch, no allocation) against dpx_reduce, through the C ABI.

The two entry points run the same kernels over the same partition, so every result must agree bit
for bit, floats included.  Each case calls the entry point twice in a row, the second time on a
smaller input: the static scratch keeps the first call's partials and the second must not see them.
"""
import numpy as np
import pytest

import dpnp_amd._lib as L
import dpnp_amd.tensor as dpt
from tests.helpers import dev, host

pytestmark = pytest.mark.gpu


def _stream():
    from dpnp_amd.tensor._device import current_stream_ptr

    return current_stream_ptr()


def _reduce(entry, op, x, trailing, out_dtype, aux=None):
    out = dpt.empty(x.shape[: x.ndim - trailing], dtype=out_dtype)
    L.check(entry(L.REDUCE_ID[op], x._as_view(), trailing, out._as_view(),
                  aux._as_view() if aux is not None else None, _stream()))
    return out


def _plan(op, x, trailing, out_dtype):
    out = dpt.empty(x.shape[: x.ndim - trailing], dtype=out_dtype)
    p = L.Plan()
    L.check(L.lib.dpx_reduce_plan(L.REDUCE_ID[op], x._as_view(), trailing, out._as_view(), p))
    return p


def _bits(a):
    a = np.ascontiguousarray(a)
    return a.view(np.uint8)


CASES = [
    # (name, op, in dtype, out dtype, big shape, small shape, trailing, transposed?)
    ("full sum f32", "sum", "f4", "f4", (1 << 24,), (1 << 20,), 1, False),
    ("rows sum f32, few long rows", "sum", "f4", "f4", (3, 1 << 22), (2, 1 << 19), 1, False),
    ("cols sum f32", "sum", "f4", "f4", (1 << 14, 1 << 10), (1 << 12, 200), 1, True),
    ("cols max f64", "max", "f8", "f8", (1 << 13, 777), (1 << 11, 130), 1, True),
    ("full prod f64", "prod", "f8", "f8", (1 << 22,), (1 << 18,), 1, False),
    ("flat sum of samples x features", "sum", "f4", "f4", (1 << 20, 8), (1 << 17, 3), 1, True),
    ("full sum int8 -> int64", "sum", "i1", "i8", (1 << 24,), (1 << 21,), 1, False),
    ("full count_nonzero u8", "count_nonzero", "u1", "i8", (1 << 24,), (1 << 19,), 1, False),
    ("full nanmean f32", "nanmean", "f4", "f4", (1 << 23,), (1 << 19,), 1, False),
    # partials wider than the result: (largest element, sum of exponentials) pairs, (count, mean, M2) triples
    ("full logsumexp f32", "logsumexp", "f4", "f4", (1 << 23,), (1 << 19,), 1, False),
    ("rows logsumexp f64", "logsumexp", "f8", "f8", (3, 1 << 21), (2, 1 << 18), 1, False),
    ("cols logsumexp f32", "logsumexp", "f4", "f4", (1 << 14, 1 << 10), (1 << 12, 200), 1, True),
    ("full one-pass squared deviations f32 -> f64", "sqdev_onepass", "f4", "f8", (1 << 24,), (1 << 20,), 1, False),
    ("cols one-pass squared deviations f64", "sqdev_onepass", "f8", "f8", (1 << 14, 1 << 10), (1 << 12, 200), 1, True),
]


@pytest.mark.parametrize("case", CASES, ids=[c[0] for c in CASES])
def test_noalloc_matches_dpx_reduce_twice_in_a_row(case):
    _name, op, idt, odt, big, small, trailing, tr = case
    rng = np.random.default_rng(20)
    split_seen = False
    for shape in (big, small):  # second call: smaller input, stale partials of the first in scratch
        if np.dtype(idt).kind == "f":
            a = rng.uniform(0.5, 1.5, shape).astype(idt) if op == "prod" else rng.standard_normal(shape).astype(idt)
            if op == "nanmean":
                a[rng.random(shape) < 0.01] = np.nan
        else:
            a = rng.integers(0, 100, shape).astype(idt)
        x = dev(a)
        if tr:
            x = x.T  # reduce the leading axis of the row-major matrix: outputs contiguous
        p = _plan(op, x, trailing, odt)
        split_seen |= p.splits > 1
        want = host(_reduce(L.lib.dpx_reduce, op, x, trailing, odt))
        got = host(_reduce(L.lib.dpx_reduce_noalloc, op, x, trailing, odt))
        assert got.dtype == want.dtype and got.shape == want.shape
        assert np.array_equal(_bits(got), _bits(want)), (shape, L.PATH_NAMES[p.path], p.splits)
        # against the host as well (the two entry points could be wrong together)
        ah = a.T if tr else a
        if op == "sum":
            ref = ah.astype("f8" if np.dtype(idt).kind == "f" else "i8").sum(axis=-1)
            np.testing.assert_allclose(got.astype("f8"), ref, rtol=1e-5, atol=1e-5 * np.abs(ah).sum(axis=-1).max())
        elif op == "max":
            assert np.array_equal(got, ah.max(axis=-1))
        elif op == "count_nonzero":
            assert np.array_equal(got, np.count_nonzero(ah, axis=-1))
        elif op == "logsumexp":
            h = ah.astype("f8")
            ref = np.log(np.exp(h - h.max(axis=-1, keepdims=True)).sum(axis=-1)) + h.max(axis=-1)
            np.testing.assert_allclose(got, ref, rtol=1e-5)
        elif op == "sqdev_onepass":
            np.testing.assert_allclose(got, ah.astype("f8").var(axis=-1) * ah.shape[-1], rtol=1e-10)
    assert split_seen, "no case exercised the scratch buffer"


def test_noalloc_with_aux_and_one_block_plans():
    rng = np.random.default_rng(21)
    a = rng.standard_normal((5, 1 << 20)).astype("f4")
    x = dev(a)
    mean = dev(a.mean(axis=1, dtype="f8").astype("f4"))
    want = host(_reduce(L.lib.dpx_reduce, "sumsqdev", x, 1, "f4", aux=mean))
    got = host(_reduce(L.lib.dpx_reduce_noalloc, "sumsqdev", x, 1, "f4", aux=mean))
    assert np.array_equal(_bits(got), _bits(want))
    np.testing.assert_allclose(got, ((a.astype("f8") - a.mean(axis=1, dtype="f8")[:, None]) ** 2).sum(axis=1), rtol=1e-5)
    # the NaN-ignoring variance around a given mean: (sum, count) pairs in scratch
    a[rng.random(a.shape) < 0.01] = np.nan
    x = dev(a)
    mean = dev(np.nanmean(a.astype("f8"), axis=1).astype("f4"))
    assert _plan("nanvar", x, 1, "f4").splits > 1
    want = host(_reduce(L.lib.dpx_reduce, "nanvar", x, 1, "f4", aux=mean))
    got = host(_reduce(L.lib.dpx_reduce_noalloc, "nanvar", x, 1, "f4", aux=mean))
    assert np.array_equal(_bits(got), _bits(want))
    np.testing.assert_allclose(got, np.nanvar(a.astype("f8"), axis=1), rtol=1e-5)
    # complex input around a complex mean, a real result
    z = (rng.standard_normal((3, 1 << 20)) + 1j * rng.standard_normal((3, 1 << 20))).astype("c8")
    x, mean = dev(z), dev(z.mean(axis=1, dtype="c16").astype("c8"))
    assert _plan("sumsqdev", x, 1, "f4").splits > 1
    want = host(_reduce(L.lib.dpx_reduce, "sumsqdev", x, 1, "f4", aux=mean))
    got = host(_reduce(L.lib.dpx_reduce_noalloc, "sumsqdev", x, 1, "f4", aux=mean))
    assert np.array_equal(_bits(got), _bits(want))
    np.testing.assert_allclose(got, z.astype("c16").var(axis=1) * z.shape[1], rtol=1e-5)
    # plans without scratch (one block per output) go the same way through both entry points
    b = dev(rng.standard_normal((4096, 512)).astype("f4"))
    assert _plan("sum", b, 1, "f4").splits == 1
    assert np.array_equal(_bits(host(_reduce(L.lib.dpx_reduce_noalloc, "sum", b, 1, "f4"))),
                          _bits(host(_reduce(L.lib.dpx_reduce, "sum", b, 1, "f4"))))


def test_noalloc_rejects_plans_beyond_the_static_scratch():
    # uint8 matrix with 500-byte rows summed over its rows: 512 blocks x 500 columns x 8 bytes of
    # partials do not fit the 2 MiB array
    x = dpt.ones((1 << 16, 500), dtype="u1").T
    p = _plan("sum", x, 1, "u8")
    assert p.scratch_bytes > L.NOALLOC_SCRATCH_BYTES
    out = dpt.zeros((500,), dtype="u8")
    rc = L.lib.dpx_reduce_noalloc(L.REDUCE_ID["sum"], x._as_view(), 1, out._as_view(), None, _stream())
    assert rc == L.ERR_BAD_ARGUMENT
    assert b"static scratch" in L.lib.dpx_last_error()
    assert not host(out).any()  # nothing was written
    assert (host(_reduce(L.lib.dpx_reduce, "sum", x, 1, "u8")) == 1 << 16).all()  # dpx_reduce takes it
    # argument checks come first and are the ones of dpx_reduce
    ro = dpt.zeros((3,), dtype="f4")
    rc = L.lib.dpx_reduce_noalloc(L.REDUCE_ID["sum"], dpt.ones((4, 7), dtype="f4")._as_view(), 1, ro._as_view(), None,
                                  _stream())
    assert rc == L.ERR_SHAPE_MISMATCH
