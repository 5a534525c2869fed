"""Arrays with more than 2^31 elements: 64-bit positions in the kernels and in the planner."""
import numpy as np
import pytest

import dpnp_amd.tensor as dpt
from tests.helpers import dev, host

pytestmark = pytest.mark.gpu

N = (1 << 31) + 12345


@pytest.fixture(scope="module")
def big():
    a = (np.arange(N, dtype=np.uint32) % 251).astype(np.uint8)
    return a, dev(a)


def test_elementwise_beyond_2p31(big):
    a, d = big
    c = dpt.add(d, d)                                   # uint8 wraps
    tail = host(c[N - 5000:])
    assert np.array_equal(tail, a[N - 5000:] + a[N - 5000:])
    assert np.array_equal(host(c[(1 << 31) - 100:(1 << 31) + 100]), (a + a)[(1 << 31) - 100:(1 << 31) + 100])
    s = host(dpt.multiply(d[::3], 3))                   # strided view of the whole range
    assert np.array_equal(s[-1000:], (a[::3] * np.uint8(3))[-1000:]) and s.shape[0] == (N + 2) // 3
    r = host(dpt.negative(d[::-1])[:1000])              # reversed: the last elements come first
    assert np.array_equal(r, (-a[::-1][:1000]).astype(np.uint8))


def test_reductions_beyond_2p31(big):
    a, d = big
    assert int(dpt.sum(d)) == int(a.sum(dtype=np.uint64))
    assert int(dpt.count_nonzero(d)) == int(np.count_nonzero(a))
    assert int(dpt.max(d)) == 250 and int(dpt.min(d)) == 0
    # the first maximum and a planted later one
    assert int(dpt.argmax(d)) == 250
    b = a.copy()
    b[N - 7] = 255
    db = dev(b)
    assert int(dpt.argmax(db)) == N - 7
    b[5] = 255
    db[5] = 255
    assert int(dpt.argmax(db)) == 5
    # two rows of more than 2^30 elements each; columns of a (n/4096, 4096) view
    rows = N // 2
    m = dpt.reshape(d[: 2 * rows], (2, rows))
    assert np.array_equal(host(dpt.sum(m, axis=1)), a[: 2 * rows].reshape(2, rows).sum(axis=1, dtype=np.uint64))
    cols = 4096
    r2 = N // cols
    m2 = dpt.reshape(d[: r2 * cols], (r2, cols))
    assert np.array_equal(host(dpt.sum(m2, axis=0)), a[: r2 * cols].reshape(r2, cols).sum(axis=0, dtype=np.uint64))
    assert np.array_equal(host(dpt.argmax(m2, axis=0)), a[: r2 * cols].reshape(r2, cols).argmax(axis=0))
