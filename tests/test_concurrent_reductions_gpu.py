"""Split reductions issued from two host threads at once, through the C ABI.

A reduction that is split over several blocks per output keeps its partial results in a scratch block of its
stream and lets the block that draws the last ticket fold them, in the same launch.  Launches on different
streams run side by side on the GPU, each on its own scratch block; launches on one stream, from whichever
thread, run in stream order on one block.  Every result here has an exact expected value (int64 sums, counts,
positions), every result is compared, and the first mismatch stops the run.
"""
import ctypes
import threading
import time

import numpy as np
import pytest

import dpnp_amd._lib as L
import dpnp_amd.tensor as dpt
from helpers import dev

pytestmark = pytest.mark.gpu

lib = L.lib


def _cases():
    """(name, entry, op id, device source view, trailing, result shape, result dtype, expected) of mixed shapes: rows
    split over blocks, columns split, a flat stream with short rows, one output over hundreds of blocks (two
    ticket levels), a search."""
    rng = np.random.default_rng(2024)
    out = []

    def add(name, a, view, trailing, op, search=False, want=None, res_dt="i8"):
        d = dev(a)
        v = view(d)
        p = L.Plan()
        res = dpt.empty(want.shape, dtype=res_dt)
        planner = lib.dpx_argreduce_plan if search else lib.dpx_reduce_plan
        ids = L.SEARCH_ID if search else L.REDUCE_ID
        L.check(planner(ids[op], v._as_view(), trailing, res._as_view(), p))
        assert p.splits > 1, (name, L.PATH_NAMES[p.path], p.splits)
        out.append((name, lib.dpx_argreduce if search else lib.dpx_reduce, ids[op], d, v, trailing, want, res_dt,
                    L.PATH_NAMES[p.path], p.splits))

    a = rng.integers(-1000, 1000, (3, 1 << 21)).astype("i8")
    add("rows split", a, lambda d: d, 1, "sum", want=a.sum(axis=1))
    a = rng.integers(-1000, 1000, (1 << 14, 384)).astype("i8")
    add("cols split", a, lambda d: d.T, 1, "sum", want=a.sum(axis=0))
    a = rng.integers(0, 100, (1 << 19, 6)).astype("i4")
    add("flat", a, lambda d: d.T, 1, "sum", want=a.sum(axis=0, dtype="i8"))
    a = rng.integers(-5, 6, (1 << 23,)).astype("i1")
    add("one output, two ticket levels", a, lambda d: d, 1, "sum", want=np.asarray(a.sum(dtype="i8")))
    a = rng.integers(0, 2, (1 << 22,)).astype("u1")
    add("count_nonzero", a, lambda d: d, 1, "count_nonzero", want=np.asarray(np.count_nonzero(a)).astype("i8"))
    a = rng.standard_normal(1 << 22).astype("f4")
    a[[77, 3_000_000]] = a.max() + 1  # first of two equal maxima
    add("argmax", a, lambda d: d, 1, "argmax", search=True, want=np.asarray(np.int64(77)))
    a = rng.standard_normal((1 << 13, 200)).astype("f8")
    add("argmin down the columns", a, lambda d: d.T, 1, "argmin", search=True, want=a.argmin(axis=0).astype("i8"))
    return out


class _Worker(threading.Thread):
    def __init__(self, cases, stream, seed, seconds, max_calls):
        super().__init__()
        self.cases, self.stream, self.seconds, self.max_calls = cases, stream, seconds, max_calls
        self.rng = np.random.default_rng(seed)
        self.calls, self.error = 0, None
        # results of this thread only: one device buffer and one host buffer per case
        self.res = [dpt.empty(c[6].shape, dtype=c[7]) for c in cases]

    def run(self):
        try:
            t0 = time.perf_counter()
            pending = []
            while self.calls < self.max_calls and time.perf_counter() - t0 < self.seconds and _stop.is_set() is False:
                k = int(self.rng.integers(len(self.cases)))
                _name, entry, op, _d, v, trailing, want, _dt, _path, _splits = self.cases[k]
                res = self.res[k]
                if entry is lib.dpx_reduce:
                    rc = entry(op, v._as_view(), trailing, res._as_view(), None, self.stream)
                else:
                    rc = entry(op, v._as_view(), trailing, res._as_view(), self.stream)
                if rc != L.OK:
                    raise RuntimeError(lib.dpx_last_error().decode())
                self.calls += 1
                pending.append(k)
                if len(pending) >= 4 or self.rng.random() < 0.3:  # read back in bursts: several launches in flight
                    self.check(pending[-1])
                    pending = []
            for k in set(pending):
                self.check(k)
        except Exception as e:  # noqa: BLE001
            self.error = e
            _stop.set()

    def check(self, k):
        want = self.cases[k][6]
        got = np.empty(want.shape, dtype=want.dtype)
        # (a copy on this thread's stream: it waits for the launches before it, and only for them)
        L.check(lib.dpx_copy_to_host(got.ctypes.data, self.res[k]._as_view().data, got.nbytes, self.stream))
        if not np.array_equal(got, want):
            bad = np.flatnonzero(np.atleast_1d(got != want))
            raise AssertionError(f"{self.cases[k][0]} ({self.cases[k][8]}, {self.cases[k][9]} splits), call {self.calls}: "
                                 f"{bad.size} wrong results, first at {bad[:3]}: {np.atleast_1d(got)[bad[:3]]} != "
                                 f"{np.atleast_1d(want)[bad[:3]]}")


_stop = threading.Event()


def _streams(n):
    out = []
    for _ in range(n):
        s = ctypes.c_void_p()
        L.check(lib.dpx_stream_create(ctypes.byref(s)))
        out.append(s)
    return out


@pytest.mark.parametrize("shared_stream", [False, True], ids=["a stream per thread", "one stream for both threads"])
def test_split_reductions_from_two_threads(shared_stream):
    from dpnp_amd.tensor import _device

    cases = _cases()
    L.check(lib.dpx_stream_synchronize(_device.current_stream_ptr()))  # the inputs are in place
    streams = _streams(1 if shared_stream else 2)
    _stop.clear()
    workers = [_Worker(cases, streams[i % len(streams)], seed=i, seconds=12.0, max_calls=2500) for i in range(2)]
    for w in workers:
        w.start()
    for w in workers:
        w.join(timeout=100)
    assert not any(w.is_alive() for w in workers), "a worker did not finish"
    for s in streams:
        L.check(lib.dpx_stream_synchronize(s))
        L.check(lib.dpx_stream_destroy(s))
    for w in workers:
        if w.error is not None:
            raise w.error
    assert min(w.calls for w in workers) >= 200, [w.calls for w in workers]
