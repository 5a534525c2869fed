"""Run by test_native_memory_gpu.py in a process of its own, with PyTorch blocked: the package on
the library's own device memory pool and stream (dpx_mem_*, dpx_stream_*).  Prints OK at the end."""
import ctypes
import os
import sys

os.environ["DPNP_AMD_BLOCK_TORCH"] = "1"
sys.path.insert(0, os.path.dirname(os.path.abspath(__file__)))
import conftest  # noqa: F401,E402  (installs the import blocker, puts the repository on sys.path)

import numpy as np  # noqa: E402

import dpnp_amd as dpnp  # noqa: E402
import dpnp_amd._lib as L  # noqa: E402
from dpnp_amd.tensor import _device  # noqa: E402

assert "torch" not in sys.modules and L.torch is None and L.MEMORY == "native"
assert _device.gpu_available()
assert isinstance(_device.Device(0).name, str)  # the marketing name may be empty where the id table is not installed

rng = np.random.default_rng(11)
# arrays, ufuncs, reductions and temporaries through the pool
a, b = rng.normal(size=(1000, 777)).astype("f4"), rng.normal(size=(1000, 777)).astype("f4")
da, db = dpnp.array(a), dpnp.array(b)
for _ in range(3):  # temporaries of one round are the next round's blocks
    r = dpnp.exp(da * db + 1).sum(axis=0)
    np.testing.assert_allclose(r.asnumpy(), np.exp(a * b + 1, dtype="f4").sum(axis=0, dtype="f4"), rtol=2e-5)
assert int(dpnp.argmax(da)) == int(a.argmax())
np.testing.assert_array_equal(dpnp.where(da > 0, da, db).asnumpy(), np.where(a > 0, a, b))
big = dpnp.ones(1 << 23, dtype="f4")  # a staggered large block
assert float(big.sum()) == float(1 << 23)
dpnp.synchronize()

# the pool through the C ABI
lib = L.lib
s1, s2, p, q = ctypes.c_void_p(), ctypes.c_void_p(), ctypes.c_void_p(), ctypes.c_void_p()
L.check(lib.dpx_stream_create(ctypes.byref(s1)))
L.check(lib.dpx_stream_create(ctypes.byref(s2)))
n = 5 << 20
L.check(lib.dpx_mem_alloc(ctypes.byref(p), n, s1))
h = rng.integers(0, 256, n, dtype=np.uint8)
L.check(lib.dpx_copy_from_host(p, h.ctypes.data, n, s1))
first = p.value
L.check(lib.dpx_mem_free(p, s1))
assert lib.dpx_mem_free(p, s1) != 0 and b"not a live block" in lib.dpx_last_error()  # double free: an error
# same stream: the block comes straight back
L.check(lib.dpx_mem_alloc(ctypes.byref(p), n - 100, s1))
assert p.value == first
L.check(lib.dpx_copy_from_host(p, h.ctypes.data, n - 100, s1))
L.check(lib.dpx_mem_free(p, s1))
# another stream: the block comes back after a device-side wait for s1, and the copy queued on
# s1 above must not land after the data written on s2
L.check(lib.dpx_mem_alloc(ctypes.byref(q), n, s2))
assert q.value == first
h2 = (h ^ 0x5A).astype(np.uint8)
L.check(lib.dpx_copy_from_host(q, h2.ctypes.data, n, s2))
out = np.zeros(n, dtype=np.uint8)
L.check(lib.dpx_copy_to_host(out.ctypes.data, q, n, s2))
assert np.array_equal(out, h2)
used, cached = ctypes.c_size_t(), ctypes.c_size_t()
L.check(lib.dpx_mem_stats(ctypes.byref(used), ctypes.byref(cached)))
assert used.value >= n
L.check(lib.dpx_mem_free(q, s2))
L.check(lib.dpx_stream_destroy(s2))
L.check(lib.dpx_stream_destroy(s1))
assert lib.dpx_stream_destroy(s1) != 0  # not a library stream any more
del da, db, r, big
L.check(lib.dpx_mem_stats(ctypes.byref(used), ctypes.byref(cached)))
assert cached.value > 0
L.check(lib.dpx_mem_release_cached())
L.check(lib.dpx_mem_stats(ctypes.byref(used), ctypes.byref(cached)))
assert cached.value == 0, cached.value
print("OK")
