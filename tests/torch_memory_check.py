"""Run by test_native_memory_gpu.py in a process of its own with DPNP_AMD_MEMORY=torch: the package on
PyTorch's caching allocator and current stream, sharing data with torch without copies.  Prints OK at the end."""
import os
import sys

os.environ["DPNP_AMD_MEMORY"] = "torch"
sys.path.insert(0, os.path.dirname(os.path.dirname(os.path.abspath(__file__))))

import numpy as np  # noqa: E402

import dpnp_amd as dpnp  # noqa: E402
import dpnp_amd._lib as L  # noqa: E402
from dpnp_amd.tensor import _device  # noqa: E402
from dpnp_amd.tensor._usmarray import usm_ndarray  # noqa: E402

torch = L.torch
assert L.MEMORY == "torch" and torch is not None and _device.gpu_available()
rng = np.random.default_rng(5)
a, b = rng.normal(size=(513, 1027)).astype("f4"), rng.normal(size=(513, 1027)).astype("f4")
da, db = dpnp.array(a), dpnp.array(b)
assert isinstance(da.get_array()._buf, torch.Tensor)
for _ in range(3):
    r = dpnp.exp(da * db + 1).sum(axis=0)
    np.testing.assert_allclose(r.asnumpy(), np.exp(a * b + 1, dtype="f4").sum(axis=0, dtype="f4"), rtol=2e-5)
assert int(dpnp.argmax(da)) == int(a.argmax())
# a torch tensor's memory seen as an array of this package (no copy), on torch's current stream
t = torch.arange(1 << 20, device="cuda", dtype=torch.float32)
view = usm_ndarray((1 << 20,), dtype="f4", buffer=t.view(torch.uint8))
assert float(dpnp.sum(dpnp.ndarray._create_from_usm_ndarray(view))) == float(t.sum())
t.mul_(2)  # torch work, then this package's, in stream order
assert float(dpnp.max(dpnp.ndarray._create_from_usm_ndarray(view))) == 2.0 * ((1 << 20) - 1)
# and under a side stream that torch makes current
side = torch.cuda.Stream()
with torch.cuda.stream(side):
    assert _device.current_stream_ptr() == side.cuda_stream
    s = dpnp.sum(da, axis=1)
side.synchronize()
np.testing.assert_allclose(s.asnumpy(), a.sum(axis=1, dtype="f8"), rtol=1e-5, atol=1e-3)
dpnp.synchronize()
print("OK")
