"""The two providers of device memory and the stream, each in a child process of its own: the package
where PyTorch cannot be imported at all (memory from dpx_mem_alloc, kernels on a stream of
dpx_stream_create: also what this process runs on by default), and the package on PyTorch's allocator
and current stream (DPNP_AMD_MEMORY=torch)."""
import os
import subprocess
import sys

import pytest

pytestmark = pytest.mark.gpu


def test_package_runs_on_its_own_allocator_and_stream():
    script = os.path.join(os.path.dirname(os.path.abspath(__file__)), "native_memory_check.py")
    env = dict(os.environ, DPNP_AMD_BLOCK_TORCH="1")
    env.pop("DPNP_AMD_MEMORY", None)
    r = subprocess.run([sys.executable, script], env=env, capture_output=True, text=True, timeout=110)
    assert r.returncode == 0 and r.stdout.strip().endswith("OK"), r.stdout[-2000:] + r.stderr[-4000:]


def test_package_runs_on_the_torch_allocator_and_stream_when_asked():
    pytest.importorskip("torch")
    script = os.path.join(os.path.dirname(os.path.abspath(__file__)), "torch_memory_check.py")
    env = dict(os.environ, DPNP_AMD_MEMORY="torch")
    env.pop("DPNP_AMD_BLOCK_TORCH", None)
    r = subprocess.run([sys.executable, script], env=env, capture_output=True, text=True, timeout=170)
    assert r.returncode == 0 and r.stdout.strip().endswith("OK"), r.stdout[-2000:] + r.stderr[-4000:]


def test_this_process_runs_on_the_native_provider_by_default():
    import dpnp_amd._lib as L

    if not os.environ.get("DPNP_AMD_MEMORY"):
        assert L.MEMORY == "native" and L.torch is None
