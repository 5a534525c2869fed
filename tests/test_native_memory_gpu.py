"""The package without PyTorch: device memory from dpx_mem_alloc, kernels on a stream of
dpx_stream_create.  Runs in a child process, because this one may already hold torch."""
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
