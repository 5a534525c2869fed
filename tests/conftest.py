import os
import sys

import pytest

sys.path.insert(0, os.path.dirname(os.path.dirname(os.path.abspath(__file__))))

if os.environ.get("DPNP_AMD_BLOCK_TORCH") == "1":
    # run the suite as on a machine without PyTorch: the package then allocates device memory
    # and creates its stream through its own library
    import importlib.abc

    class _NoTorch(importlib.abc.MetaPathFinder):
        def find_spec(self, name, path=None, target=None):
            if name == "torch" or name.startswith("torch."):
                raise ImportError("torch is blocked in this process (DPNP_AMD_BLOCK_TORCH=1)")
            return None

    assert "torch" not in sys.modules, "torch was imported before the tests could block it"
    sys.meta_path.insert(0, _NoTorch())


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs an AMD GPU (run with -m gpu on an MI355X box)")


def _gpu_present():
    try:
        from dpnp_amd.tensor import _device

        return _device.gpu_available()
    except Exception:
        return False


def pytest_collection_modifyitems(config, items):
    if _gpu_present():
        return
    skip = pytest.mark.skip(reason="no GPU in this process")
    for item in items:
        if "gpu" in item.keywords:
            item.add_marker(skip)
