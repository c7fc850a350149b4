import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)
sys.path.insert(0, os.path.dirname(os.path.abspath(__file__)))


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu on the GPU box)")


def pytest_collection_modifyitems(config, items):
    import torch
    if torch.cuda.is_available():
        return
    skip = pytest.mark.skip(reason="no GPU in this environment")
    for item in items:
        if "gpu" in item.keywords:
            item.add_marker(skip)


@pytest.fixture(params=["fixed_shape_kernels", "run_time_geometry_kernels"])
def kernel_path(request):
    """Gather and scatter have kernel instances compiled for the benchmark configurations' block shapes beside the
    kernels that take any geometry at run time.  Tests that use this fixture run twice: as the library dispatches
    by itself, and with the library's test hook keeping it on the run-time-geometry kernels."""
    import ctypes
    from sbnet_amd import _lib
    hook = _lib.load().sbnet_test_force_generic
    hook.restype, hook.argtypes = ctypes.c_int, [ctypes.c_int]
    prev = hook(1 if request.param == "run_time_geometry_kernels" else 0)
    yield request.param
    hook(prev)
