import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu)")


def _have_gpu() -> bool:
    import torch
    return torch.cuda.is_available()


def pytest_collection_modifyitems(config, items):
    # GPU tests are skipped (not failed) when someone runs the whole suite on a CPU box.
    if _have_gpu():
        return
    skip = pytest.mark.skip(reason="no GPU in this process")
    for item in items:
        if "gpu" in item.keywords:
            item.add_marker(skip)


@pytest.fixture(scope="session")
def sa():
    """The library with PyTorch's device allocations routed through it, as in the reference's
    scripts (test.py:14-16): installed before the first device allocation of the process, so
    every tensor any GPU test makes comes from sideaware_malloc_auto."""
    from l2_torch_alloc_amd import wrapper
    wrapper.sideaware_init()
    return wrapper
