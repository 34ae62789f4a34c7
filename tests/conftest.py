"""Shared test set-up: import paths, the `gpu` marker, seeded helpers."""

import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
for p in (ROOT, os.path.join(ROOT, "falcon-perception_amd")):
    if p not in sys.path:
        sys.path.insert(0, p)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu)")
    config.addinivalue_line("markers", "bigmem: holds tens of GB of HBM and asserts that they are free: needs a GPU "
                                       "no other process is using (deselect with -m 'gpu and not bigmem')")


def pytest_collection_modifyitems(config, items):
    import torch

    if torch.cuda.is_available():
        return
    skip = pytest.mark.skip(reason="no GPU in this environment")
    for item in items:
        if "gpu" in item.keywords:
            item.add_marker(skip)


@pytest.fixture(scope="session")
def native_lib():
    """The built C-ABI library (never built from inside a test)."""
    from falcon_perception_amd import _native

    return _native.lib()


@pytest.fixture(autouse=True)
def give_large_pools_back(request):
    """Tests that hold tens of GB (the 180 GB pool, the 2^32-lane append, the far pages) hand the memory back
    to the driver when they end, not when the process does: the driver clears freed device memory in the
    background, and a process that starts while 180 GB are being cleared measures 4 % less HBM bandwidth."""
    yield
    if "gpu" not in request.keywords:
        return
    import torch

    if torch.cuda.is_available() and torch.cuda.memory_reserved() > (8 << 30):
        torch.cuda.empty_cache()
