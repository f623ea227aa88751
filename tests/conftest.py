import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run on the GPU box)")


def pytest_collection_modifyitems(config, items):
    """GPU tests are skipped, not failed, when no device is present."""
    try:
        import torch

        have_gpu = torch.cuda.is_available()
    except Exception:  # pragma: no cover
        have_gpu = False
    if have_gpu:
        return
    skip = pytest.mark.skip(reason="no HIP device in this process")
    for item in items:
        if "gpu" in item.keywords:
            item.add_marker(skip)


@pytest.fixture
def diagnostic_build():
    """Runs the test's ops in libtuna_amd_bench.so (the product's object files plus process-wide routing switches and
    launch counters), so that tuna_set_* and tuna_*_launches apply to the calls the test makes.  Yields that library."""
    from tuna_amd import _lib

    with _lib.diagnostic_build() as L:
        yield L
