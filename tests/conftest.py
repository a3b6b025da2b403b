import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu on the GPU box)")


def pytest_collection_modifyitems(config, items):
    """GPU tests are skipped unless a device is visible, so that a plain
    `pytest tests/` on a CPU-only machine stays green."""
    try:
        import torch

        have_gpu = torch.cuda.is_available()
    except Exception:
        have_gpu = False
    if have_gpu:
        return
    skip = pytest.mark.skip(reason="no GPU visible")
    for item in items:
        if "gpu" in item.keywords:
            item.add_marker(skip)


@pytest.fixture
def tune():
    """tune(name, value): sets one of the library's GTM_* switches for the rest of the test (value
    None = not set); every switch a test touched is unset again when the test ends.  The library reads
    the environment only once, at load, so a test changes its switches through gtm_tuning_set."""
    from graphtsetlinmachine_amd import _abi

    touched = []

    def set_switch(name, value="1"):
        _abi.call("gtm_tuning_set", name.encode(), None if value is None else str(value).encode())
        touched.append(name)

    yield set_switch
    for name in touched:
        _abi.call("gtm_tuning_set", name.encode(), None)
