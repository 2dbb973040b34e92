import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs an MI355X (run with -m gpu on the GPU box)")


def _gpu_available() -> bool:
    try:
        from minit_amd import lib
        return lib.device_count() > 0
    except Exception:
        return False


@pytest.fixture(scope="session")
def hip():
    """The loaded HIP library; GPU tests fail (not skip) if it cannot be loaded."""
    from minit_amd import lib
    lib.cdll()
    assert lib.device_count() > 0, "no HIP device visible"
    return lib


def pytest_collection_modifyitems(config, items):
    if _gpu_available():
        return
    skip = pytest.mark.skip(reason="no HIP device in this environment")
    for item in items:
        if "gpu" in item.keywords:
            item.add_marker(skip)
