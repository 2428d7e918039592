import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
for p in (ROOT, os.path.join(ROOT, "tests")):
    if p not in sys.path:
        sys.path.insert(0, p)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu on the GPU box)")


def _gpu_present() -> bool:
    try:
        from oxibonsai_amd import _lib
        return _lib.lib().oxb_hip_device_count() > 0
    except Exception:
        return False


@pytest.fixture(scope="session")
def backend():
    """The native-hip backend; GPU tests fail (not skip) when the library cannot start on a GPU box."""
    import oxibonsai_amd as ox
    return ox.NativeHipBackend(0)


def pytest_collection_modifyitems(config, items):
    if _gpu_present():
        return
    skip = pytest.mark.skip(reason="no GPU in this container")
    for it in items:
        if "gpu" in it.keywords:
            it.add_marker(skip)
