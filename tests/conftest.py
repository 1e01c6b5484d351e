import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
for p in (ROOT, os.path.join(ROOT, "aether-ml_amd")):
    if p not in sys.path:
        sys.path.insert(0, p)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu)")


def _gpu_present():
    return os.path.exists("/dev/kfd")


def pytest_collection_modifyitems(config, items):
    if _gpu_present():
        return
    skip = pytest.mark.skip(reason="no GPU in this container")
    for item in items:
        if "gpu" in item.keywords:
            item.add_marker(skip)


@pytest.fixture
def tune():
    """Kernel-choice overrides of the library for one test (aeth_debug_set): `tune(gather_bm=128)`.
    Every switch goes back to "decide from the shape" when the test ends."""
    from aether import _lib

    def set_switches(**switches):
        for name, value in switches.items():
            _lib.debug_set(name, value)

    yield set_switches
    _lib.debug_set(None)
