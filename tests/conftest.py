import os
import sys

import numpy as np
import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu)")


def _gpu_present():
    """True when this machine exposes an AMD GPU.  The answer does not depend on the
    library having been built: on a GPU machine without it the tests fail loudly."""
    if not os.path.exists("/dev/kfd"):
        return False
    from sapphire_amd import capi
    if not os.path.exists(capi.LIB_PATH):
        return True
    return capi.device_count() > 0


def pytest_collection_modifyitems(config, items):
    # GPU tests never silently pass without the card: they are skipped with a reason
    # only when no device is visible (the CPU container), and fail if the library is absent
    # on a machine that has one.
    has_gpu = None
    for item in items:
        if "gpu" in item.keywords:
            if has_gpu is None:
                has_gpu = _gpu_present()
            if not has_gpu:
                item.add_marker(pytest.mark.skip(reason="no GPU visible in this process"))


@pytest.fixture(scope="session")
def dev():
    """The C ABI bound to device 0."""
    from sapphire_amd import capi
    capi.call("sph_set_device", 0)
    return capi
