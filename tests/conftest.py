import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
for p in (ROOT, os.path.join(ROOT, "oracle"), os.path.dirname(os.path.abspath(__file__))):
    if p not in sys.path:
        sys.path.insert(0, p)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu on the GPU box)")


@pytest.fixture(scope="session")
def hip():
    """The HIP device: initialises libzenu_hip.so on device 0 (fails loudly if absent)."""
    import zenu_amd
    from zenu_amd import _lib
    _lib.check(zenu_amd.lib().zenu_hip_init(0), "zenu_hip_init")
    yield zenu_amd
