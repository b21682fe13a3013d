import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu on the GPU box)")


@pytest.fixture(scope="session")
def gpu():
    """The product package with device 0 selected; fails loudly when there is no GPU."""
    import tcbnn_amd
    from tcbnn_amd import _lib
    n = _lib.device_count()
    assert n >= 1, "no HIP device visible: GPU tests need an MI355X"
    _lib.set_device(0)
    return tcbnn_amd
