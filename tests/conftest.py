import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs an MI355X (run with -m gpu on the GPU box)")


@pytest.fixture(scope="session")
def gpu():
    """The GPU library, loaded; fails (never skips) when there is no device, because a
    `-m gpu` run that silently does nothing would look like a pass."""
    from incin_amd import capi
    capi.load()
    n = capi.device_count()
    assert n >= 1, "no ROCm device visible"
    return capi
