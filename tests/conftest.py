import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs an MI355X (gfx950) device")


@pytest.fixture(scope="session")
def ctx():
    """One C-ABI context on device 0 for the whole session."""
    from fusilli_amd import capi
    c = capi.Context(0)
    yield c
    c.close()
