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


@pytest.fixture
def knobs(monkeypatch):
    """Sets FUSILLI_HIP_* tuning variables for one test.  The library parses
    them once per process, so every change is followed by fhip_tuning_reload,
    also when the test ends and the variables are gone again."""
    from fusilli_amd import capi
    lib = capi.load()

    def set_knobs(**kv):
        for name, value in kv.items():
            monkeypatch.setenv("FUSILLI_HIP_" + name, str(value))
        assert lib.fhip_tuning_reload() == 0

    yield set_knobs
    monkeypatch.undo()
    lib.fhip_tuning_reload()
