import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
sys.path.insert(0, ROOT)
sys.path.insert(0, os.path.join(ROOT, "oracle"))
sys.path.insert(0, os.path.dirname(os.path.abspath(__file__)))

import __graft_entry__ as entry  # noqa: E402

entry.load_package()


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (gfx950)")


def _built(path):
    return os.path.exists(path)


@pytest.fixture(scope="session", autouse=True)
def _native_built():
    """Tests load what is built; they build only if nothing is."""
    from polarai_framework_amd import LIB_DEVICE
    import polar_oracle
    if not _built(LIB_DEVICE) or not _built(polar_oracle.LIB_PATH):
        entry.build()


@pytest.fixture(scope="session")
def dev():
    from polarai_framework_amd import capi
    d = capi.Device(0)  # raises without a GPU: gpu tests must not pass silently
    yield d
    d.close()
