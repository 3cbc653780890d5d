import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu)")


@pytest.fixture(scope="session")
def oracle():
    import oracle as o
    o.build(("oracle",))
    return o


@pytest.fixture(params=["wide", "narrow"])
def lane_shape(request, monkeypatch):
    """Launches too small to fill the device take 4-byte lanes by default; test modules that ask for this
    fixture run every test with that policy and with the 16-byte lanes large launches get (the library
    reads the switch on every call)."""
    monkeypatch.setenv("FBGEMM_AMD_NARROW_BELOW_WAVES", "0" if request.param == "wide" else "1024")
    return request.param
