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


@pytest.fixture(params=["wide", "narrow", "general"])
def lane_shape(request):
    """The three routes a pooled lookup can take, for test modules that ask for this fixture:
    "wide" = 16-byte lanes, the lean kernel where the shape allows it (what large launches get);
    "narrow" = 4-byte lanes (what launches too small to fill the device get by default);
    "general" = 16-byte lanes with the lean kernel switched off (everything through the general kernel)."""
    import fbgemm_amd
    lib = fbgemm_amd.lib()
    lib.fbgemm_amd_set_narrow_below_waves(1024 if request.param == "narrow" else 0)
    lib.fbgemm_amd_set_lean(0 if request.param == "general" else 1)
    yield request.param
    lib.fbgemm_amd_set_narrow_below_waves(-1)
    lib.fbgemm_amd_set_lean(-1)
