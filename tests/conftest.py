import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs an MI355X (runs the HIP kernels through the C ABI)")


@pytest.fixture(scope="session")
def gpu():
    """Selects device 0 and hands out the C-ABI library; fails (not skips) when
    the library is missing, because a GPU test that silently ran elsewhere
    would prove nothing."""
    import shadow_amd
    lib = shadow_amd.hip()
    assert shadow_amd.device_count() >= 1, "no HIP device visible"
    shadow_amd.check(lib.shdw_hip_set_device(0))
    return lib
