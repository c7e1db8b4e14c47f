import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs an MI355X (runs the HIP library through the C ABI)")


@pytest.fixture(scope="session")
def gpu():
    """The C-ABI library with a live device; GPU tests fail (not skip) when it is missing."""
    from aspen_amd import api
    assert os.path.exists(api.LIB_PATH), "libaspen_amd.so has not been built"
    assert api.lib().aspen_hip_init() == 0, api.lib().aspen_hip_last_error().decode()
    api.lib().aspen_hip_set_flags(2)     # count executed tiles so that run_stats() can be asserted on
    api.lib().aspen_keep_layer_outputs(1)   # the parity tests compare EVERY layer, also those only a fused shortcut consumes
    return api
