import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
sys.path.insert(0, ROOT)
sys.path.insert(0, os.path.dirname(os.path.abspath(__file__)))


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs an MI355X (gfx950) GPU; run with -m gpu on the GPU box")


@pytest.fixture(scope="session")
def gpu():
    """The loaded HIP library with device 0 selected. A missing library is an error (no fallback); a missing GPU skips."""
    from ufsm_amd import lib
    from ufsm_amd.lp import load
    load()                                   # raises when libufsm_lp.so is not built
    if lib.mi_device_count() == 0:
        pytest.skip("no GPU visible")
    assert lib.mi_init(0) == 0, "device 0 is not a gfx950 GPU"
    yield lib
    from ufsm_amd import LP
    LP.check()
