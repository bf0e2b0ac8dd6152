import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: test needs a real MI355X (run with -m gpu)")


@pytest.fixture(scope="session")
def lib():
    """The loaded C-ABI library; GPU tests call the HIP path through it."""
    from alto_amd import _lib
    return _lib.load()


@pytest.fixture
def software_sr():
    """Stochastic rounding with ``use_asm=None`` runs the software rule for the duration of the test (the library's
    default is the hardware converts, as in the reference on gfx950)."""
    import alto_amd.mxfp4 as m
    from alto_amd.mxfp4 import _runtime as rt
    before = rt.hardware_stochastic_rounding()
    m.use_hardware_stochastic_rounding(False)
    yield
    m.use_hardware_stochastic_rounding(before)
