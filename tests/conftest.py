import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu on the GPU box)")


@pytest.fixture(scope="session")
def fixtures():
    import numpy as np
    return np.load(os.path.join(ROOT, "tests", "golden", "reference_fixture.npz"), allow_pickle=False)


@pytest.fixture(scope="session")
def kats():
    import json
    with open(os.path.join(ROOT, "tests", "golden", "kats.json")) as fh:
        return json.load(fh)


@pytest.fixture(scope="session", autouse=True)
def _library_test_hooks():
    """The library ignores its tuning and test hooks (cusig_amd_force_*, ...) until they are switched on."""
    import ctypes
    try:
        from pysiglib_amd import _loader as L
    except Exception:       # no built library: the tests that need it fail on their own
        yield
        return
    L.CUSIG.cusig_amd_enable_test_hooks.argtypes = (ctypes.c_int,)
    L.CUSIG.cusig_amd_enable_test_hooks.restype = None
    L.CUSIG.cusig_amd_enable_test_hooks(1)
    yield
    L.CUSIG.cusig_amd_enable_test_hooks(0)
