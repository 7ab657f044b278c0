import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
for _p in (ROOT, os.path.join(ROOT, "tests")):
    if _p not in sys.path:
        sys.path.insert(0, _p)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu on the GPU box)")


@pytest.fixture(scope="session")
def oracle():
    from oracle.loader import Oracle
    return Oracle()


@pytest.fixture(scope="session")
def ttmi():
    """The C ABI, loaded through ctypes.  GPU tests call the kernels only through this."""
    from turbotransformers_amd import capi
    return capi.load()


@pytest.fixture(autouse=True)
def _release_kept_tensors():
    yield
    try:
        import helpers
        helpers._KEEP.clear()
    except ImportError:
        pass
