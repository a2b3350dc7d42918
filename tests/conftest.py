import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)
sys.path.insert(0, os.path.dirname(os.path.abspath(__file__)))


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu)")


@pytest.fixture(scope="session", autouse=True)
def _native_libraries():
    """Loads what is built; builds only if nothing is."""
    from horovod_amd import build
    build.ensure_built()


@pytest.fixture(scope="session")
def orc():
    import oracle_util
    return oracle_util.Oracle()


@pytest.fixture(scope="session")
def ref():
    """The reference's own half.h/half.cc built into oracle/_ref (only where the
    reference tree was mounted at build time)."""
    import oracle_util
    r = oracle_util.load_ref()
    if r is None:
        pytest.skip("oracle/_ref/libhvdref.so not built (reference tree absent)")
    return r


@pytest.fixture(scope="session")
def gpu():
    import torch
    if not torch.cuda.is_available():
        pytest.skip("no GPU")
    import gpu_util
    return gpu_util.Gpu()
