import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu on the GPU box)")


@pytest.fixture(scope="session")
def gpu():
    """(ctx, stream) on device 0 through the C ABI.  No skip: a GPU test without a GPU or without
    the built library must fail."""
    import trueno_amd as t
    ctx = t.CudaContext(0)
    stream = t.CudaStream(ctx)
    yield ctx, stream
    stream.synchronize()


@pytest.fixture(scope="session")
def coracle():
    from oracle.cref import COracle
    return COracle()
