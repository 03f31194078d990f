import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu on the GPU box)")


@pytest.fixture(scope="session")
def oracle_ops():
    from oracle.jvm_oracle import JvmOracleOperations
    return JvmOracleOperations()


@pytest.fixture(scope="session")
def hip():
    """The process-wide HIP operations object. No fallback: fails if the library or the
    GPU is missing."""
    import kten_amd
    ops = kten_amd.platform(0)
    yield ops
    ops.sync()


@pytest.fixture()
def gc(hip):
    """Every raw tensor a test creates is released when the test ends."""
    with hip.garbageCollector():
        yield hip
