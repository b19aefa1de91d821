import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run by `pytest -m gpu` on the GPU box)")


@pytest.fixture(scope="session")
def oracle():
    import oracle as o
    return o


@pytest.fixture(scope="session")
def ref(oracle):
    """The reference's own host objects (oracle/_ref), skipped where they were not built."""
    r = oracle.ref_lib()
    if r is None:
        pytest.skip("oracle/_ref not built (no reference tree here)")
    return r
