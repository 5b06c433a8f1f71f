import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run on the GPU box)")


@pytest.fixture(scope="session")
def bruteforce_lib():
    """ctypes handle of the C brute-force checker (built on demand with gcc)."""
    import ctypes

    from oracle.build_oracle import build

    lib = ctypes.CDLL(build(force=False))
    return lib
