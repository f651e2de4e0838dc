import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu on the GPU box)")


@pytest.fixture(scope="session")
def built_library():
    """Path of libsspmm_amd.so; compiles it first only when no built library is there."""
    from sspmm_amd import _lib
    harness = os.path.join(ROOT, "sspmm_amd", "bin", "sspmm_test")
    if not (os.path.exists(_lib.library_path()) and os.path.exists(harness)):
        _lib.build_library(force=False)
    return _lib.library_path()


@pytest.fixture(scope="session")
def oracle():
    from oracle import oracle as O
    O.build()
    return O
