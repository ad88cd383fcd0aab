import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu on the GPU box)")


@pytest.fixture(scope="session")
def oracle():
    """The CPU parity checker (oracle/): built on demand with gcc."""
    from oracle import binary_backend
    return binary_backend.BinaryBackend


@pytest.fixture(scope="session")
def hip():
    """The device backend; a GPU test that reaches this without the HIP library fails loudly."""
    from nx_amd.backend import HipNxBackend
    return HipNxBackend
