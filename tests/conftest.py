import ctypes
import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu on the GPU box)")


@pytest.fixture(scope="session")
def host():
    """The C++ host layer with the CPU oracle plugged in as the backend of CPU tensors."""
    import homura_amd
    from tests import oracle

    h = homura_amd.load_host()
    h.register_cpu_backend(oracle.backend_address())
    return h
