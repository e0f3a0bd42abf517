import os
import sys

import pytest

# The full-size tests generate their data with torch on the device.  A process can hold one HIP runtime:
# torch ships its own, and it has to be the one that is loaded first (the library then binds to it, as it
# does under bench.py); loaded after the library's, torch finds no device.
try:
    import torch  # noqa: F401
except ImportError:
    pass

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu on the GPU box)")


@pytest.fixture(scope="session")
def oracle():
    from oracle import oracle as orc
    orc.build()
    return orc
