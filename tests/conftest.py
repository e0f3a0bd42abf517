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


WRAPPER_BIN = os.path.join(ROOT, "tests", "cpp", "test_wrapper")
# (returncode, stdout, stderr) of the C++ wrapper program's GPU run, made before this process touches the GPU
wrapper_gpu_run = {}


def pytest_sessionstart(session):
    """The C++ program that drives include/ascend/*.h runs as a child process, and on the GPU boxes a process that
    has initialised the HIP runtime must not fork (the parent ends in a segmentation fault; the cause is not known:
    the child does nothing but exec, and the same fork is harmless before the runtime is up).  So the program's GPU run
    is made here, once, before any test has loaded the library, and tests/test_cpp_wrapper.py asserts on what it
    left -- whatever order the files run in."""
    import subprocess
    import tempfile
    markexpr = session.config.getoption("-m", default="") or ""
    if "not gpu" in markexpr or not os.path.exists("/dev/kfd") or not os.path.exists(WRAPPER_BIN):
        return
    with tempfile.TemporaryDirectory() as tmp:
        try:
            out = subprocess.run([WRAPPER_BIN, "gpu", tmp], capture_output=True, text=True, timeout=300)
            wrapper_gpu_run.update(returncode=out.returncode, stdout=out.stdout, stderr=out.stderr)
        except subprocess.TimeoutExpired as e:
            wrapper_gpu_run.update(returncode=-1, stdout=str(e.stdout), stderr="timed out after 300 s")


@pytest.fixture(scope="session")
def oracle():
    from oracle import oracle as orc
    orc.build()
    return orc
