"""Runs the C++ program that drives the header-only AscendIndexIVFPQ / AscendIndexFlat wrappers."""
import os
import subprocess

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
BIN = os.path.join(ROOT, "tests", "cpp", "test_wrapper")


def _binary():
    if not os.path.exists(BIN):
        import __graft_entry__
        __graft_entry__.build()
    return BIN


def _skip_if_this_process_uses_the_gpu():
    """The program runs as a child process.  A process that has initialised the HIP runtime must not fork on the
    GPU boxes these tests run on (the fork ends in a segmentation fault of the parent), so these tests only run
    while this process has not loaded the library yet -- as it has not when the files run in their usual order."""
    import sys
    capi = sys.modules.get("indexsdk_amd._capi")
    if os.path.exists("/dev/kfd") and capi is not None and getattr(capi, "_lib", None) is not None:
        pytest.skip("this process has already loaded the GPU library: run tests/test_cpp_wrapper.py first or alone")


def test_wrapper_constructor_messages_host_only():
    _skip_if_this_process_uses_the_gpu()
    out = subprocess.run([_binary()], capture_output=True, text=True, timeout=120)
    assert out.returncode == 0, out.stdout + out.stderr
    assert "wrapper test ok" in out.stdout


@pytest.mark.gpu
def test_wrapper_train_add_search_on_gpu(tmp_path):
    if not os.path.exists(BIN):
        pytest.skip("tests/cpp/test_wrapper has not been built (run __graft_entry__.build())")
    _skip_if_this_process_uses_the_gpu()
    out = subprocess.run([BIN, "gpu", str(tmp_path)], capture_output=True, text=True, timeout=300)
    assert out.returncode == 0, out.stdout + out.stderr
    assert "wrapper test ok" in out.stdout
