"""Runs the C++ program that drives the header-only AscendIndexIVFPQ / AscendIndexFlat wrappers."""
import os
import subprocess
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
BIN = os.path.join(ROOT, "tests", "cpp", "test_wrapper")


def _binary():
    if not os.path.exists(BIN):
        import __graft_entry__
        __graft_entry__.build()
    return BIN


def _this_process_uses_the_gpu():
    capi = sys.modules.get("indexsdk_amd._capi")
    return os.path.exists("/dev/kfd") and capi is not None and getattr(capi, "_lib", None) is not None


def test_wrapper_constructor_messages_host_only():
    """Constructor checks and their messages: host code only.  On a GPU box the program is a child of a process that
    may already hold the HIP runtime, which must not fork there (tests/conftest.py): then the GPU run that the
    session made at its start stands for this one -- it goes through the same checks first."""
    if _this_process_uses_the_gpu():
        from conftest import wrapper_gpu_run
        assert wrapper_gpu_run, "the session did not run the wrapper program before the library was loaded"
        assert wrapper_gpu_run["returncode"] == 0, wrapper_gpu_run["stdout"] + wrapper_gpu_run["stderr"]
        return
    out = subprocess.run([_binary()], capture_output=True, text=True, timeout=120)
    assert out.returncode == 0, out.stdout + out.stderr
    assert "wrapper test ok" in out.stdout


@pytest.mark.gpu
def test_wrapper_train_add_search_on_gpu():
    """train / add / search / copyFrom / copyTo through the C++ class hierarchy on the GPU: the run was made when the
    session started (tests/conftest.py); a missing run is a failure, not a skip."""
    from conftest import wrapper_gpu_run
    assert os.path.exists(BIN), "tests/cpp/test_wrapper has not been built (run __graft_entry__.build())"
    assert wrapper_gpu_run, "the session did not run the wrapper program (no /dev/kfd at session start?)"
    assert wrapper_gpu_run["returncode"] == 0, wrapper_gpu_run["stdout"] + wrapper_gpu_run["stderr"]
    assert "wrapper test ok" in wrapper_gpu_run["stdout"]
