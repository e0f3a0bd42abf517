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


def test_wrapper_constructor_messages_host_only():
    out = subprocess.run([_binary()], capture_output=True, text=True, timeout=120)
    assert out.returncode == 0, out.stdout + out.stderr
    assert "wrapper test ok" in out.stdout


@pytest.mark.gpu
def test_wrapper_train_add_search_on_gpu(tmp_path):
    if not os.path.exists(BIN):
        pytest.skip("tests/cpp/test_wrapper has not been built (run __graft_entry__.build())")
    out = subprocess.run([BIN, "gpu", str(tmp_path)], capture_output=True, text=True, timeout=300)
    assert out.returncode == 0, out.stdout + out.stderr
    assert "wrapper test ok" in out.stdout
