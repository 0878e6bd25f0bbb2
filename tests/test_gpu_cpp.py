"""Runs the C++ host-layer tests (tests/cpp/test_nn.cpp over include/agpu_nn.hpp) on the GPU."""
import os
import subprocess

import pytest

pytestmark = pytest.mark.gpu
ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def test_cpp_nn_layer(dev):
    exe = os.path.join(ROOT, "tests", "cpp", "test_nn")
    assert os.path.exists(exe), "tests/cpp/test_nn is not built; run __graft_entry__.build()"
    r = subprocess.run([exe], capture_output=True, text=True, timeout=110)
    print(r.stdout)
    print(r.stderr)
    assert r.returncode == 0, r.stdout[-2000:]
    assert "PASSED: 0 failed" in r.stdout
