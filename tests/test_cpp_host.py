"""Runs the host-only C++ tests of include/agpu_nn.hpp (tests/cpp/test_gpu_array_host.cpp): the life cycle of GpuArray
that needs no GPU, as the reference tests it (gpu_array.rs:434-514)."""
import os
import subprocess

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def test_gpu_array_host_life_cycle():
    exe = os.path.join(ROOT, "tests", "cpp", "test_gpu_array_host")
    assert os.path.exists(exe), "tests/cpp/test_gpu_array_host is not built; run __graft_entry__.build()"
    r = subprocess.run([exe], capture_output=True, text=True, timeout=60)
    assert r.returncode == 0, r.stdout + r.stderr
    assert "PASSED: 0 failed" in r.stdout
