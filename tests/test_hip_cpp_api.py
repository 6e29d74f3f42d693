"""Runs the C++ tests of the C-ABI and of include/kvcm_hip.hpp (tests/cpp/test_cpp_api.cpp) on the GPU."""
import os
import subprocess

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
BINARY = os.path.join(ROOT, "tests", "cpp", "kvcm_cpp_tests")


@pytest.mark.gpu
def test_cpp_api_binary():
    assert os.path.exists(BINARY), "build it first: make -C tests/cpp (or python __graft_entry__.py)"
    proc = subprocess.run([BINARY], stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True, timeout=120)
    print(proc.stdout)
    assert proc.returncode == 0, proc.stdout
    assert "0 failed" in proc.stdout
