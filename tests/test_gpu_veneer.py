"""Runs the C++ test of the Cuda_Stream veneer (tests/cpp/test_veneer.cpp, built by
__graft_entry__.build()) on the GPU."""
import os
import subprocess

import pytest

pytestmark = pytest.mark.gpu
BIN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "cpp", "test_veneer")


def test_cpp_veneer(device):
    assert os.path.exists(BIN), "tests/cpp/test_veneer is not built (run __graft_entry__.build())"
    r = subprocess.run([BIN], capture_output=True, text=True, timeout=120)
    print(r.stdout, r.stderr)
    assert r.returncode == 0, r.stdout[-2000:]
