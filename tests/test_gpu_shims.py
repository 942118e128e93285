"""Runs the C++ drop-in layer's own test program (tests/cpp/test_shims.cpp, built by
make -C innova_amd/csrc) on the GPU."""
import os
import subprocess

import pytest

pytestmark = pytest.mark.gpu
ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def test_cpp_shims_program():
    exe = os.path.join(ROOT, "tests", "cpp", "test_shims")
    assert os.path.exists(exe), "tests/cpp/test_shims is not built (make -C innova_amd/csrc)"
    r = subprocess.run([exe], capture_output=True, text=True, timeout=120)
    assert r.returncode == 0, r.stdout[-3000:] + r.stderr[-2000:]
    assert "0 failures" in r.stdout
