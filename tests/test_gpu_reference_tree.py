"""Runs the reference-tree drop-ins on the GPU: oracle/_ref/test_reference_tree is built (where the reference tree is
mounted) from the patched backend dispatch, innova_amd/csrc/shim/oil_{backend,engines}_gfx950.cpp and
tests/cpp/test_reference_tree.cpp, and linked against the compiled reference's tensor and math code."""
import os
import subprocess

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
EXE = os.path.join(ROOT, "oracle", "_ref", "test_reference_tree")


@pytest.mark.gpu
def test_reference_tree_dropins():
    if not os.path.exists(EXE):
        pytest.skip("oracle/_ref/test_reference_tree not built (needs the reference tree: make -C oracle ref)")
    r = subprocess.run([EXE], capture_output=True, text=True, timeout=240)
    assert r.returncode == 0, r.stdout[-4000:] + r.stderr[-2000:]
    assert "all reference-tree checks passed" in r.stdout
