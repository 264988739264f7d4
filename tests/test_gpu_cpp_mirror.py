"""Runs the C++ host mirror of the reference interface (Qsa / QsaState) on the GPU."""
import os
import subprocess

import pytest

pytestmark = pytest.mark.gpu
BIN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "cpp", "qsa_mirror_test")


def test_cpp_mirror_of_the_reference_interface():
    assert os.path.exists(BIN), "tests/cpp/qsa_mirror_test is not built (run __graft_entry__.build())"
    proc = subprocess.run([BIN], capture_output=True, text=True, timeout=120)
    print(proc.stdout)
    assert proc.returncode == 0, proc.stdout + proc.stderr
    assert "all checks passed" in proc.stdout
