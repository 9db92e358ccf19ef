"""Runs the C++ tests of the nts:: host layer (tests/cpp/nts_tests.cpp) on the GPU:
the reference's known-answer cases through _MatrixMul / MatrixMul / _MatrixMul2D /
_MatrixMulBatched / MulAndShift on device tensors, plus seeded cases against the oracle."""
import os
import subprocess

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
NTS_TESTS = os.path.join(ROOT, "tests", "cpp", "build", "nts_tests")


@pytest.mark.gpu
def test_nts_host_layer_on_gpu():
    assert os.path.exists(NTS_TESTS), "build tests/cpp first (__graft_entry__.build())"
    print("\n[gpu-case] nts_tests", flush=True)
    p = subprocess.run([NTS_TESTS], capture_output=True, text=True, timeout=120)
    print(p.stdout)
    print(p.stderr)
    assert p.returncode == 0, p.stdout + p.stderr
    assert "OK! Everything is good!" in p.stdout
    assert p.stdout.count("passed") == 22 and "FAILED" not in p.stdout
