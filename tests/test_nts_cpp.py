"""Runs the C++ tests of the nts:: host layer (tests/cpp/nts_tests.cpp) on the GPU:
the reference's known-answer cases through _MatrixMul / MatrixMul / _MatrixMul2D /
_MatrixMulBatched / MulAndShift on device tensors, plus seeded cases against the oracle."""
import os
import subprocess

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
NTS_TESTS = os.path.join(ROOT, "tests", "cpp", "build", "nts_tests")


def built():
    """The test program, compiled now if the tree holds the libraries but not the program (g++ only; a few seconds)."""
    if not os.path.exists(NTS_TESTS):
        subprocess.run(["make", "-s", "-C", os.path.join(ROOT, "tests", "cpp")], capture_output=True, text=True, timeout=300)
    return os.path.exists(NTS_TESTS)


@pytest.mark.gpu
def test_nts_host_layer_on_gpu():
    assert built(), "tests/cpp/build/nts_tests is missing and does not build here: run __graft_entry__.build()"
    print("\n[gpu-case] nts_tests", flush=True)
    p = subprocess.run([NTS_TESTS], capture_output=True, text=True, timeout=120)
    print(p.stdout)
    print(p.stderr)
    assert p.returncode == 0, p.stdout + p.stderr
    assert "OK! Everything is good!" in p.stdout
    assert p.stdout.count("passed") == 23 and "FAILED" not in p.stdout


def test_host_tensors_reach_the_functions_the_host_tree_hands_in():
    """No GPU needed: host tensors go through nts::SetHostMatrixMul2D / SetHostSumDim (the reference's known
    answers on the CPU side of _MatrixMul2D, _MatrixMul, _MatrixMulBatched, MulAndShift)."""
    assert built(), "tests/cpp/build/nts_tests is missing and does not build here: run __graft_entry__.build()"
    p = subprocess.run([NTS_TESTS, "--host"], capture_output=True, text=True, timeout=60)
    assert p.returncode == 0 and "TestHostDispatch" in p.stdout and "passed" in p.stdout, p.stdout + p.stderr
