"""Pins oracle_rectify (oracle/nts_oracle.c), the checker of the activation that the fused linear
layer applies: the known answers of the reference's TRectify, the compiled reference's _Rectify
bit for bit, and the definition max(0, x) with its two special values."""
import numpy as np


def test_known_answers_of_the_reference(oracle):
    # TRectify.cpp:43-46 (case 1) and the forward half of case 2 (:125-127: x, then max(0, x))
    x = np.array([[0.0, -1.0, 2.0], [3.0, -4.0, -5.0]], np.float32)
    assert np.array_equal(oracle.rectify(x), np.array([[0.0, 0.0, 2.0], [3.0, 0.0, 0.0]], np.float32))
    x = np.array([[-1.0, 1.0, 2.0], [3.0, -4.0, -5.0]], np.float32)
    assert np.array_equal(oracle.rectify(x), np.maximum(x, 0))


def test_against_compiled_reference_and_definition(oracle, reference):
    x = oracle.normal((1000,), 77, 0.0, 3.0)
    x[:4] = [0.0, -0.0, np.nan, -np.inf]
    got, ref = oracle.rectify(x), reference.rectify(x)
    assert np.array_equal(got.view(np.uint32), ref.view(np.uint32))
    assert np.array_equal(got[4:], np.maximum(x[4:], 0))
    # x < 0 is false for a negative zero and for a NaN: both pass through
    assert got[0] == 0 and np.signbit(got[1]) and np.isnan(got[2]) and got[3] == 0
