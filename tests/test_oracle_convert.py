"""Pins oracle_convert_data_type (oracle/nts_oracle.c), the checker of the data type conversion.

Evidence: the known answers of the reference's TConvertDataType (cases 1 and 2, and the product of
case 3 that runs conversion, half product and conversion back); the compiled reference's own host
code for float <-> int, bit for bit (its host code for half casts the value to an integer, a defect
that nothing follows); numpy's IEEE half for every one of the 65536 half patterns and for random,
sub-normal, tie, overflow and NaN inputs; round trips.
"""
import numpy as np
import pytest

from oracle.binding import X_FLOAT, X_FLOAT16, X_INT, X_NOTRANS


def test_known_answers_of_the_reference(oracle):
    # TConvertDataType.cpp:45-50 (float -> int), :120-125 (int -> float)
    a = np.array([[1.0, 2.0], [0.5, 4.0], [5.0, 6.0]], np.float32)
    assert np.array_equal(oracle.convert(a, X_INT), np.array([[1, 2], [0, 4], [5, 6]], np.int32))
    b = np.array([[1, 2], [0, 4], [5, 6]], np.int32)
    assert np.array_equal(oracle.convert(b, X_FLOAT), np.array([[1, 2], [0, 4], [5, 6]], np.float32))
    # case 3 (:214-243): convert both operands to half, multiply, convert back; every value is exact in half
    d1 = np.array([[1.0, -2.0], [0.5, -4.0], [0.0, 6.0]], np.float32)
    d2 = np.array([[1.0, 2.0, 3.0], [0.0, 4.0, 5.0]], np.float32)
    answer = np.array([[1.0, -6.0, -7.0], [0.5, -15.0, -18.5], [0.0, 24.0, 30.0]], np.float32)
    h1 = oracle.convert(oracle.convert(d1, X_FLOAT16), X_FLOAT)
    h2 = oracle.convert(oracle.convert(d2, X_FLOAT16), X_FLOAT)
    assert np.array_equal(h1, d1) and np.array_equal(h2, d2)              # the round trip of :231-235
    c = oracle.matmul2d(h1, X_NOTRANS, h2, X_NOTRANS)
    assert np.array_equal(oracle.convert(oracle.convert(c, X_FLOAT16), X_FLOAT), answer)


def test_float_int_against_compiled_reference(oracle, reference):
    rng = np.random.default_rng(3)
    x = np.concatenate([rng.standard_normal(1000) * 1000, rng.standard_normal(100) * 1e8, [0.0, -0.0, 0.99, -0.99, 2147483520.0,
                        -2147483648.0, 1e-30]]).astype(np.float32)
    assert np.array_equal(oracle.convert(x, X_INT), reference.convert(x, X_INT))
    i = np.concatenate([rng.integers(-2**31, 2**31 - 1, 1000), [0, 1, -1, 2**24 + 1, 2**31 - 1, -2**31, 33554435]]).astype(np.int32)
    assert np.array_equal(oracle.convert(i, X_FLOAT), reference.convert(i, X_FLOAT))


def test_float_int_against_numpy_and_saturation(oracle):
    rng = np.random.default_rng(4)
    x = (rng.standard_normal(5000) * 1e5).astype(np.float32)
    assert np.array_equal(oracle.convert(x, X_INT), x.astype(np.int32))           # C cast: toward zero
    assert np.array_equal(oracle.convert(x, X_INT), np.trunc(x).astype(np.int32))
    i = rng.integers(-2**31, 2**31 - 1, 5000).astype(np.int32)
    assert np.array_equal(oracle.convert(i, X_FLOAT), i.astype(np.float32))       # round to nearest even
    edge = np.array([3e9, -3e9, np.inf, -np.inf, np.nan, 2147483648.0], np.float32)
    assert np.array_equal(oracle.convert(edge, X_INT),
                          np.array([2**31 - 1, -2**31, 2**31 - 1, -2**31, 0, 2**31 - 1], np.int32))


def test_half_against_numpy(oracle):
    # every half pattern widens exactly, and narrows back to itself (NaN payloads aside)
    bits = np.arange(65536, dtype=np.uint16)
    wide = oracle.convert(bits, X_FLOAT)
    ref = bits.view(np.float16).astype(np.float32)
    assert np.array_equal(wide.view(np.uint32), ref.view(np.uint32))
    back = oracle.convert(wide, X_FLOAT16)
    finite = ~np.isnan(ref)
    assert np.array_equal(back[finite], bits[finite]) and np.isnan(back[~finite].view(np.float16)).all()
    # narrowing: random magnitudes over the whole half range and beyond, ties, sub-normals, overflow
    rng = np.random.default_rng(5)
    x = (rng.standard_normal(200000) * np.exp(rng.uniform(-20, 12, 200000))).astype(np.float32)
    ties = (np.arange(2048, 4096, dtype=np.float32) + 0.5)                        # halfway between two halves
    sub = (rng.uniform(-1, 1, 1000) * 6.2e-5).astype(np.float32)
    big = np.array([65504.0, 65519.9, 65520.0, 1e6, -65520.0, np.inf, -np.inf], np.float32)
    for v in (x, ties, sub, big):
        with np.errstate(over="ignore"):
            assert np.array_equal(oracle.convert(v, X_FLOAT16), v.astype(np.float16).view(np.uint16))


def test_equal_types_and_refused_pairs(oracle):
    x = np.array([1.5, 2.5], np.float32)
    assert np.array_equal(oracle.convert(x, X_FLOAT), x)
    with pytest.raises(ValueError):
        oracle.convert(np.array([1, 2], np.int32), X_FLOAT16)                     # ConvertDataType.cu:134-136
    with pytest.raises(ValueError):
        oracle.convert(np.array([1, 2], np.uint16), X_INT)
