"""Pins the attention half of the CPU checker: oracle_softmax and oracle_attention
(oracle/nts_oracle.c), the inference path of the transformer sample's attention
(Split, Scale, BMMul(q, k^T), Sum with the mask, Softmax, BMMul with v, Merge).

Evidence: the known answers of the reference's TSoftmax; the results of the COMPILED
reference's own operators (live where oracle/_ref is built, and as the committed fixture
tests/golden/ref_generated_attention.npz everywhere), bit for bit; and the mathematics:
the closed form in double precision, rows that sum to one, invariance under a shift of a
row, a one-key attention that returns v, uniform scores that return the mean of v, and a
mask that removes keys giving the same result as an attention without those keys.
"""
import numpy as np
import pytest


def softmax64(x):
    x = x.astype(np.float64)
    e = np.exp(x - x.max(-1, keepdims=True))
    return e / e.sum(-1, keepdims=True)


def attention64(q, k, v, heads, scale, mask=None):
    """out[b, l, h*dh:(h+1)*dh] = softmax(scale q_h k_h^T + mask[h, b]) v_h in double precision."""
    B, lq, H = q.shape
    lk = k.shape[1]
    dh = H // heads
    qh = q.astype(np.float64).reshape(B, lq, heads, dh).transpose(2, 0, 1, 3)
    kh = k.astype(np.float64).reshape(B, lk, heads, dh).transpose(2, 0, 1, 3)
    vh = v.astype(np.float64).reshape(B, lk, heads, dh).transpose(2, 0, 1, 3)
    s = scale * (qh @ kh.transpose(0, 1, 3, 2))
    if mask is not None:
        s = s + mask.astype(np.float64)
    p = softmax64(s)
    return (p @ vh).transpose(1, 2, 0, 3).reshape(B, lq, H)


# ---- softmax --------------------------------------------------------------------------

def test_softmax_known_answers_of_the_reference(oracle):
    # TSoftmax.cpp:44-47, compared as the test does (CheckData, 1e-4)
    x = np.array([[0.0, 1.0, 2.0], [0.5, 0.7, 1.4]], np.float32)
    answer = np.array([[0.0900, 0.2447, 0.6652], [0.2136, 0.2609, 0.5254]], np.float32)
    assert oracle.check_data(oracle.softmax(x), answer, 1e-4)


def test_softmax_fixture(oracle, generated_attention):
    names = generated_attention.of_kind("softmax")
    assert len(names) == 8
    for name in names:
        d = generated_attention.case(name)
        got = oracle.softmax(d["x"])
        assert np.array_equal(got, d["y"]), name
        assert np.abs(got - softmax64(d["x"])).max() <= 2e-6, name


def test_softmax_against_compiled_reference(oracle, reference):
    rng = np.random.default_rng(5)
    for shape, std in [((7, 5), 1.0), ((9, 32), 2.0), ((3, 4, 64), 4.0), ((5, 31), 10.0), ((2, 160), 1.0),
                       ((4, 1), 1.0), ((3, 100), 50.0)]:
        x = (rng.standard_normal(shape) * std).astype(np.float32)
        assert np.array_equal(oracle.softmax(x), reference.softmax(x)), shape
    # masked rows as the sample builds them: some scores at -1e9
    x = rng.standard_normal((6, 64)).astype(np.float32)
    x[:, 20:] += np.float32(-1e9)
    assert np.array_equal(oracle.softmax(x), reference.softmax(x))


def test_softmax_properties(oracle):
    x = oracle.normal((50, 77), 31, 0.0, 3.0)
    y = oracle.softmax(x)
    assert np.abs(y.sum(-1, dtype=np.float64) - 1).max() <= 1e-5
    assert (y >= 0).all() and (y <= 1).all()
    # a constant added to a row changes nothing: on inputs that are multiples of 2^-10 the shifted
    # inputs and their differences from the maximum are exact
    xq = np.round(x * 1024).astype(np.float32) / np.float32(1024)
    assert np.array_equal(oracle.softmax(xq + np.float32(64.0)), oracle.softmax(xq))
    # order is kept, equal inputs get equal outputs
    i = np.argsort(x[0])
    assert (np.diff(y[0][i]) >= 0).all()
    assert np.array_equal(oracle.softmax(np.full((3, 8), 7.0, np.float32)), np.full((3, 8), 0.125, np.float32))


# ---- attention ------------------------------------------------------------------------

def test_attention_fixture(oracle, generated_attention):
    names = generated_attention.of_kind("attention")
    assert len(names) == 9
    for name in names:
        d = generated_attention.case(name)
        heads, scale = int(d["params"][0]), float(d["scal"][0])
        mask = d.get("mask")
        got = oracle.attention(d["q"], d["k"], d["v"], heads, scale, mask)
        assert np.array_equal(got, d["out"]), name
        ref = attention64(d["q"], d["k"], d["v"], heads, scale, mask)
        assert np.abs(got - ref).max() <= 2e-5 * max(1.0, np.abs(ref).max()), name


def test_attention_against_compiled_reference(oracle, reference):
    for i, (B, lq, lk, H, nh, masked) in enumerate([(2, 6, 10, 16, 2, False), (1, 35, 33, 48, 3, True),
                                                     (3, 17, 96, 64, 4, True), (2, 3, 1, 8, 1, False)]):
        q, k, v = oracle.normal((B, lq, H), 70 + i), oracle.normal((B, lk, H), 80 + i), oracle.normal((B, lk, H), 90 + i)
        mask = None
        if masked:
            mask = np.where(oracle.uniform((nh, B, lq, lk), 100 + i, 0.0, 1.0) < 0.4, -1e9, 0.0).astype(np.float32)
            mask[..., -1] = 0.0
        scale = float(np.float32(1.0 / np.sqrt(H / nh)))
        assert np.array_equal(oracle.attention(q, k, v, nh, scale, mask), reference.attention(q, k, v, nh, scale, mask)), i


def test_attention_special_cases(oracle):
    B, lq, lk, H, nh = 2, 11, 13, 24, 3
    q, k, v = oracle.normal((B, lq, H), 1), oracle.normal((B, lk, H), 2), oracle.normal((B, lk, H), 3)
    # one key: the probabilities are exactly 1, every query row returns v's only row
    k1, v1 = np.ascontiguousarray(k[:, :1]), np.ascontiguousarray(v[:, :1])
    out = oracle.attention(q, k1, v1, nh, 0.3)
    assert np.array_equal(out, np.broadcast_to(v[:, :1], (B, lq, H)))
    # scale 0: uniform probabilities, the result is the mean of v's rows
    out = oracle.attention(q, k, v, nh, 0.0)
    assert np.abs(out - v.astype(np.float64).mean(1, keepdims=True)).max() <= 1e-6
    # a mask that removes keys 5.. equals attention over keys 0..4 (exp(-1e9 - max) is exactly 0)
    mask = np.zeros((nh, B, lq, lk), np.float32)
    mask[..., 5:] = -1e9
    full = oracle.attention(q, k, v, nh, 0.2, mask)
    cut = oracle.attention(q, np.ascontiguousarray(k[:, :5]), np.ascontiguousarray(v[:, :5]), nh, 0.2)
    assert np.abs(full - cut).max() <= 1e-6
    # heads are independent: head 1's columns depend on head 1's columns only
    q2 = q.copy()
    q2[..., :8] = 0
    out2 = oracle.attention(q2, k, v, nh, 0.2)
    out1 = oracle.attention(q, k, v, nh, 0.2)
    assert np.array_equal(out1[..., 8:], out2[..., 8:]) and not np.array_equal(out1[..., :8], out2[..., :8])
    # hidden size not divisible by the heads is refused
    with pytest.raises(ValueError):
        oracle.attention(q, k, v, 5, 0.2)


def test_attention_probs_against_compiled_reference_and_closed_form(oracle, reference):
    """The first half of the chain on its own: bit for bit against the reference's operators, rows sum to 1,
    the closed form in double precision, and consistency with the whole chain."""
    for i, (B, lq, lk, H, nh, masked) in enumerate([(2, 6, 10, 16, 2, False), (1, 35, 33, 48, 3, True), (2, 17, 96, 64, 4, True)]):
        q, k, v = oracle.normal((B, lq, H), 170 + i), oracle.normal((B, lk, H), 180 + i), oracle.normal((B, lk, H), 190 + i)
        mask = None
        if masked:
            mask = np.where(oracle.uniform((nh, B, lq, lk), 200 + i, 0.0, 1.0) < 0.4, -1e9, 0.0).astype(np.float32)
            mask[..., -1] = 0.0
        scale = float(np.float32(1.0 / np.sqrt(H / nh)))
        p = oracle.attention_probs(q, k, nh, scale, mask)
        assert np.array_equal(p, reference.attention_probs(q, k, nh, scale, mask)), i
        assert np.abs(p.sum(-1, dtype=np.float64) - 1).max() <= 1e-5
        dh = H // nh
        qh = q.astype(np.float64).reshape(B, lq, nh, dh).transpose(2, 0, 1, 3)
        kh = k.astype(np.float64).reshape(B, lk, nh, dh).transpose(2, 0, 1, 3)
        s = scale * (qh @ kh.transpose(0, 1, 3, 2)) + (mask if mask is not None else 0.0)
        assert np.abs(p - softmax64(s)).max() <= 2e-6
        # the whole chain is these probabilities times v, merged (in the oracle's own arithmetic: bit for bit)
        vh = np.ascontiguousarray(v.reshape(B, lk, nh, dh).transpose(2, 0, 1, 3))
        o = oracle.matmul_batched(p, 1, vh, 1)
        assert np.array_equal(o.transpose(1, 2, 0, 3).reshape(B, lq, H), oracle.attention(q, k, v, nh, scale, mask))
