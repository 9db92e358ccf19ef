"""Pins the CPU checker (oracle/) before anything is compared against it.

Three kinds of evidence, none of which re-types the checker's own formula:
  * the known-answer vectors of the reference's own tests,
  * the outputs of the COMPILED reference: live where oracle/_ref is built,
    and as the committed fixture tests/golden/ref_generated.npz everywhere,
  * what the mathematics fixes: double-precision products, exactness cases,
    transposition and scaling identities.
"""
import itertools

import numpy as np
import pytest

from oracle.binding import X_NOTRANS, X_TRANS, bmm_shape, mm_shape

T = {X_NOTRANS: "n", X_TRANS: "t"}


def op(x, trans):
    return np.swapaxes(x, -1, -2) if trans == X_TRANS else x


def f64(a, ta, b, tb, alpha=1.0, beta=0.0, c=None):
    r = alpha * (op(a.astype(np.float64), ta) @ op(b.astype(np.float64), tb))
    if beta != 0:
        r = r + beta * c.astype(np.float64)
    return r


# ---- the reference's own known answers ------------------------------------

def test_known_answers(oracle, known_answers):
    assert len(known_answers) == 12
    for case in known_answers:
        a = np.array(case["a"], np.float32)
        b = np.array(case["b"], np.float32)
        ans = np.array(case["answer"], np.float32)
        if case["op"] == "matmul2d":
            got = oracle.matmul2d(a, case["transA"], b, case["transB"])
        elif case["op"] == "matmul":
            got = oracle.matmul(a, case["transA"], b, case["transB"])
        elif case["op"] == "matmul_batched":
            got = oracle.matmul_batched(a, case["transA"], b, case["transB"])
        else:
            got = oracle.sumdim(a, b, case["n"], case["beta"])
        assert got.shape == ans.shape, case["name"]
        assert oracle.check_data(got, ans, 1e-4), case["name"]
        assert np.array_equal(got, ans), case["name"]       # small integers: exact


def test_sumdim_case3_of_the_reference(oracle):
    # TSumDim.cpp:257-330: (20, 40, 4000) zeros + ones(40) along dim 1 = ones
    a = np.zeros((20, 40, 400), np.float32)
    b = np.ones((40,), np.float32)
    assert np.array_equal(oracle.sumdim(a, b, 1), np.ones_like(a))


# ---- the compiled reference, live ------------------------------------------

def test_reference_passes_its_own_tests(reference):
    assert reference.run_matmul_tests() == 31


def test_reference_enum_values(reference):
    v = reference.enum_values()
    assert (v["X_TRANS"], v["X_NOTRANS"], v["X_FLOAT"], v["X_FLOAT16"]) == (0, 1, 2, 3)
    assert v["sizeof_XTensor"] == 400


@pytest.mark.parametrize("ta,tb", list(itertools.product((X_NOTRANS, X_TRANS), repeat=2)))
def test_matmul2d_bit_exact_with_reference(oracle, reference, ta, tb):
    for (M, N, K), (alpha, beta) in itertools.product(((37, 29, 53), (64, 64, 128), (1, 5, 300), (130, 3, 1)),
                                                      ((1.0, 0.0), (0.5, 1.0), (1.0, 1.0), (0.7, 0.3), (2.0, 0.0))):
        a = oracle.uniform((K, M) if ta == X_TRANS else (M, K), 11 * M + K)
        b = oracle.normal((N, K) if tb == X_TRANS else (K, N), 13 * N + K)
        c0 = oracle.uniform((M, N), 17)
        mine = oracle.matmul2d(a, ta, b, tb, c0.copy(), alpha, beta)
        theirs = reference.matmul2d(a, ta, b, tb, c0.copy(), alpha, beta)
        assert np.array_equal(mine, theirs), (M, N, K, alpha, beta)


def test_nd_and_batched_bit_exact_with_reference(oracle, reference):
    cases = [((3, 2, 3), X_NOTRANS, (3, 4), X_NOTRANS), ((4, 5, 6), X_TRANS, (5, 7), X_NOTRANS),
             ((3, 2, 3), X_NOTRANS, (2, 3, 2), X_NOTRANS), ((2, 4, 3), X_TRANS, (3, 5, 4), X_TRANS),
             ((2, 2, 3, 4), X_NOTRANS, (7, 4), X_TRANS)]
    for sa, ta, sb, tb in cases:
        a = oracle.uniform(sa, 5)
        b = oracle.uniform(sb, 6)
        c0 = oracle.uniform(mm_shape(sa, ta, sb, tb), 7)
        for alpha, beta in ((1.0, 0.0), (0.3, 1.0)):
            assert np.array_equal(oracle.matmul(a, ta, b, tb, c0.copy(), alpha, beta),
                                  reference.matmul(a, ta, b, tb, c0.copy(), alpha, beta))
        c, shape = reference.matmul_alloc(a, ta, b, tb, 1.0)
        assert shape == mm_shape(sa, ta, sb, tb)
        assert np.array_equal(c, oracle.matmul(a, ta, b, tb))
    for sa, ta, sb, tb in [((4, 6, 5), X_NOTRANS, (4, 7, 5), X_TRANS), ((2, 3, 5, 6), X_TRANS, (2, 3, 5, 4), X_NOTRANS)]:
        a = oracle.uniform(sa, 8)
        b = oracle.uniform(sb, 9)
        c0 = oracle.uniform(bmm_shape(sa, ta, sb, tb), 10)
        assert np.array_equal(oracle.matmul_batched(a, ta, b, tb, c0.copy(), 0.125, 1.0),
                              reference.matmul_batched(a, ta, b, tb, c0.copy(), 0.125, 1.0))


def test_broadcast_dim_index_against_reference(oracle, reference):
    dims = (1, 2, 3, 4)
    for ao, bo in itertools.product((1, 2, 3), repeat=2):
        for ashape in itertools.product(dims, repeat=ao):
            for bshape in itertools.product(dims, repeat=bo):
                assert oracle.broadcast_dim_index(ashape, bshape) == reference.broadcast_dim_index(ashape, bshape)


def test_mulandshift_bit_exact_with_reference(oracle, reference):
    x = oracle.uniform((4, 6, 10), 21)
    w = oracle.normal((10, 8), 22, 0, 0.02)
    for bshape in ((8,), (1, 8), (6,), (4, 1, 1)):
        bias = oracle.normal(bshape, 23, 0, 0.02)
        mine, n = oracle.mulandshift(x, w, bias, 0.5)
        assert np.array_equal(mine, reference.mulandshift(x, w, bias, 0.5))
    wt = np.ascontiguousarray(w.T)
    bias = oracle.normal((8,), 24)
    mine, n = oracle.mulandshift(x, wt, bias, 1.0, X_NOTRANS, X_TRANS)
    assert n == 2
    assert np.array_equal(mine, reference.mulandshift(x, wt, bias, 1.0, X_NOTRANS, X_TRANS))


# ---- the compiled reference, as committed fixtures --------------------------

def test_generated_fixture_products(oracle, generated):
    for kind, fn in (("matmul2d", oracle.matmul2d), ("matmul", oracle.matmul), ("matmul_batched", oracle.matmul_batched)):
        names = generated.of_kind(kind)
        assert names
        for name in names:
            d = generated.case(name)
            ta, tb = (int(v) for v in d["params"])
            alpha, beta = (float(v) for v in d["scal"])
            got = fn(d["a"], ta, d["b"], tb, d["c0"].copy(), alpha, beta)
            assert got.shape == d["c"].shape, name
            assert np.array_equal(got, d["c"]), name
            if "calloc" in d:
                assert np.array_equal(fn(d["a"], ta, d["b"], tb, None, alpha, 0.0), d["calloc"]), name


def test_generated_fixture_broadcast_dim_index(oracle, generated):
    table = generated.case("broadcast_dim_index")["table"]
    assert len(table) > 1000
    for row in table:
        ao, bo = int(row[3]), int(row[7])
        assert oracle.broadcast_dim_index(tuple(row[:ao]), tuple(row[4:4 + bo])) == int(row[8])


def test_generated_fixture_mulandshift(oracle, generated):
    names = generated.of_kind("mulandshift")
    assert len(names) >= 10
    dims_hit = set()
    for name in names:
        d = generated.case(name)
        ov, tx, tw = (int(v) for v in d["params"])
        got, n = oracle.mulandshift(d["x"], d["w"], d["bias"], float(d["scal"][0]), tx, tw)
        assert np.array_equal(got, d["c"]), name
        dims_hit.add(n == got.ndim - 1)
    assert dims_hit == {True, False}      # both the last-dimension and an earlier-dimension bias occur


# ---- what the mathematics fixes ---------------------------------------------

@pytest.mark.parametrize("ta,tb", list(itertools.product((X_NOTRANS, X_TRANS), repeat=2)))
def test_against_double_precision(oracle, ta, tb):
    M, N, K = 37, 29, 53
    a = oracle.uniform((K, M) if ta == X_TRANS else (M, K), 1)
    b = oracle.uniform((N, K) if tb == X_TRANS else (K, N), 2)
    c0 = oracle.uniform((M, N), 3)
    for alpha, beta in ((1.0, 0.0), (0.5, 1.0), (-1.5, 0.25)):
        got = oracle.matmul2d(a, ta, b, tb, c0.copy(), alpha, beta)
        assert np.abs(got - f64(a, ta, b, tb, alpha, beta, c0)).max() < 2e-5


def test_exactness_cases(oracle):
    # K = 1 outer product and small integers: every fp32 operation is exact
    u = np.arange(1, 8, dtype=np.float32).reshape(7, 1)
    v = np.arange(-3, 6, dtype=np.float32).reshape(1, 9)
    assert np.array_equal(oracle.matmul2d(u, X_NOTRANS, v, X_NOTRANS), u @ v)
    rng = np.random.default_rng(0)
    a = rng.integers(-8, 9, (33, 65)).astype(np.float32)
    b = rng.integers(-8, 9, (65, 17)).astype(np.float32)
    exact = (a.astype(np.int64) @ b.astype(np.int64)).astype(np.float32)
    for ta, tb in itertools.product((X_NOTRANS, X_TRANS), repeat=2):
        aa = np.ascontiguousarray(a.T) if ta == X_TRANS else a
        bb = np.ascontiguousarray(b.T) if tb == X_TRANS else b
        assert np.array_equal(oracle.matmul2d(aa, ta, bb, tb), exact)
    # an identity operand reproduces the other one
    x = oracle.uniform((12, 12), 4)
    eye = np.eye(12, dtype=np.float32)
    assert np.array_equal(oracle.matmul2d(x, X_NOTRANS, eye, X_NOTRANS), x)
    assert np.array_equal(oracle.matmul2d(eye, X_TRANS, x, X_TRANS), x.T)


def test_transposition_identity(oracle):
    # (A B)^T = B^T A^T: the TT product of the swapped operands is the transpose, bit for bit
    a = oracle.uniform((21, 34), 5)
    b = oracle.uniform((34, 13), 6)
    c = oracle.matmul2d(a, X_NOTRANS, b, X_NOTRANS)
    ct = oracle.matmul2d(b, X_TRANS, a, X_TRANS)
    assert np.array_equal(ct, c.T)
    # and the four layouts of one product agree
    c2 = oracle.matmul2d(np.ascontiguousarray(a.T), X_TRANS, np.ascontiguousarray(b.T), X_TRANS)
    assert np.array_equal(c2, c)


def test_scaling_and_accumulation(oracle):
    a = oracle.uniform((16, 40), 7)
    b = oracle.uniform((40, 24), 8)
    c1 = oracle.matmul2d(a, X_NOTRANS, b, X_NOTRANS)
    # alpha = 2 only shifts exponents
    assert np.array_equal(oracle.matmul2d(a, X_NOTRANS, b, X_NOTRANS, None, 2.0, 0.0), 2 * c1)
    # beta = 1 on top of the product itself doubles it
    assert np.array_equal(oracle.matmul2d(a, X_NOTRANS, b, X_NOTRANS, c1.copy(), 1.0, 1.0), 2 * c1)
    # beta = 0: whatever c held never reaches the result
    junk = np.full((16, 24), np.nan, np.float32)
    junk[::2] = np.inf
    assert np.array_equal(oracle.matmul2d(a, X_NOTRANS, b, X_NOTRANS, junk, 1.0, 0.0), c1)


def test_batched_and_flatten_equivalences(oracle):
    a = oracle.uniform((3, 4, 10, 6), 9)
    b = oracle.uniform((3, 4, 6, 5), 10)
    c = oracle.matmul_batched(a, X_NOTRANS, b, X_NOTRANS, None, 0.5)
    for i, j in itertools.product(range(3), range(4)):
        assert np.array_equal(c[i, j], oracle.matmul2d(a[i, j].copy(), X_NOTRANS, b[i, j].copy(), X_NOTRANS, None, 0.5))
    # N-D a against one matrix: the flattened product equals the per-block products
    w = oracle.uniform((6, 7), 11)
    flat = oracle.matmul(a, X_NOTRANS, w, X_NOTRANS)
    assert flat.shape == (3, 4, 10, 7)
    for i, j in itertools.product(range(3), range(4)):
        assert np.array_equal(flat[i, j], oracle.matmul2d(a[i, j].copy(), X_NOTRANS, w, X_NOTRANS))
    # N-D x N-D: block (p, q) of the result is a_p b_q
    x = oracle.uniform((2, 5, 3), 12)
    y = oracle.uniform((4, 3, 6), 13)
    z = oracle.matmul(x, X_NOTRANS, y, X_NOTRANS)
    assert z.shape == (2, 4, 5, 6)
    for p, q in itertools.product(range(2), range(4)):
        assert np.array_equal(z[p, q], oracle.matmul2d(x[p].copy(), X_NOTRANS, y[q].copy(), X_NOTRANS))


def test_shape_errors(oracle):
    a = np.zeros((3, 4), np.float32)
    with pytest.raises(ValueError):
        oracle.matmul2d(a, X_NOTRANS, np.zeros((5, 2), np.float32), X_NOTRANS)
    with pytest.raises(ValueError):
        oracle.matmul_batched(np.zeros((2, 3, 4), np.float32), X_NOTRANS, np.zeros((3, 4, 2), np.float32), X_NOTRANS)
    with pytest.raises(ValueError):       # a bias of the result's own shape: the reference aborts ("TODO!")
        oracle.mulandshift(a, np.zeros((4, 2), np.float32), np.zeros((3, 2), np.float32))


def test_mulandshift_is_product_plus_broadcast(oracle):
    x = oracle.uniform((5, 6, 8), 14)
    w = oracle.normal((8, 9), 15, 0, 0.02)
    bias = oracle.normal((9,), 16, 0, 0.02)
    got, n = oracle.mulandshift(x, w, bias, 1.0)
    assert n == 2
    assert np.array_equal(got, oracle.matmul(x, X_NOTRANS, w, X_NOTRANS) + bias)
    bias6 = oracle.normal((6,), 17)
    got, n = oracle.mulandshift(x, w, bias6, 1.0)
    assert n == 1
    assert np.array_equal(got, oracle.matmul(x, X_NOTRANS, w, X_NOTRANS) + bias6[None, :, None])
    scalar = np.array(0.25, np.float32)
    got, n = oracle.mulandshift(x, w, scalar, 1.0)
    assert np.array_equal(got, oracle.matmul(x, X_NOTRANS, w, X_NOTRANS) + np.float32(0.25))


# ---- helpers of the checker --------------------------------------------------

def test_comparator(oracle):
    assert oracle.is_float_equal(1.0, 1.0, 1e-4)
    assert oracle.is_float_equal(1.0, 1.00005, 1e-4)           # absolute branch
    assert oracle.is_float_equal(1e6, 1e6 + 50, 1e-4)          # relative branch
    assert not oracle.is_float_equal(1.0, 1.01, 1e-4)
    assert not oracle.is_float_equal(1e6, 1e6 + 500, 1e-4)
    assert not oracle.is_float_equal(float("nan"), float("nan"), 1e-4)


def test_half_conversion_against_numpy(oracle):
    bits = np.arange(65536, dtype=np.uint16)
    mine = oracle.from_f16_bits(bits)
    theirs = bits.view(np.float16).astype(np.float32)
    assert np.array_equal(mine.view(np.uint32)[~np.isnan(theirs)], theirs.view(np.uint32)[~np.isnan(theirs)])
    assert np.isnan(mine[np.isnan(theirs)]).all()
    # every finite half survives the round trip
    finite = np.isfinite(theirs)
    assert np.array_equal(oracle.to_f16_bits(theirs[finite]), bits[finite])
    # round-to-nearest-even on random floats, sub-normals, ties and the overflow edge
    rng = np.random.default_rng(1)
    x = np.concatenate([
        rng.standard_normal(200000).astype(np.float32) * np.float32(0.02),
        (rng.standard_normal(50000) * 1e-6).astype(np.float32),
        (rng.standard_normal(50000) * 3e4).astype(np.float32),
        np.array([65504, 65519.996, 65520, 7e4, 2.0 ** -24, 2.0 ** -25, 2.0 ** -25 * 1.0000001, 2.0 ** -14,
                  1 + 2.0 ** -11, 1 + 3 * 2.0 ** -11, 0.0, -0.0, np.inf, -np.inf], np.float32),
    ])
    with np.errstate(over="ignore"):
        assert np.array_equal(oracle.to_f16_bits(x), x.astype(np.float16).view(np.uint16))
    assert np.isnan(oracle.from_f16_bits(oracle.to_f16_bits(np.array([np.nan], np.float32)))).all()


def test_seeded_fills(oracle):
    u = oracle.uniform((100000,), 42)
    assert np.array_equal(u, oracle.uniform((100000,), 42))
    assert not np.array_equal(u, oracle.uniform((100000,), 43))
    assert -1 <= u.min() and u.max() < 1 and abs(u.mean()) < 0.01 and abs(u.var() - 1 / 3) < 0.01
    g = oracle.normal((100001,), 42, 0.0, 0.02)
    assert abs(g.mean()) < 3e-4 and abs(g.std() - 0.02) < 3e-4
    # first values of the stream, so that a change of generator cannot go unnoticed
    assert np.array_equal(oracle.uniform((3,), 1), np.array([0.13312314450740814, 0.4915635287761688, 0.9420055150985718], np.float32))
    assert np.allclose(oracle.normal((3,), 1), [-0.03426732122898102, -1.2926084995269775, -2.5000674724578857], rtol=1e-6)
