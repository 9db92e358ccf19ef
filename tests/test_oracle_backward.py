"""Pins the backward half of the CPU checker: _ReduceSum and the autograd step of
MatrixMul, MatrixMulBatched and MulAndShift (oracle/nts_oracle.c).

Evidence: the known answers of the reference's TReduceSum; the gradients the COMPILED
reference leaves behind (live where oracle/_ref is built, and as the committed fixture
tests/golden/ref_generated_backward.npz everywhere), bit for bit; and the calculus: for
E = sum(dedc * c), dE/da and dE/db have closed forms in double precision, and a central
finite difference of the FORWARD checker must agree with them.
"""
import itertools

import numpy as np
import pytest

from oracle.binding import X_NOTRANS, X_TRANS, bmm_shape, mm_shape


def op(x, trans):
    return np.swapaxes(x, -1, -2) if trans == X_TRANS else x


def unop(g, trans):
    """Gradient with respect to the stored operand from the gradient with respect to op(operand)."""
    return np.swapaxes(g, -1, -2) if trans == X_TRANS else g


def closed_form(a, ta, b, tb, dedc, alpha):
    A, B, G = op(a.astype(np.float64), ta), op(b.astype(np.float64), tb), dedc.astype(np.float64)
    return unop(alpha * (G @ np.swapaxes(B, -1, -2)), ta), unop(alpha * (np.swapaxes(A, -1, -2) @ G), tb)


# ---- _ReduceSum ----------------------------------------------------------------

def test_reduce_sum_known_answers_of_the_reference(oracle):
    # TReduceSum.cpp:36-99 (case 1) and :632-667 (case 7)
    s = np.array([[0, 1, 2, 3], [4, 5, 6, 7]], np.float32)
    assert np.array_equal(oracle.reduce_sum(s, 0), np.array([4, 6, 8, 10], np.float32))
    assert np.array_equal(oracle.reduce_sum(s, 1), np.array([6, 22], np.float32))
    assert np.array_equal(oracle.reduce_sum(np.array([0, 1, 2, 3], np.float32), 0), np.float32(6))
    # cases 2-6 (:172-616) reduce tensors of ones along dimension 1 and expect that dimension's
    # size; same construction at sizes that finish quickly, covering the three code paths
    for shape in ((50, 1024), (1000, 50), (5, 4096), (20, 100, 32), (50, 1000, 5)):
        got = oracle.reduce_sum(np.ones(shape, np.float32), 1)
        assert np.array_equal(got, np.full(shape[:1] + shape[2:], shape[1], np.float32)), shape


def test_reduce_sum_fixture(oracle, generated_backward):
    names = generated_backward.of_kind("reduce_sum")
    assert len(names) == 9
    for name in names:
        d = generated_backward.case(name)
        got = oracle.reduce_sum(d["x"], int(d["params"][0]))
        assert np.array_equal(got, d["y"]), name
        assert np.allclose(got, d["x"].astype(np.float64).sum(int(d["params"][0])), rtol=0, atol=2e-5), name


def test_reduce_sum_against_compiled_reference(oracle, reference):
    rng = np.random.default_rng(11)
    for shape, dim in [((13, 9), 0), ((13, 9), 1), ((40, 256), 0), ((40, 256), 1), ((3, 64, 5), 1), ((3, 7, 96), 2),
                       ((3, 7, 96), 0), ((2, 3, 4, 32), 3), ((2, 3, 4, 32), 1), ((1, 33), 1), ((300, 31), 0)]:
        x = rng.standard_normal(shape).astype(np.float32)
        assert np.array_equal(oracle.reduce_sum(x, dim), reference.reduce_sum(x, dim)), (shape, dim)


# ---- GradMatrixMul / GradMatrixMulBatched -------------------------------------------

def test_grad_fixtures(oracle, generated_backward):
    n = 0
    for name in generated_backward.of_kind("grad_matmul"):
        d = generated_backward.case(name)
        ta, tb = (int(v) for v in d["params"])
        deda, dedb = oracle.grad_matmul(d["a"], ta, d["b"], tb, d["dedc"], float(d["scal"][0]),
                                        d["deda0"].copy(), d["dedb0"].copy())
        assert np.array_equal(deda, d["deda"]) and np.array_equal(dedb, d["dedb"]), name
        n += 1
    for name in generated_backward.of_kind("grad_matmul_batched"):
        d = generated_backward.case(name)
        ta, tb = (int(v) for v in d["params"])
        deda, dedb = oracle.grad_matmul_batched(d["a"], ta, d["b"], tb, d["dedc"], float(d["scal"][0]),
                                                d["deda0"].copy(), d["dedb0"].copy())
        assert np.array_equal(deda, d["deda"]) and np.array_equal(dedb, d["dedb"]), name
        n += 1
    assert n == 14


@pytest.mark.parametrize("ta,tb", list(itertools.product((X_NOTRANS, X_TRANS), repeat=2)))
def test_grad_matmul_closed_form_and_compiled_reference(oracle, ta, tb, request):
    rng = np.random.default_rng(5 + 2 * ta + tb)
    M, K, N = 23, 31, 17
    a = rng.standard_normal((K, M) if ta == X_TRANS else (M, K)).astype(np.float32)
    b = rng.standard_normal((N, K) if tb == X_TRANS else (K, N)).astype(np.float32)
    dedc = rng.standard_normal((M, N)).astype(np.float32)
    deda0 = rng.standard_normal(a.shape).astype(np.float32)
    dedb0 = rng.standard_normal(b.shape).astype(np.float32)
    deda, dedb = oracle.grad_matmul(a, ta, b, tb, dedc, 0.6, deda0.copy(), dedb0.copy())
    ea, eb = closed_form(a, ta, b, tb, dedc, 0.6)
    assert np.abs(deda - (deda0 + ea)).max() < 2e-5 * np.abs(ea).max()
    assert np.abs(dedb - (dedb0 + eb)).max() < 2e-5 * np.abs(eb).max()
    # a gradient that is not wanted is left alone
    only_b = oracle.grad_matmul(a, ta, b, tb, dedc, 0.6, None, dedb0.copy())
    assert only_b[0] is None and np.array_equal(only_b[1], dedb)
    from oracle.binding import Reference
    if Reference.available():
        ra, rb, _ = Reference().grad(0, a, ta, b, tb, dedc, 0.6, deda0.copy(), dedb0.copy())
        assert np.array_equal(ra, deda) and np.array_equal(rb, dedb)


def test_grad_matmul_matches_a_finite_difference_of_the_forward_checker(oracle):
    """E(a, b) = sum(dedc * matmul(a, b)): nudging one element of a or b by +-h changes E by
    2 h times the gradient, up to fp32 rounding of the forward products."""
    rng = np.random.default_rng(2)
    for ta, tb in itertools.product((X_NOTRANS, X_TRANS), repeat=2):
        M, K, N = 6, 5, 4
        a = rng.standard_normal((K, M) if ta == X_TRANS else (M, K)).astype(np.float32)
        b = rng.standard_normal((N, K) if tb == X_TRANS else (K, N)).astype(np.float32)
        dedc = rng.standard_normal((M, N)).astype(np.float32)
        deda, dedb = oracle.grad_matmul(a, ta, b, tb, dedc, 1.5, np.zeros_like(a), np.zeros_like(b))

        def E(a_, b_):
            return float((dedc.astype(np.float64) * oracle.matmul2d(a_, ta, b_, tb, None, 1.5)).sum())

        h = np.float32(2.0 ** -6)
        for which, grad in ((0, deda), (1, dedb)):
            for idx in [(0, 0), (1, 2), (grad.shape[0] - 1, grad.shape[1] - 1)]:
                ap, am, bp, bm = a.copy(), a.copy(), b.copy(), b.copy()
                (ap if which == 0 else bp)[idx] += h
                (am if which == 0 else bm)[idx] -= h
                fd = (E(ap, bp) - E(am, bm)) / (2.0 * float(h))
                assert abs(fd - grad[idx]) < 2e-3 * max(1.0, abs(fd)), (ta, tb, which, idx)


def test_grad_matmul_flatten_rule_and_todo(oracle, reference):
    rng = np.random.default_rng(4)
    a = rng.standard_normal((3, 4, 6)).astype(np.float32)
    b = rng.standard_normal((6, 5)).astype(np.float32)
    dedc = rng.standard_normal((3, 4, 5)).astype(np.float32)
    z = lambda x: np.zeros_like(x)
    deda, dedb = oracle.grad_matmul(a, X_NOTRANS, b, X_NOTRANS, dedc, 1.0, z(a), z(b))
    # the flatten rule is the 2-D rule on the folded tensors
    da2, db2 = oracle.grad_matmul(a.reshape(12, 6), X_NOTRANS, b, X_NOTRANS, dedc.reshape(12, 5), 1.0,
                                  np.zeros((12, 6), np.float32), z(b))
    assert np.array_equal(deda.reshape(12, 6), da2) and np.array_equal(dedb, db2)
    ra, rb, _ = reference.grad(0, a, X_NOTRANS, b, X_NOTRANS, dedc, 1.0, z(a), z(b))
    assert np.array_equal(ra, deda) and np.array_equal(rb, dedb)
    # a transposed N-D a has no backward in the reference ("TODO!")
    with pytest.raises(ValueError, match="TODO"):
        oracle.grad_matmul(np.zeros((3, 6, 4), np.float32), X_TRANS, b, X_NOTRANS, dedc, 1.0, None, z(b))


@pytest.mark.parametrize("ta,tb", list(itertools.product((X_NOTRANS, X_TRANS), repeat=2)))
def test_grad_matmul_batched(oracle, ta, tb):
    rng = np.random.default_rng(9 + 2 * ta + tb)
    M, K, N = 7, 11, 5
    a = rng.standard_normal((2, 3, K, M) if ta == X_TRANS else (2, 3, M, K)).astype(np.float32)
    b = rng.standard_normal((2, 3, N, K) if tb == X_TRANS else (2, 3, K, N)).astype(np.float32)
    dedc = rng.standard_normal(bmm_shape(a.shape, ta, b.shape, tb)).astype(np.float32)
    deda0 = rng.standard_normal(a.shape).astype(np.float32)
    dedb0 = rng.standard_normal(b.shape).astype(np.float32)
    deda, dedb = oracle.grad_matmul_batched(a, ta, b, tb, dedc, 0.125, deda0.copy(), dedb0.copy())
    ea, eb = closed_form(a, ta, b, tb, dedc, 0.125)
    assert np.abs(deda - (deda0 + ea)).max() < 2e-5 * np.abs(ea).max()
    assert np.abs(dedb - (dedb0 + eb)).max() < 2e-5 * np.abs(eb).max()
    from oracle.binding import Reference
    if Reference.available():
        ra, rb, _ = Reference().grad(1, a, ta, b, tb, dedc, 0.125, deda0.copy(), dedb0.copy())
        assert np.array_equal(ra, deda) and np.array_equal(rb, dedb)


# ---- GradMulAndShift ------------------------------------------------------------

def test_grad_mulandshift_fixture(oracle, generated_backward):
    names = generated_backward.of_kind("grad_mulandshift")
    assert len(names) == 6
    seen = set()
    for name in names:
        d = generated_backward.case(name)
        n = int(d["params"][0])
        seen.add(n == d["dedc"].ndim - 1)
        dedx, dedw, dedb = oracle.grad_mulandshift(d["x"], d["w"], d["dedc"], n, float(d["scal"][0]),
                                                   d["dedx0"].copy(), d["dedw0"].copy(), d["dedb0"].copy())
        assert np.array_equal(dedx, d["dedx"]) and np.array_equal(dedw, d["dedw"]) and np.array_equal(dedb, d["dedb"]), name
    assert seen == {True, False}


def test_grad_mulandshift_closed_form_and_compiled_reference(oracle):
    rng = np.random.default_rng(21)
    for sx, sw, sb in [((4, 6, 8), (8, 64), (64,)), ((10, 8), (8, 7), (7,)), ((5, 6, 8), (8, 7), (6,)),
                       ((4, 32, 8), (8, 32), (4,))]:
        x = rng.standard_normal(sx).astype(np.float32)
        w = rng.standard_normal(sw).astype(np.float32)
        bias = rng.standard_normal(sb).astype(np.float32)
        cshape = mm_shape(sx, X_NOTRANS, sw, X_NOTRANS)
        dedc = rng.standard_normal(cshape).astype(np.float32)
        n = oracle.broadcast_dim_index(cshape, sb)
        g0 = [rng.standard_normal(s).astype(np.float32) for s in (sx, sw, sb)]
        dedx, dedw, dedb = oracle.grad_mulandshift(x, w, dedc, n, 0.5, *[g.copy() for g in g0])
        G = dedc.astype(np.float64)
        ex = 0.5 * (G @ w.astype(np.float64).T)
        ew = 0.5 * (x.astype(np.float64).reshape(-1, sx[-1]).T @ G.reshape(-1, cshape[-1]))
        eb = G.sum(axis=tuple(i for i in range(len(cshape)) if i != n))
        assert np.abs(dedx - (g0[0] + ex)).max() < 2e-5 * np.abs(ex).max()
        assert np.abs(dedw - (g0[1] + ew)).max() < 2e-5 * np.abs(ew).max()
        assert np.abs(dedb - (g0[2] + eb)).max() < 2e-5 * np.abs(eb).max()
        from oracle.binding import Reference
        if Reference.available():
            rx, rw, rb = Reference().grad(2, x, X_NOTRANS, w, X_NOTRANS, dedc, 0.5, *[g.copy() for g in g0[:2]],
                                          bias=bias, dedbias=g0[2].copy())
            assert np.array_equal(rx, dedx) and np.array_equal(rw, dedw) and np.array_equal(rb, dedb)
