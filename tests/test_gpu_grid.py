"""Parity of ntsamd_matrix_mul_batched_grid (products over matrices that stand inside larger tensors, with
their own leading dimensions and two batch strides) with the CPU oracle, through the C ABI.

The oracle multiplies each item on a contiguous copy (_MatrixMul2D semantics); what is under test is the
addressing: which elements the kernels read and write, and that they write nothing else (every result tensor
starts as a pattern that must survive outside the items).

Limits: fp32 normwise 1e-5 sqrt(K), fp16 1e-2.
"""
import numpy as np
import pytest

import niutensor_amd as nt
from niutensor_amd import X_NOTRANS, X_TRANS
from tolerance import assert_fp16, assert_fp32

pytestmark = pytest.mark.gpu


def torch_():
    import torch
    return torch


def dev(x, gpu):
    return torch_().from_numpy(np.ascontiguousarray(x)).to(gpu)


@pytest.fixture(autouse=True)
def name_the_case(request):
    print("\n[gpu-case] %s" % request.node.nodeid, flush=True)
    yield


def item(flat, n, m, ld, start):
    """View of the n x m matrix with rows ld apart that starts at element `start` of a flat array."""
    return np.lib.stride_tricks.as_strided(flat[start:], shape=(n, m), strides=(ld * flat.itemsize, flat.itemsize))


def grid_on_the_oracle(oracle, a, ta, lda, sa, b, tb, ldb, sb, c, ldc, sc, c0, c1, na, ma, nb, mb, nc, mc, alpha, beta):
    """The expected result tensor: every item through the oracle's 2-D product, the rest of c untouched."""
    a32, b32 = a.astype(np.float32).ravel(), b.astype(np.float32).ravel()
    want = c.astype(np.float32).ravel().copy()
    for i1 in range(c1):
        for i0 in range(c0):
            am = np.ascontiguousarray(item(a32, na, ma, lda, i0 * sa[0] + i1 * sa[1]))
            bm = np.ascontiguousarray(item(b32, nb, mb, ldb, i0 * sb[0] + i1 * sb[1]))
            cv = item(want, nc, mc, ldc, i0 * sc[0] + i1 * sc[1])
            cm = np.ascontiguousarray(cv)
            cv[...] = oracle.matmul2d(am, ta, bm, tb, c=cm, alpha=alpha, beta=beta)
    return want.reshape(c.shape)


def run_grid(gpu, a, ta, lda, sa, b, tb, ldb, sb, c, ldc, sc, c0, c1, na, ma, nb, mb, nc, mc, alpha, beta):
    torch = torch_()
    cd = dev(c, gpu)
    nt.matrix_mul_batched_grid(dev(a, gpu), ta, lda, sa, dev(b, gpu), tb, ldb, sb, cd, ldc, sc,
                               c0, c1, na, ma, nb, mb, nc, mc, alpha, beta)
    torch.cuda.synchronize()
    return cd.cpu().numpy()


@pytest.mark.parametrize("B,nh,lq,lk,dh,dtype", [
    (4, 8, 128, 128, 64, np.float32),      # the transformer's attention shape
    (3, 2, 100, 77, 32, np.float32),       # ragged lengths
    (2, 3, 33, 65, 20, np.float32),        # head width that is no multiple of the tile or of 8
    (1, 5, 7, 9, 3, np.float32),           # rows of the merged tensors at odd offsets
    (4, 8, 128, 128, 64, np.float16),
    (2, 3, 40, 72, 24, np.float16),        # multiples of 8: the fast path
    (2, 3, 33, 65, 20, np.float16),        # not: the generic kernel
])
def test_attention_context_on_merged_tensors(gpu, oracle, B, nh, lq, lk, dh, dtype):
    """out[b, :, h*dh:(h+1)*dh] = probs[h, b] . v[b, :, h*dh:(h+1)*dh]: BMMul(att, Split(v)) and the Merge
    after it (source/sample/transformer/submodel/Attention.cpp:235-242) without either copy."""
    H = nh * dh
    probs = oracle.uniform((nh, B, lq, lk), 11, 0.0, 1.0).astype(dtype)
    v = oracle.normal((B, lk, H), 12).astype(dtype)
    out = np.full((B, lq, H), 7.0, dtype=dtype)
    args = (probs, X_NOTRANS, lk, (lq * lk, B * lq * lk), v, X_NOTRANS, H, (lk * H, dh),
            out, H, (lq * H, dh), B, nh, lq, lk, lk, dh, lq, dh, 1.0, 0.0)
    got = run_grid(gpu, *args)
    want = grid_on_the_oracle(oracle, *args)
    # the same thing the long way round: Split, batched product, Merge
    vs = v.astype(np.float32).reshape(B, lk, nh, dh).transpose(2, 0, 1, 3)
    chain = np.matmul(probs.astype(np.float32), vs).transpose(1, 2, 0, 3).reshape(B, lq, H)
    np.testing.assert_allclose(want, chain, rtol=1e-4, atol=1e-4)
    if dtype == np.float32:
        assert_fp32(got, want, lk, what="context")
    else:
        assert_fp16(got, want, what="context")


@pytest.mark.parametrize("dtype", [np.float32, np.float16])
def test_scores_of_merged_queries_and_keys(gpu, oracle, dtype):
    """scores[h, b] = 0.125 * q[b, :, head h] . k[b, :, head h]^T: both operands read where they stand."""
    B, nh, lq, lk, dh = 3, 4, 50, 70, 16
    H = nh * dh
    q = oracle.normal((B, lq, H), 21).astype(dtype)
    k = oracle.normal((B, lk, H), 22).astype(dtype)
    s = np.zeros((nh, B, lq, lk), dtype=dtype)
    args = (q, X_NOTRANS, H, (lq * H, dh), k, X_TRANS, H, (lk * H, dh),
            s, lk, (lq * lk, B * lq * lk), B, nh, lq, dh, lk, dh, lq, lk, 0.125, 0.0)
    got = run_grid(gpu, *args)
    want = grid_on_the_oracle(oracle, *args)
    if dtype == np.float32:
        assert_fp32(got, want, dh, what="scores")
    else:
        assert_fp16(got, want, what="scores")


@pytest.mark.parametrize("dtype", [np.float32, np.float16])
def test_gradient_of_merged_values_accumulates(gpu, oracle, dtype):
    """dV[b, :, head h] += probs[h, b]^T . dOut[b, :, head h]: a transposed first operand and beta = 1,
    the step GradMatrixMulBatched takes for the second operand (source/network/XBackwardMath.cpp:1098-1170),
    on merged gradients."""
    B, nh, lq, lk, dh = 2, 3, 48, 40, 24
    H = nh * dh
    probs = oracle.uniform((nh, B, lq, lk), 31, 0.0, 1.0).astype(dtype)
    dout = oracle.normal((B, lq, H), 32).astype(dtype)
    dv = oracle.normal((B, lk, H), 33).astype(dtype)
    args = (probs, X_TRANS, lk, (lq * lk, B * lq * lk), dout, X_NOTRANS, H, (lq * H, dh),
            dv, H, (lk * H, dh), B, nh, lq, lk, lq, dh, lk, dh, 1.0, 1.0)
    got = run_grid(gpu, *args)
    want = grid_on_the_oracle(oracle, *args)
    if dtype == np.float32:
        assert_fp32(got, want, lq, what="dV")
    else:
        assert_fp16(got, want, what="dV")


def test_padding_between_and_around_the_items_is_left_alone(gpu, oracle):
    """Items narrower than their rows and further apart than their size: the gaps of c keep their pattern
    (exactly), and the gaps of a and b, filled with NaN, reach no result."""
    c0, c1, n, k, m = 3, 2, 37, 29, 21
    lda, ldb, ldc = k + 5, m + 3, m + 6
    sa = (n * lda + 11, c0 * (n * lda + 11) + 2)
    sb = (k * ldb + 4, c0 * (k * ldb + 4) + 6)
    sc = (n * ldc + 9, c0 * (n * ldc + 9) + 1)
    a = np.full(c1 * sa[1] + 64, np.nan, dtype=np.float32)
    b = np.full(c1 * sb[1] + 64, np.nan, dtype=np.float32)
    c = np.arange(c1 * sc[1] + 64, dtype=np.float32)
    for i1 in range(c1):
        for i0 in range(c0):
            item(a, n, k, lda, i0 * sa[0] + i1 * sa[1])[...] = oracle.normal((n, k), 40 + i0 + 10 * i1)
            item(b, k, m, ldb, i0 * sb[0] + i1 * sb[1])[...] = oracle.normal((k, m), 60 + i0 + 10 * i1)
    args = (a, X_NOTRANS, lda, sa, b, X_NOTRANS, ldb, sb, c, ldc, sc, c0, c1, n, k, k, m, n, m, 1.0, 0.0)
    got = run_grid(gpu, *args)
    want = grid_on_the_oracle(oracle, *args)
    inside = np.zeros(c.shape, dtype=bool)
    for i1 in range(c1):
        for i0 in range(c0):
            item(inside, n, m, ldc, i0 * sc[0] + i1 * sc[1])[...] = True
    assert np.array_equal(got[~inside], c[~inside])
    assert np.isfinite(got).all()
    assert_fp32(got[inside], want[inside], k, what="items")


def test_the_last_item_may_end_with_the_allocation(gpu, oracle):
    """The last head of the last row ends exactly where the tensor ends: nothing beyond it is read as data
    (a transposed operand's rows past K come back as zeros from the range check, not from memory)."""
    torch = torch_()
    B, nh, L, dh = 2, 4, 130, 20
    H = nh * dh
    x = oracle.normal((B, L, H), 71)
    y = oracle.normal((B, L, H), 72)
    # gram[h, b] = x[b, :, head h]^T . y[b, :, head h]: both operands MN-contiguous, k = L with a ragged last slab
    g = np.zeros((nh, B, dh, dh), dtype=np.float32)
    args = (x, X_TRANS, H, (L * H, dh), y, X_NOTRANS, H, (L * H, dh),
            g, dh, (dh * dh, B * dh * dh), B, nh, L, dh, L, dh, dh, dh, 1.0, 0.0)
    got = run_grid(gpu, *args)
    want = grid_on_the_oracle(oracle, *args)
    assert_fp32(got, want, L, what="gram")
    del torch


def test_argument_errors(gpu):
    torch = torch_()
    t = torch.zeros(4096, device=gpu)
    with pytest.raises(nt.NtsAmdError, match="leading dimension"):
        nt.matrix_mul_batched_grid(t, X_NOTRANS, 7, (64, 0), t, X_NOTRANS, 8, (64, 0), t, 8, (64, 0),
                                   2, 1, 8, 8, 8, 8, 8, 8)
    with pytest.raises(nt.NtsAmdError, match="overlap"):
        nt.matrix_mul_batched_grid(t, X_NOTRANS, 8, (64, 0), t, X_NOTRANS, 8, (64, 0), t, 16, (4, 128),
                                   2, 2, 8, 8, 8, 8, 8, 8)
    with pytest.raises(nt.NtsAmdError, match="overlap"):
        # heads side by side in a row, batches one row short of clearing them
        nt.matrix_mul_batched_grid(t, X_NOTRANS, 8, (64, 0), t, X_NOTRANS, 8, (64, 0), t, 16, (8, 7 * 16 + 8),
                                   2, 2, 8, 8, 8, 8, 8, 8)
    with pytest.raises(nt.NtsAmdError, match="negative"):
        nt.matrix_mul_batched_grid(t, X_NOTRANS, 8, (-64, 0), t, X_NOTRANS, 8, (64, 0), t, 8, (64, 128),
                                   2, 2, 8, 8, 8, 8, 8, 8)
    # nothing to do is no error
    nt.matrix_mul_batched_grid(t, X_NOTRANS, 8, (64, 0), t, X_NOTRANS, 8, (64, 0), t, 8, (64, 128),
                               0, 2, 8, 8, 8, 8, 8, 8)


def test_benchmark_shape_against_split_product_merge(gpu, oracle):
    """32 sentences x 8 heads at full size: the product on merged tensors equals, bit for bit, the same kernels
    run on tensors that were split and merged by copies (same tiles, same order of accumulation: only the
    addressing differs), and one head of one sentence against the oracle."""
    torch = torch_()
    B, nh, L, dh = 32, 8, 128, 64
    H = nh * dh
    probs = dev(oracle.uniform((nh, B, L, L), 81, 0.0, 1.0), gpu)
    probs /= probs.sum(-1, keepdim=True)
    v = dev(oracle.normal((B, L, H), 82), gpu)
    out = torch.full((B, L, H), float("nan"), device=gpu)
    nt.matrix_mul_batched_grid(probs, X_NOTRANS, L, (L * L, B * L * L), v, X_NOTRANS, H, (L * H, dh),
                               out, H, (L * H, dh), B, nh, L, L, L, dh, L, dh)
    vs = v.view(B, L, nh, dh).permute(2, 0, 1, 3).contiguous()
    os_ = torch.empty((nh, B, L, dh), device=gpu)
    nt.matrix_mul_batched_strided(probs, X_NOTRANS, vs, X_NOTRANS, os_, nh * B, L * L, L * dh, L * dh,
                                  L, L, L, dh, L, dh)
    torch.cuda.synchronize()
    assert torch.equal(out, os_.permute(1, 2, 0, 3).reshape(B, L, H))
    b, h = 17, 5
    ref = oracle.matmul2d(probs[h, b].cpu().numpy(), X_NOTRANS,
                          np.ascontiguousarray(v[b, :, h * dh:(h + 1) * dh].cpu().numpy()), X_NOTRANS)
    assert_fp32(out[b, :, h * dh:(h + 1) * dh].cpu().numpy(), ref, L, what="sentence 17, head 5")
