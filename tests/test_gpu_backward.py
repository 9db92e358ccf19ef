"""Parity of the backward-side entry points with the CPU oracle, through the C ABI:
products whose k range is cut into pieces (which meet in a workspace and are added in a fixed order,
or add to c with atomics when the knob asks for that), products that return
the column sums of op(b) on the side, the [x][y][z] reduction, and the three gradient
steps (MatrixMul, MatrixMulBatched, MulAndShift) assembled from them the way the nts::
layer assembles them, against the oracle and the compiled reference's fixtures.
Limits are in tests/tolerance.py."""
import itertools

import numpy as np
import pytest

import niutensor_amd as nt
from niutensor_amd import X_NOTRANS, X_TRANS
from tolerance import assert_fp16, assert_fp32

pytestmark = pytest.mark.gpu

TRANS = list(itertools.product((X_NOTRANS, X_TRANS), repeat=2))
ENV = ("NTSAMD_TILE_CFG", "NTSAMD_SPLIT_K", "NTSAMD_F32_SPLIT_ATOMIC")


def torch_():
    import torch
    return torch


def dev(x, gpu, half=False):
    t = torch_().from_numpy(np.ascontiguousarray(x)).to(gpu)
    return t.half() if half else t


def stored(shape, trans):
    return (shape[1], shape[0]) if trans == X_TRANS else shape


def halfed(oracle, x):
    return oracle.from_f16_bits(oracle.to_f16_bits(x))


@pytest.fixture(autouse=True)
def name_the_case(request):
    print("\n[gpu-case] %s" % request.node.nodeid, flush=True)
    for k in ENV:
        nt.tuning_set(k, None)
    yield
    for k in ENV:
        nt.tuning_set(k, None)


# ---- k cut into pieces ------------------------------------------------------------

@pytest.mark.parametrize("atomic", (False, True))
@pytest.mark.parametrize("ta,tb", TRANS)
def test_split_k_against_oracle(gpu, oracle, ta, tb, atomic):
    """Forced piece counts on both tile shapes, every beta, a ragged k and a bias. Through the workspace (the
    pieces are added in their order by a second kernel, which also applies beta and the bias) and with the
    pieces adding to c with atomics (beta 1: nothing to prepare, 0: c is cleared first, other: c is scaled
    first; the bias rides on the first piece)."""
    torch = torch_()
    nt.tuning_set("NTSAMD_F32_SPLIT_ATOMIC", 1 if atomic else None)
    for cfg, splits, (M, N, K) in (("0", "2", (128, 256, 1024)), ("0", "4", (100, 72, 1500)), ("1", "8", (64, 192, 4096)),
                                   ("1", "4", (37, 64, 1111)), ("0", "16", (256, 128, 4100))):
        nt.tuning_set("NTSAMD_TILE_CFG", cfg)
        nt.tuning_set("NTSAMD_SPLIT_K", splits)
        a = oracle.uniform(stored((M, K), ta), 11)
        b = oracle.uniform(stored((K, N), tb), 12)
        c0 = oracle.uniform((M, N), 13)
        mag1 = oracle.matmul2d(np.abs(a), ta, np.abs(b), tb)
        for alpha, beta in ((1.0, 1.0), (0.5, 0.0), (-1.25, 0.5)):
            ref = oracle.matmul2d(a, ta, b, tb, c0.copy(), alpha, beta)
            c = dev(c0, gpu) if beta != 0 else torch.full((M, N), float("nan"), device=gpu)
            nt.matrix_mul(dev(a, gpu), ta, dev(b, gpu), tb, c, alpha, beta)
            assert_fp32(c.cpu().numpy(), ref, K, abs(alpha) * mag1 + abs(beta) * np.abs(c0),
                        what="cfg%s splits %s %dx%dx%d alpha=%g beta=%g" % (cfg, splits, M, N, K, alpha, beta))
        bias = oracle.uniform((N,), 14)
        ref = oracle.matmul2d(a, ta, b, tb, c0.copy(), 1.0, 1.0) + bias
        c = dev(c0, gpu)
        nt.matrix_mul(dev(a, gpu), ta, dev(b, gpu), tb, c, 1.0, 1.0, bias=dev(bias, gpu))
        assert_fp32(c.cpu().numpy(), ref, K, mag1 + np.abs(c0) + np.abs(bias), what="split bias")


def test_split_k_is_chosen_for_weight_gradient_shapes_and_can_be_turned_off(gpu, oracle):
    """dE/dw of a linear layer: few tiles, long k. The library's own choice (pieces) and the
    forced single piece must agree within the limit; and a batch of such products too."""
    M, N, K = 256, 512, 4096
    a = oracle.uniform((K, M), 1)
    b = oracle.normal((K, N), 2, 0, 0.5)
    c0 = oracle.uniform((M, N), 3)
    ref = oracle.matmul2d(a, X_TRANS, b, X_NOTRANS, c0.copy(), 1.0, 1.0)
    mag = oracle.matmul2d(np.abs(a), X_TRANS, np.abs(b), X_NOTRANS) + np.abs(c0)
    got = {}
    for mode in (None, "1"):
        if mode:
            nt.tuning_set("NTSAMD_SPLIT_K", mode)
        c = dev(c0, gpu)
        nt.matrix_mul(dev(a, gpu), X_TRANS, dev(b, gpu), X_NOTRANS, c, 1.0, 1.0)
        got[mode] = c.cpu().numpy()
        assert_fp32(got[mode], ref, K, mag, what="weight gradient, split mode %s" % mode)
    # strided batch of long-k products
    nt.tuning_set("NTSAMD_SPLIT_K", None)
    B, M, N, K = 3, 64, 64, 2048
    a, b, c0 = oracle.uniform((B, M, K), 4), oracle.uniform((B, K, N), 5), oracle.uniform((B, M, N), 6)
    ref = oracle.matmul_batched(a, X_NOTRANS, b, X_NOTRANS, c0.copy(), 0.5, 0.25)
    c = dev(c0, gpu)
    nt.matrix_mul_batched_strided(dev(a, gpu), X_NOTRANS, dev(b, gpu), X_NOTRANS, c, B, M * K, K * N, M * N,
                                  M, K, K, N, M, N, 0.5, 0.25)
    assert_fp32(c.cpu().numpy(), ref, K, what="batched long k")


def test_split_k_gives_the_same_bits_on_every_run(gpu, oracle):
    """Weight-gradient shapes (few tiles, a long k) are cut along k by the library's own choice. The pieces are
    added in their order, so twenty runs of a float product, of a half one and of the column sums over many rows
    give bit-identical results, as the reference's cublasSgemm does."""
    torch = torch_()
    for half in (False, True):
        for (M, N, K) in ((512, 512, 4096), (256, 512, 4096), (100, 200, 3000 if not half else 3008)):
            a = dev(oracle.normal((K, M), 1, 0, 0.5), gpu, half)
            b = dev(oracle.normal((K, N), 2, 0, 0.5), gpu, half)
            c0 = dev(oracle.uniform((M, N), 3), gpu, half)
            first = None
            for run in range(20):
                c = c0.clone()
                nt.matrix_mul(a, X_TRANS, b, X_NOTRANS, c, 1.0, 1.0)
                if first is None:
                    first = c
                assert torch.equal(c, first), "half=%d %dx%dx%d run %d" % (half, M, N, K, run)
    xs = oracle.normal((8192, 300), 4)
    x = dev(xs, gpu).reshape(8192, 300, 1)
    first = None
    for run in range(20):
        out = torch.full((300,), float("nan"), device=gpu)
        nt.reduce_sum_xz(x, out)
        if first is None:
            first = out
            assert_fp32(out.cpu().numpy(), oracle.reduce_sum(xs, 0), 8192, oracle.reduce_sum(np.abs(xs), 0),
                        what="column sums in pieces")
        assert torch.equal(out, first), "column sums run %d" % run


def test_two_host_threads_on_one_stream_keep_their_pieces_apart(gpu, oracle):
    """Two host threads issue half weight gradients (512 x 512 x 4096, cut along k) to the NULL stream, as every
    caller of the nts:: layer does. Each call's product and summing kernels must stay together on the stream: were
    they to interleave (A product, B product, A sum, B sum), A would sum B's pieces. Every result is checked."""
    import threading
    torch = torch_()
    M, N, K = 512, 512, 4096
    work = []
    for t in range(2):
        a = halfed(oracle, oracle.normal((K, M), 50 + t, 0, 0.5))
        b = halfed(oracle, oracle.normal((K, N), 60 + t, 0, 0.5))
        work.append((dev(a, gpu, True), dev(b, gpu, True), oracle.matmul2d(a, X_TRANS, b, X_NOTRANS)))
    L = nt.load()
    failures = []

    def issue(t):
        a, b, ref = work[t]
        outs = [torch.empty((M, N), device=gpu, dtype=torch.float16) for _ in range(40)]
        for c in outs:
            rc = L.ntsamd_matrix_mul(0, None, a.data_ptr(), X_TRANS, nt.X_FLOAT16, b.data_ptr(), X_NOTRANS, nt.X_FLOAT16,
                                     c.data_ptr(), nt.X_FLOAT16, K, M, K, N, M, N, 1.0, 0.0)
            if rc != 0:
                failures.append("thread %d: rc %d" % (t, rc))
                return
        torch.cuda.synchronize()
        for i, c in enumerate(outs):
            if not torch.equal(c, outs[0]):
                failures.append("thread %d: product %d differs from the thread's first" % (t, i))
                break
        try:
            assert_fp16(outs[0].float().cpu().numpy(), ref, what="thread %d" % t)
        except AssertionError as e:
            failures.append(str(e))

    torch.cuda.synchronize()
    threads = [threading.Thread(target=issue, args=(t,)) for t in range(2)]
    for th in threads:
        th.start()
    for th in threads:
        th.join()
    assert not failures, failures


def test_workspaces_can_be_released_and_come_back(gpu, oracle):
    torch = torch_()
    M, N, K = 256, 256, 4096
    a, b = dev(oracle.normal((K, M), 1, 0, 0.5), gpu), dev(oracle.normal((K, N), 2, 0, 0.5), gpu)
    c1, c2 = torch.empty((M, N), device=gpu), torch.empty((M, N), device=gpu)
    nt.tuning_set("NTSAMD_SPLIT_K", 8)
    nt.matrix_mul(a, X_TRANS, b, X_NOTRANS, c1)
    nt.release_workspaces(0)
    nt.release_workspaces(-1)            # nothing left to free: still fine
    nt.matrix_mul(a, X_TRANS, b, X_NOTRANS, c2)
    assert torch.equal(c1, c2)
    assert_fp32(c1.cpu().numpy(), oracle.matmul2d(a.cpu().numpy(), X_TRANS, b.cpu().numpy(), X_NOTRANS), K)


# ---- column sums on the side -----------------------------------------------------------

def column_sums(oracle, b, tb):
    """Sums over k of op(b)[k][j] with the reference's _ReduceSum (rows of b for X_NOTRANS)."""
    return oracle.reduce_sum(b, 0 if tb == X_NOTRANS else 1)


@pytest.mark.parametrize("half", (False, True))
@pytest.mark.parametrize("ta,tb", TRANS)
def test_matrix_mul_colsum(gpu, oracle, half, ta, tb):
    torch = torch_()
    # 16-byte friendly shapes ride in the product kernel; the ragged ones take the separate pass
    shapes = [(128, 128, 64), (64, 256, 512), (200, 72, 100), (96, 40, 2048), (33, 29, 57), (5, 7, 3), (130, 64, 33)]
    for cfg in ("0", "1"):
        nt.tuning_set("NTSAMD_TILE_CFG", cfg)
        for i, (M, N, K) in enumerate(shapes):
            a = oracle.normal(stored((M, K), ta), 100 + i, 0, 0.5)
            b = oracle.normal(stored((K, N), tb), 200 + i, 0, 0.5)
            c0 = oracle.uniform((M, N), 300 + i)
            s0 = oracle.uniform((N,), 400 + i)
            if half:
                a, b, c0, s0 = (halfed(oracle, v) for v in (a, b, c0, s0))
            for alpha, beta, sbeta in ((1.0, 0.0, 0.0), (0.5, 1.0, 1.0), (1.0, 1.0, -0.5)):
                ref = oracle.matmul2d(a, ta, b, tb, c0.copy(), alpha, beta)
                sref = sbeta * s0 + column_sums(oracle, b, tb)
                c = dev(c0, gpu, half) if beta != 0 else dev(np.full((M, N), np.nan, np.float32), gpu, half)
                s = dev(s0, gpu, half) if sbeta != 0 else dev(np.full((N,), np.nan, np.float32), gpu, half)
                nt.matrix_mul_colsum(dev(a, gpu, half), ta, dev(b, gpu, half), tb, c, s, alpha, beta, sbeta)
                what = "cfg%s %dx%dx%d half=%d alpha=%g beta=%g sbeta=%g" % (cfg, M, N, K, half, alpha, beta, sbeta)
                smag = np.abs(sbeta * s0) + column_sums(oracle, np.abs(b), tb)
                if half:
                    assert_fp16(c.float().cpu().numpy(), ref, what=what)
                    # the sums are rounded to half once, from an fp32 total
                    assert np.abs(s.float().cpu().numpy() - sref).max() <= 2.0 ** -10 * smag.max() + 1e-6, what
                else:
                    assert_fp32(c.cpu().numpy(), ref, K, what=what)
                    assert_fp32(s.cpu().numpy(), sref, K, smag, what=what + " sums")


def test_colsum_with_split_k_and_without_a_product(gpu, oracle):
    M, N, K = 128, 256, 4096
    a, b = oracle.uniform((K, M), 1), oracle.uniform((K, N), 2)
    c0, s0 = oracle.uniform((M, N), 3), oracle.uniform((N,), 4)
    for splits in ("1", "8"):
        nt.tuning_set("NTSAMD_SPLIT_K", splits)
        for sbeta in (1.0, 0.0, 0.5):
            c, s = dev(c0, gpu), dev(s0, gpu)
            nt.matrix_mul_colsum(dev(a, gpu), X_TRANS, dev(b, gpu), X_NOTRANS, c, s, 1.0, 1.0, sbeta)
            assert_fp32(c.cpu().numpy(), oracle.matmul2d(a, X_TRANS, b, X_NOTRANS, c0.copy(), 1.0, 1.0), K)
            assert_fp32(s.cpu().numpy(), sbeta * s0 + oracle.reduce_sum(b, 0), K,
                        np.abs(sbeta * s0) + oracle.reduce_sum(np.abs(b), 0), what="splits %s sbeta %g" % (splits, sbeta))
    # a product with no rows still owes the sums
    nt.tuning_set("NTSAMD_SPLIT_K", None)
    torch = torch_()
    s = dev(s0, gpu)
    nt.matrix_mul_colsum(torch.empty((K, 0), device=gpu), X_TRANS, dev(b, gpu), X_NOTRANS,
                         torch.empty((0, N), device=gpu), s, 1.0, 0.0, 1.0)
    assert_fp32(s.cpu().numpy(), s0 + oracle.reduce_sum(b, 0), K)


def test_half_colsum_with_k_cut(gpu, oracle):
    """The half weight gradient with its bias gradient: cut along k the product leaves the sums to a pass of its
    own over b (the pieces gather none); both ways give the same sums and a product within the half limit."""
    M, N, K = 128, 256, 4096
    a, b = halfed(oracle, oracle.normal((K, M), 1, 0, 0.5)), halfed(oracle, oracle.normal((K, N), 2, 0, 0.5))
    c0, s0 = halfed(oracle, oracle.uniform((M, N), 3)), halfed(oracle, oracle.uniform((N,), 4))
    ref = oracle.matmul2d(a, X_TRANS, b, X_NOTRANS, c0.copy(), 1.0, 1.0)
    for splits in ("1", "8", None):
        if splits is None:
            nt.tuning_set("NTSAMD_SPLIT_K", None)
        else:
            nt.tuning_set("NTSAMD_SPLIT_K", splits)
        for sbeta in (1.0, 0.0):
            c, s = dev(c0, gpu, True), dev(s0, gpu, True)
            nt.matrix_mul_colsum(dev(a, gpu, True), X_TRANS, dev(b, gpu, True), X_NOTRANS, c, s, 1.0, 1.0, sbeta)
            what = "pieces %s sbeta %g" % (splits, sbeta)
            assert_fp16(c.float().cpu().numpy(), ref, what=what)
            sref = sbeta * s0 + oracle.reduce_sum(b, 0)
            smag = np.abs(sbeta * s0) + oracle.reduce_sum(np.abs(b), 0)
            assert np.abs(s.float().cpu().numpy() - sref).max() <= 2.0 ** -10 * smag.max() + 1e-6, what
    nt.tuning_set("NTSAMD_SPLIT_K", None)


# ---- the reduction ------------------------------------------------------------------------

@pytest.mark.parametrize("half", (False, True))
def test_reduce_sum_xz(gpu, oracle, half):
    for i, shape in enumerate([(1, 5, 1), (7, 5, 1), (300, 64, 1), (4096, 200, 1), (1000, 37, 1), (4, 6, 32), (5, 7, 3),
                               (1, 40, 129), (24, 8, 2048), (3, 1, 1)]):
        x = oracle.uniform(shape, 50 + i)
        o0 = oracle.uniform((shape[1],), 70 + i)
        if half:
            x, o0 = halfed(oracle, x), halfed(oracle, o0)
        for beta in (0.0, 1.0, -0.5):
            ref = beta * o0 + oracle.reduce_sum(oracle.reduce_sum(x, 2), 0)
            mag = np.abs(beta * o0) + np.abs(x).sum((0, 2))
            out = dev(o0, gpu, half) if beta != 0 else dev(np.full(shape[1:2], np.nan, np.float32), gpu, half)
            nt.reduce_sum_xz(dev(x, gpu, half), out, beta)
            got = out.float().cpu().numpy()
            what = "%s half=%d beta=%g" % (shape, half, beta)
            if half:
                assert np.abs(got - ref).max() <= 2.0 ** -10 * mag.max() + 1e-6, what
            else:
                assert_fp32(got, ref, shape[0] * shape[2], mag, what=what)


# ---- the gradient steps, assembled as the nts:: layer assembles them -----------------------------

def gpu_grad_matmul(gpu, a, ta, b, tb, dedc, alpha, deda, dedb, col_sum=None):
    """The four cases of XMathGrad::GradMatrixMul (source/network/XBackwardMath.cpp:636-696) on 2-D device tensors."""
    N_, T_ = X_NOTRANS, X_TRANS
    mm = lambda p, tp, q, tq, r: nt.matrix_mul(p, tp, q, tq, r, alpha, 1.0)
    if (ta, tb) == (N_, N_):
        mm(dedc, N_, b, T_, deda)
        if col_sum is not None:
            nt.matrix_mul_colsum(a, T_, dedc, N_, dedb, col_sum, alpha, 1.0, 1.0)
        else:
            mm(a, T_, dedc, N_, dedb)
    elif (ta, tb) == (T_, N_):
        mm(b, N_, dedc, T_, deda)
        mm(a, N_, dedc, N_, dedb)
    elif (ta, tb) == (N_, T_):
        mm(dedc, N_, b, N_, deda)
        mm(dedc, T_, a, N_, dedb)
    else:
        mm(b, T_, dedc, T_, deda)
        mm(dedc, T_, a, T_, dedb)


def test_gradient_fixtures_of_the_compiled_reference(gpu, generated_backward):
    n = 0
    for name in generated_backward.of_kind("grad_matmul"):
        d = generated_backward.case(name)
        ta, tb = (int(v) for v in d["params"])
        a2 = d["a"].reshape(-1, d["a"].shape[-1])
        g2 = d["dedc"].reshape(-1, d["dedc"].shape[-1])
        deda, dedb = dev(d["deda0"].reshape(a2.shape), gpu), dev(d["dedb0"], gpu)
        gpu_grad_matmul(gpu, dev(a2, gpu), ta, dev(d["b"], gpu), tb, dev(g2, gpu), float(d["scal"][0]), deda, dedb)
        K = max(a2.shape + d["b"].shape)
        assert_fp32(deda.cpu().numpy().reshape(d["deda"].shape), d["deda"], K, what=name)
        assert_fp32(dedb.cpu().numpy(), d["dedb"], K, what=name)
        n += 1
    for name in generated_backward.of_kind("grad_mulandshift"):
        d = generated_backward.case(name)
        nn = int(d["params"][0])
        x2 = d["x"].reshape(-1, d["x"].shape[-1])
        g = d["dedc"]
        g2 = g.reshape(-1, g.shape[-1])
        dedx, dedw, dedb = dev(d["dedx0"].reshape(x2.shape), gpu), dev(d["dedw0"], gpu), dev(d["dedb0"].ravel(), gpu)
        ride = nn == g.ndim - 1
        gpu_grad_matmul(gpu, dev(x2, gpu), X_NOTRANS, dev(d["w"], gpu), X_NOTRANS, dev(g2, gpu), float(d["scal"][0]),
                        dedx, dedw, col_sum=dedb if ride else None)
        if not ride:
            xs, zs = int(np.prod(g.shape[:nn])), int(np.prod(g.shape[nn + 1:]))
            nt.reduce_sum_xz(dev(g.reshape(xs, g.shape[nn], zs), gpu), dedb, 1.0)
        K = max(x2.shape + d["w"].shape)
        assert_fp32(dedx.cpu().numpy().reshape(d["dedx"].shape), d["dedx"], K, what=name)
        assert_fp32(dedw.cpu().numpy(), d["dedw"], K, what=name)
        assert_fp32(dedb.cpu().numpy().reshape(d["dedb"].shape), d["dedb"], g.size // d["dedb"].size, what=name)
        n += 1
    assert n == 16


def test_linear_layer_backward_at_full_size(gpu, oracle):
    """The backward of the benchmark's linear layer (x[4096x512] w[512x2048] + bias): dE/dx = dE/dc w^T
    (NT, k = 2048), dE/dw = x^T dE/dc (TN, k = 4096, cut into pieces) with dE/dbias on the side.
    Checked in double precision on sampled rows, against the oracle on a slab, and through
    linearity: running the step twice from zero doubles every gradient (up to the atomics' order)."""
    torch = torch_()
    M, K, N = 4096, 512, 2048
    x = oracle.uniform((M, K), 1)
    w = oracle.normal((K, N), 2, 0, 0.02)
    g = oracle.normal((M, N), 3, 0, 1.0)
    dx, dw, db = (torch.zeros(s, device=gpu) for s in ((M, K), (K, N), (N,)))
    X, W, G = dev(x, gpu), dev(w, gpu), dev(g, gpu)
    gpu_grad_matmul(gpu, X, X_NOTRANS, W, X_NOTRANS, G, 1.0, dx, dw, col_sum=db)
    once = [t.cpu().numpy().copy() for t in (dx, dw, db)]
    rows = np.random.default_rng(0).choice(M, 48, replace=False)
    ex = g[rows].astype(np.float64) @ w.astype(np.float64).T
    assert_fp32(once[0][rows], ex, N, np.abs(g[rows]).astype(np.float64) @ np.abs(w).astype(np.float64).T, what="dE/dx")
    krows = np.random.default_rng(1).choice(K, 48, replace=False)
    ew = x[:, krows].astype(np.float64).T @ g.astype(np.float64)
    assert_fp32(once[1][krows], ew, M, np.abs(x[:, krows]).astype(np.float64).T @ np.abs(g).astype(np.float64), what="dE/dw")
    assert_fp32(once[2], g.astype(np.float64).sum(0), M, np.abs(g).astype(np.float64).sum(0), what="dE/dbias")
    slab = oracle.matmul2d(np.ascontiguousarray(g[:64]), X_NOTRANS, w, X_TRANS)
    assert_fp32(once[0][:64], slab, N, what="dE/dx against the oracle")
    gpu_grad_matmul(gpu, X, X_NOTRANS, W, X_NOTRANS, G, 1.0, dx, dw, col_sum=db)
    for t, o, k in zip((dx, dw, db), once, (N, M, M)):
        assert_fp32(t.cpu().numpy(), 2.0 * o.astype(np.float64), k, what="second step adds")


@pytest.mark.parametrize("half", (False, True))
def test_attention_backward_batches(gpu, oracle, half):
    """GradMatrixMulBatched (XBackwardMath.cpp:709-786) for S = Q K^T / 8: dE/dQ += dE/dS K / 8,
    dE/dK += dE/dS^T Q / 8, as strided batches with beta = 1."""
    B, L, D = 16, 128, 64
    q, k, gs = oracle.normal((B, L, D), 1), oracle.normal((B, L, D), 2), oracle.normal((B, L, L), 3)
    dq0, dk0 = oracle.uniform((B, L, D), 4), oracle.uniform((B, L, D), 5)
    if half:
        q, k, gs, dq0, dk0 = (halfed(oracle, v) for v in (q, k, gs, dq0, dk0))
    rq, rk = oracle.grad_matmul_batched(q, X_NOTRANS, k, X_TRANS, gs, 0.125, dq0.copy(), dk0.copy())
    dq, dk = dev(dq0, gpu, half), dev(dk0, gpu, half)
    Q, K_, G = dev(q, gpu, half), dev(k, gpu, half), dev(gs, gpu, half)
    nt.matrix_mul_batched_strided(G, X_NOTRANS, K_, X_NOTRANS, dq, B, L * L, L * D, L * D, L, L, L, D, L, D, 0.125, 1.0)
    nt.matrix_mul_batched_strided(G, X_TRANS, Q, X_NOTRANS, dk, B, L * L, L * D, L * D, L, L, L, D, L, D, 0.125, 1.0)
    if half:
        assert_fp16(dq.float().cpu().numpy(), rq, what="dE/dQ")
        assert_fp16(dk.float().cpu().numpy(), rk, what="dE/dK")
    else:
        assert_fp32(dq.cpu().numpy(), rq, L, what="dE/dQ")
        assert_fp32(dk.cpu().numpy(), rk, L, what="dE/dK")
