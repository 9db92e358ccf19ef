"""Parity of the gfx950 kernels with the CPU oracle, through the C ABI.

Same seeded inputs on both sides at sizes the oracle finishes in seconds; the
committed fixtures (known answers of the reference's tests, outputs of the
compiled reference); and, at the full benchmark sizes, double-precision checks
on sampled rows plus size-independent properties (scaling, accumulation,
transposition). Limits are in tests/tolerance.py.
"""
import itertools

import numpy as np
import pytest

import niutensor_amd as nt
from niutensor_amd import BIAS_COL, BIAS_ROW, X_NOTRANS, X_TRANS
from tolerance import FP16_LIMIT, assert_fp16, assert_fp32, fp32_limit, normwise, scaled

pytestmark = pytest.mark.gpu

TRANS = list(itertools.product((X_NOTRANS, X_TRANS), repeat=2))


def torch_():
    import torch
    return torch


def dev_tensor(x, gpu, half=False):
    torch = torch_()
    t = torch.from_numpy(np.ascontiguousarray(x)).to(gpu)
    return t.half() if half else t


def stored(shape_mk, trans):
    """Stored shape of an operand whose logical shape is (rows, cols) after trans()."""
    return (shape_mk[1], shape_mk[0]) if trans == X_TRANS else shape_mk


def magnitude(oracle, a, ta, b, tb, alpha, beta=0.0, c0=None, bias=None):
    mag = abs(alpha) * oracle.matmul2d(np.abs(a), ta, np.abs(b), tb)
    if beta != 0:
        mag = mag + abs(beta) * np.abs(c0)
    if bias is not None:
        mag = mag + np.abs(bias)
    return mag


@pytest.fixture(autouse=True)
def name_the_case(request):
    # a GPU fault can take the box with it: say which test is running first
    print("\n[gpu-case] %s" % request.node.nodeid, flush=True)
    nt.tuning_set("NTSAMD_TILE_CFG", None)
    nt.tuning_set("NTSAMD_SPLIT_K", None)
    yield
    nt.tuning_set("NTSAMD_TILE_CFG", None)
    nt.tuning_set("NTSAMD_SPLIT_K", None)


# ---- fixtures held by the reference and by the compiled reference ------------

def test_known_answers_2d(gpu, oracle, known_answers):
    torch = torch_()
    for case in known_answers:
        if case["op"] not in ("matmul2d",) and not (case["op"] in ("matmul", "matmul_batched") and np.ndim(case["a"]) == 2):
            continue
        a = dev_tensor(np.array(case["a"], np.float32), gpu)
        b = dev_tensor(np.array(case["b"], np.float32), gpu)
        ans = np.array(case["answer"], np.float32)
        c = torch.full(ans.shape, float("nan"), device=gpu)
        nt.matrix_mul(a, case["transA"], b, case["transB"], c)
        assert oracle.check_data(c.cpu().numpy(), ans, 1e-4), case["name"]
        assert np.array_equal(c.cpu().numpy(), ans), case["name"]


def test_known_answers_batched_and_paired(gpu, oracle, known_answers):
    torch = torch_()
    by_name = {c["name"]: c for c in known_answers}
    # TMatrixMulBatched case 2: block i with block i, one strided batch
    case = by_name["TMatrixMulBatched.case2"]
    a = dev_tensor(np.array(case["a"], np.float32), gpu)
    b = dev_tensor(np.array(case["b"], np.float32), gpu)
    c = torch.empty((2, 2, 2), device=gpu)
    nt.matrix_mul_batched_strided(a, X_NOTRANS, b, X_NOTRANS, c, 2, 6, 6, 4, 2, 3, 3, 2, 2, 2)
    assert np.array_equal(c.cpu().numpy(), np.array(case["answer"], np.float32))
    # TMatrixMul case 3: every block of a with every block of b; not equally spaced, so a pointer list
    case = by_name["TMatrixMul.case3"]
    a = dev_tensor(np.array(case["a"], np.float32), gpu)
    b = dev_tensor(np.array(case["b"], np.float32), gpu)
    c = torch.empty((3, 2, 2, 2), device=gpu)
    al, bl, cl = [], [], []
    for p in range(3):
        for q in range(2):
            al.append(a[p]); bl.append(b[q]); cl.append(c[p, q])
    nt.matrix_mul_batched(al, X_NOTRANS, bl, X_NOTRANS, cl)
    assert np.array_equal(c.cpu().numpy(), np.array(case["answer"], np.float32))
    # TMatrixMul case 4: the flattened product
    case = by_name["TMatrixMul.case4"]
    a = dev_tensor(np.array(case["a"], np.float32).reshape(6, 3), gpu)
    b = dev_tensor(np.array(case["b"], np.float32), gpu)
    c = torch.empty((6, 2), device=gpu)
    nt.matrix_mul(a, X_NOTRANS, b, X_NOTRANS, c)
    assert np.array_equal(c.cpu().numpy().reshape(3, 2, 2), np.array(case["answer"], np.float32))


def test_compiled_reference_fixture(gpu, generated):
    """Outputs of the real NiuTensor CPU code (tests/golden/ref_generated.npz)."""
    torch = torch_()
    n = 0
    for name in generated.of_kind("matmul2d"):
        d = generated.case(name)
        ta, tb = (int(v) for v in d["params"])
        alpha, beta = (float(v) for v in d["scal"])
        c = dev_tensor(d["c0"], gpu)
        nt.matrix_mul(dev_tensor(d["a"], gpu), ta, dev_tensor(d["b"], gpu), tb, c, alpha, beta)
        K = d["a"].shape[0] if ta == X_TRANS else d["a"].shape[1]
        assert_fp32(c.cpu().numpy(), d["c"], K, what=name)
        n += 1
    for name in generated.of_kind("matmul_batched"):
        d = generated.case(name)
        ta, tb = (int(v) for v in d["params"])
        alpha, beta = (float(v) for v in d["scal"])
        a, b, c0 = d["a"], d["b"], d["c0"]
        c = dev_tensor(c0, gpu)
        count = int(np.prod(a.shape[:-2]))
        nt.matrix_mul_batched_strided(dev_tensor(a, gpu), ta, dev_tensor(b, gpu), tb, c, count,
                                      a.shape[-1] * a.shape[-2], b.shape[-1] * b.shape[-2], c0.shape[-1] * c0.shape[-2],
                                      a.shape[-2], a.shape[-1], b.shape[-2], b.shape[-1], c0.shape[-2], c0.shape[-1],
                                      alpha, beta)
        K = a.shape[-2] if ta == X_TRANS else a.shape[-1]
        assert_fp32(c.cpu().numpy(), d["c"], K, what=name)
        n += 1
    for name in generated.of_kind("mulandshift"):
        d = generated.case(name)
        ov, tx, tw = (int(v) for v in d["params"])
        x, w, bias, cref = d["x"], d["w"], d["bias"], d["c"]
        if not (tx == X_NOTRANS and w.ndim == 2):
            continue
        # the flattened product with the bias in the epilogue, as the host layer issues it
        rows = int(np.prod(x.shape[:-1]))
        x2 = dev_tensor(x.reshape(rows, x.shape[-1]), gpu)
        c = torch.full((rows, cref.shape[-1]), float("nan"), device=gpu)
        hit = [i for i in range(cref.ndim) if cref.shape[i] == bias.size][-1]
        if hit == cref.ndim - 1:
            mode, div = BIAS_COL, 1
        else:
            mode, div = BIAS_ROW, int(np.prod(cref.shape[hit + 1:-1]))
        nt.matrix_mul(x2, tx, dev_tensor(w, gpu), tw, c, float(d["scal"][0]), 0.0,
                      bias=dev_tensor(bias.ravel(), gpu), bias_mode=mode, bias_row_div=div)
        assert_fp32(c.cpu().numpy().reshape(cref.shape), cref, x.shape[-1], what=name)
        n += 1
    assert n > 45


# ---- seeded inputs against the oracle ------------------------------------------

SHAPES = [(1, 1, 1), (5, 7, 3), (37, 29, 53), (64, 64, 16), (63, 65, 17), (127, 129, 31), (128, 128, 64),
          (130, 70, 33), (200, 24, 100), (256, 384, 128), (300, 260, 101), (1, 300, 40), (300, 1, 40), (96, 96, 1),
          (32, 300, 70), (17, 515, 129)]


@pytest.mark.parametrize("ta,tb", TRANS)
def test_fp32_against_oracle(gpu, oracle, ta, tb):
    torch = torch_()
    # 128 x 128, 64 x 64, 32 x 128 (at most 32 rows; else the rule's choice), 16 rows per workgroup on the same kernel
    for cfg in ("0", "1", "3", "4"):
        nt.tuning_set("NTSAMD_TILE_CFG", cfg)
        for i, (M, N, K) in enumerate(SHAPES):
            a = oracle.uniform(stored((M, K), ta), 1000 + i)
            b = oracle.uniform(stored((K, N), tb), 2000 + i)
            c0 = oracle.uniform((M, N), 3000 + i)
            for alpha, beta in ((1.0, 0.0), (0.5, 1.0), (-1.25, 0.5)):
                ref = oracle.matmul2d(a, ta, b, tb, c0.copy(), alpha, beta)
                c = dev_tensor(c0, gpu) if beta != 0 else torch.full((M, N), float("nan"), device=gpu)
                nt.matrix_mul(dev_tensor(a, gpu), ta, dev_tensor(b, gpu), tb, c, alpha, beta)
                assert_fp32(c.cpu().numpy(), ref, K, magnitude(oracle, a, ta, b, tb, alpha, beta, c0),
                            what="cfg%s %dx%dx%d alpha=%g beta=%g" % (cfg, M, N, K, alpha, beta))


@pytest.mark.parametrize("ta,tb", TRANS)
def test_fp16_against_oracle(gpu, oracle, ta, tb):
    torch = torch_()
    # 128 x 128, 64 x 64 with slabs of 32 and of 64 along k, 256 x 256 (eight waves up to k = 2048, four beyond: the
    # last shape)
    for cfg, slab64 in (("0", None), ("1", "0"), ("1", "1"), ("2", None)):
        nt.tuning_set("NTSAMD_TILE_CFG", cfg)
        nt.tuning_set("NTSAMD_F16_SLAB64", slab64)
        for i, (M, N, K) in enumerate(SHAPES + [(264, 520, 2304)]):
            # round the inputs to half first; the oracle then runs in fp32 on those values
            a = oracle.from_f16_bits(oracle.to_f16_bits(oracle.normal(stored((M, K), ta), 4000 + i, 0, 0.5)))
            b = oracle.from_f16_bits(oracle.to_f16_bits(oracle.normal(stored((K, N), tb), 5000 + i, 0, 0.5)))
            c0 = oracle.from_f16_bits(oracle.to_f16_bits(oracle.uniform((M, N), 6000 + i)))
            for alpha, beta in ((1.0, 0.0), (0.5, 1.0)):
                ref = oracle.matmul2d(a, ta, b, tb, c0.copy(), alpha, beta)
                c = dev_tensor(c0, gpu, True) if beta != 0 else torch.full((M, N), float("nan"), device=gpu).half()
                nt.matrix_mul(dev_tensor(a, gpu, True), ta, dev_tensor(b, gpu, True), tb, c, alpha, beta)
                assert_fp16(c.float().cpu().numpy(), ref, what="cfg%s slab64=%s %dx%dx%d alpha=%g beta=%g" % (cfg, slab64, M, N, K, alpha, beta))
    nt.tuning_set("NTSAMD_F16_SLAB64", None)


@pytest.mark.parametrize("ta,tb", TRANS)
def test_half_products_cut_along_k(gpu, oracle, ta, tb):
    """Few tiles and a long k (weight gradients, the few rows of a decoding step): k is cut into pieces whose fp32
    partial products a second kernel adds up and finishes (alpha, beta, bias by column, rectifier, either result
    type). Forced here on both tile shapes with 2 and 16 pieces, ragged edges and a ragged last piece; the last
    two shapes are cut by the dispatcher's own choice as well (no forcing: the first turn of the loop)."""
    torch = torch_()
    # 51 columns: rows of c that the adding kernel cannot take four elements at a time (cut only where b is stored
    # n x k: the 16-byte path needs whole 16-byte pieces along the rows of b)
    shapes = [(8, 8, 264), (72, 136, 1000), (40, 51, 1024), (200, 24, 4096), (16, 512, 2048), (256, 256, 2304)]
    for cfg, pieces, slab64 in ((None, None, None), ("0", "2", None), ("0", "16", None), ("1", "2", "1"), ("1", "16", "1"), ("1", "2", "0"), ("1", "16", "0")):
        for key, val in (("NTSAMD_TILE_CFG", cfg), ("NTSAMD_SPLIT_K", pieces), ("NTSAMD_F16_SLAB64", slab64)):
            nt.tuning_set(key, val)
        for i, (M, N, K) in enumerate(shapes if cfg else shapes[-2:]):
            a = oracle.from_f16_bits(oracle.to_f16_bits(oracle.normal(stored((M, K), ta), 8000 + i, 0, 0.5)))
            b = oracle.from_f16_bits(oracle.to_f16_bits(oracle.normal(stored((K, N), tb), 8100 + i, 0, 0.5)))
            bias = oracle.from_f16_bits(oracle.to_f16_bits(oracle.normal((N,), 8300 + i)))
            for out_float in (False, True):
                c0 = oracle.uniform((M, N), 8200 + i)
                if not out_float:
                    c0 = oracle.from_f16_bits(oracle.to_f16_bits(c0))
                for alpha, beta, with_bias, act in ((1.0, 0.0, False, nt.ACT_NONE), (0.5, 1.0, False, nt.ACT_NONE),
                                                    (1.0, 0.0, True, nt.ACT_NONE), (1.0, 0.5, True, nt.ACT_RECTIFY)):
                    ref = oracle.matmul2d(a, ta, b, tb, c0.copy(), alpha, beta)
                    if with_bias:
                        ref = ref + bias[None, :]
                    if act == nt.ACT_RECTIFY:
                        ref = np.maximum(ref, 0)
                    c = dev_tensor(c0, gpu, not out_float) if beta != 0 else \
                        torch.full((M, N), float("nan"), device=gpu, dtype=torch.float32 if out_float else torch.float16)
                    nt.matrix_mul(dev_tensor(a, gpu, True), ta, dev_tensor(b, gpu, True), tb, c, alpha, beta,
                                  bias=dev_tensor(bias, gpu, not out_float) if with_bias else None, act=act)
                    what = "cfg%s pieces=%s %dx%dx%d alpha=%g beta=%g bias=%s act=%d float=%s" % (
                        cfg, pieces, M, N, K, alpha, beta, with_bias, act, out_float)
                    if out_float:
                        assert_fp32(c.cpu().numpy(), ref, K, what=what)
                    else:
                        assert_fp16(c.float().cpu().numpy(), ref, what=what)


@pytest.mark.parametrize("ta,tb", TRANS)
def test_half_products_fetched_through_registers_cut_along_k(gpu, oracle, ta, tb):
    """The same cut for the kernel that fetches its operands through registers (rows of any length: the gradient
    of a layer with a 30011-word vocabulary has few tiles and k = 30011): forced on both tile shapes with 2 and 16
    pieces, odd row lengths, a ragged last piece, bases that are only 2-byte aligned."""
    torch = torch_()
    shapes = [(9, 7, 263), (72, 135, 1001), (40, 51, 1024), (130, 66, 4099)]
    try:
        nt.tuning_set("NTSAMD_F16_FETCH", 2)
        for cfg, pieces in (("0", "2"), ("0", "16"), ("1", "2"), ("1", "16"), (None, None)):
            for key, val in (("NTSAMD_TILE_CFG", cfg), ("NTSAMD_SPLIT_K", pieces)):
                nt.tuning_set(key, val)
            for i, (M, N, K) in enumerate(shapes if cfg else shapes[-1:]):
                a = oracle.from_f16_bits(oracle.to_f16_bits(oracle.normal(stored((M, K), ta), 8600 + i, 0, 0.5)))
                b = oracle.from_f16_bits(oracle.to_f16_bits(oracle.normal(stored((K, N), tb), 8700 + i, 0, 0.5)))
                bias = oracle.from_f16_bits(oracle.to_f16_bits(oracle.normal((N,), 8800 + i)))
                abuf = torch.zeros(a.size + 1, device=gpu, dtype=torch.float16)
                bbuf = torch.zeros(b.size + 1, device=gpu, dtype=torch.float16)
                abuf[1:] = dev_tensor(a.ravel(), gpu, True)
                bbuf[1:] = dev_tensor(b.ravel(), gpu, True)
                for out_float in (False, True):
                    c0 = oracle.uniform((M, N), 8900 + i)
                    if not out_float:
                        c0 = oracle.from_f16_bits(oracle.to_f16_bits(c0))
                    for alpha, beta, with_bias, act in ((1.0, 0.0, False, nt.ACT_NONE), (0.5, 1.0, True, nt.ACT_RECTIFY)):
                        ref = oracle.matmul2d(a, ta, b, tb, c0.copy(), alpha, beta)
                        if with_bias:
                            ref = ref + bias[None, :]
                        if act == nt.ACT_RECTIFY:
                            ref = np.maximum(ref, 0)
                        c = dev_tensor(c0, gpu, not out_float) if beta != 0 else \
                            torch.full((M, N), float("nan"), device=gpu, dtype=torch.float32 if out_float else torch.float16)
                        nt.matrix_mul(abuf[1:].view(a.shape), ta, bbuf[1:].view(b.shape), tb, c, alpha, beta,
                                      bias=dev_tensor(bias, gpu, not out_float) if with_bias else None, act=act)
                        what = "cfg%s pieces=%s %dx%dx%d alpha=%g beta=%g float=%s" % (cfg, pieces, M, N, K, alpha, beta, out_float)
                        if out_float:
                            assert_fp32(c.cpu().numpy(), ref, K, what=what)
                        else:
                            assert_fp16(c.float().cpu().numpy(), ref, what=what)
    finally:
        nt.tuning_set("NTSAMD_F16_FETCH", None)


def test_batches_of_half_products_cut_along_k(gpu, oracle):
    """Three products with their own strides between them and rows of c longer than the result is wide (the heads
    of a merged tensor): every piece of every item finds its place in the workspace and in c, and what lies
    between the rows of c stays as it was. Twice in a row on one stream: the second call reuses the workspace."""
    torch = torch_()
    nt.tuning_set("NTSAMD_TILE_CFG", "1")
    nt.tuning_set("NTSAMD_SPLIT_K", "4")
    M, N, K, count = 40, 72, 1536, 3
    ldc, between = 3 * N, N
    a = oracle.from_f16_bits(oracle.to_f16_bits(oracle.normal((count, M, K), 8400, 0, 0.5)))
    b = oracle.from_f16_bits(oracle.to_f16_bits(oracle.normal((count, K, N), 8401, 0, 0.5)))
    for turn in range(2):
        whole = torch.full((M, ldc), -7.0, device=gpu, dtype=torch.float16)
        nt.matrix_mul_batched_grid(dev_tensor(a, gpu, True), X_NOTRANS, K, (M * K, 0), dev_tensor(b, gpu, True), X_NOTRANS, N, (K * N, 0),
                                   whole, ldc, (between, 0), count, 1, M, K, K, N, M, N, 1.0 + turn, 0.0)
        got = whole.float().cpu().numpy()
        for i in range(count):
            ref = oracle.matmul2d(a[i], X_NOTRANS, b[i], X_NOTRANS, None, 1.0 + turn, 0.0)
            assert_fp16(got[:, i * between:i * between + N], ref, what="item %d turn %d" % (i, turn))


def test_half_products_cut_along_k_on_two_streams(gpu, oracle):
    """The partial products of a cut product live in a workspace that belongs to the stream: two streams that run
    such products at the same time must not see each other's. The sums are added in a fixed order, so each result
    must equal, bit for bit, what the same product gives on its own."""
    torch = torch_()
    nt.tuning_set("NTSAMD_TILE_CFG", "1")
    nt.tuning_set("NTSAMD_SPLIT_K", "8")
    M, N, K = 64, 512, 4096
    ops = []
    for i in range(2):
        a = dev_tensor(oracle.normal((M, K), 8500 + i, 0, 0.5), gpu, True)
        b = dev_tensor(oracle.normal((K, N), 8510 + i, 0, 0.5), gpu, True)
        alone = torch.empty((M, N), device=gpu, dtype=torch.float16)
        nt.matrix_mul(a, X_NOTRANS, b, X_NOTRANS, alone)
        ops.append((a, b, alone, torch.empty_like(alone)))
    torch.cuda.synchronize()
    ref = oracle.matmul2d(ops[0][0].float().cpu().numpy(), X_NOTRANS, ops[0][1].float().cpu().numpy(), X_NOTRANS)
    assert_fp16(ops[0][2].float().cpu().numpy(), ref, what="alone")
    streams = [torch.cuda.Stream(), torch.cuda.Stream()]
    for turn in range(30):
        for (a, b, alone, c), st in zip(ops, streams):
            with torch.cuda.stream(st):
                nt.matrix_mul(a, X_NOTRANS, b, X_NOTRANS, c)
    torch.cuda.synchronize()
    for i, (a, b, alone, c) in enumerate(ops):
        assert torch.equal(c, alone), "stream %d" % i


def test_fp16_bits_match_the_oracle_conversion(gpu, oracle):
    """Small integers: every product and sum is exact in fp32 and representable in half,
    so the half result must equal the oracle's result bit for bit (RNE store)."""
    rng = np.random.default_rng(3)
    a = rng.integers(-4, 5, (70, 40)).astype(np.float32)
    b = rng.integers(-4, 5, (40, 50)).astype(np.float32)
    ref = oracle.matmul2d(a, X_NOTRANS, b, X_NOTRANS)
    torch = torch_()
    c = torch.empty((70, 50), device=gpu, dtype=torch.float16)
    nt.matrix_mul(dev_tensor(a, gpu, True), X_NOTRANS, dev_tensor(b, gpu, True), X_NOTRANS, c)
    assert np.array_equal(c.cpu().numpy().view(np.uint16), oracle.to_f16_bits(ref))
    # rounding of a half result: alpha makes values that need RNE
    c2 = torch.empty((70, 50), device=gpu, dtype=torch.float16)
    nt.matrix_mul(dev_tensor(a, gpu, True), X_NOTRANS, dev_tensor(b, gpu, True), X_NOTRANS, c2, 1.0 / 3.0)
    want = oracle.to_f16_bits((ref * np.float32(1.0 / 3.0)).astype(np.float32))
    assert np.array_equal(c2.cpu().numpy().view(np.uint16), want)


def test_half_in_float_out(gpu, oracle):
    torch = torch_()
    a = oracle.from_f16_bits(oracle.to_f16_bits(oracle.normal((45, 77), 1)))
    b = oracle.from_f16_bits(oracle.to_f16_bits(oracle.normal((31, 77), 2)))
    ref = oracle.matmul2d(a, X_NOTRANS, b, X_TRANS)
    c = torch.empty((45, 31), device=gpu)
    nt.matrix_mul(dev_tensor(a, gpu, True), X_NOTRANS, dev_tensor(b, gpu, True), X_TRANS, c)
    assert_fp32(c.cpu().numpy(), ref, 77)


@pytest.mark.parametrize("ta,tb", TRANS)
def test_half_in_float_out_on_the_main_path(gpu, oracle, ta, tb):
    """16-byte aligned half operands with a float result (a half product that feeds a softmax, as
    the reference converts the scores and the output layer's logits to float): every tile shape,
    ragged edges, beta, and a float bias by column. The products of halves are exact in fp32, so
    the fp32 limit applies."""
    torch = torch_()
    for cfg in ("0", "1", "2"):
        nt.tuning_set("NTSAMD_TILE_CFG", cfg)
        for i, (M, N, K) in enumerate([(8, 8, 8), (64, 72, 40), (136, 264, 96), (257, 120, 64), (300, 520, 128)]):
            a = oracle.from_f16_bits(oracle.to_f16_bits(oracle.normal(stored((M, K), ta), 7000 + i, 0, 0.5)))
            b = oracle.from_f16_bits(oracle.to_f16_bits(oracle.normal(stored((K, N), tb), 7100 + i, 0, 0.5)))
            c0 = oracle.uniform((M, N), 7200 + i)
            bias = oracle.normal((N,), 7300 + i)
            for alpha, beta, with_bias in ((1.0, 0.0, False), (0.5, 1.0, False), (1.0, 0.0, True)):
                ref = oracle.matmul2d(a, ta, b, tb, c0.copy(), alpha, beta)
                if with_bias:
                    ref = ref + bias[None, :]
                c = dev_tensor(c0, gpu) if beta != 0 else torch.full((M, N), float("nan"), device=gpu)
                nt.matrix_mul(dev_tensor(a, gpu, True), ta, dev_tensor(b, gpu, True), tb, c, alpha, beta,
                              bias=dev_tensor(bias, gpu) if with_bias else None)
                assert_fp32(c.cpu().numpy(), ref, K, what="cfg%s %dx%dx%d alpha=%g beta=%g bias=%s" % (cfg, M, N, K, alpha, beta, with_bias))


@pytest.mark.parametrize("ta,tb", TRANS)
def test_fp32_rows_of_any_length_and_alignment(gpu, oracle, ta, tb):
    """Float operands whose rows are not multiples of four long and whose first element sits on any
    dword: k tails of 1, 2 and 3, ragged m and n, batches whose items start on odd elements. Both
    operands lie inside larger buffers filled with NaN, so a read past either end of a matrix, or a
    k >= K that is not discarded, would poison the result."""
    torch = torch_()
    for cfg in ("0", "1"):
        nt.tuning_set("NTSAMD_TILE_CFG", cfg)
        for i, (M, N, K, shift) in enumerate([(129, 67, 33, 1), (70, 131, 130, 3), (255, 257, 63, 2), (3, 2, 1, 1), (64, 64, 515, 5)]):
            a = oracle.uniform(stored((M, K), ta), 8100 + i)
            b = oracle.uniform(stored((K, N), tb), 8200 + i)
            c0 = oracle.uniform((M, N), 8300 + i)
            abuf = torch.full((a.size + shift + 7,), float("nan"), device=gpu)
            bbuf = torch.full((b.size + shift + 7,), float("nan"), device=gpu)
            abuf[shift:shift + a.size] = dev_tensor(a.ravel(), gpu)
            bbuf[shift:shift + b.size] = dev_tensor(b.ravel(), gpu)
            av, bv = abuf[shift:shift + a.size].view(a.shape), bbuf[shift:shift + b.size].view(b.shape)
            for alpha, beta in ((1.0, 0.0), (0.5, 1.0)):
                ref = oracle.matmul2d(a, ta, b, tb, c0.copy(), alpha, beta)
                c = dev_tensor(c0, gpu) if beta != 0 else torch.full((M, N), float("nan"), device=gpu)
                nt.matrix_mul(av, ta, bv, tb, c, alpha, beta)
                assert_fp32(c.cpu().numpy(), ref, K, magnitude(oracle, a, ta, b, tb, alpha, beta, c0),
                            what="cfg%s %dx%dx%d shift %d alpha=%g beta=%g" % (cfg, M, N, K, shift, alpha, beta))
    nt.tuning_set("NTSAMD_TILE_CFG", None)
    # a batch of products whose items are an odd number of elements apart
    count, M, N, K = 5, 45, 51, 37
    a = oracle.uniform((count,) + stored((M, K), ta), 8400)
    b = oracle.uniform((count,) + stored((K, N), tb), 8401)
    ref = oracle.matmul_batched(a, ta, b, tb, None, 0.75)
    c = torch.full((count, M, N), float("nan"), device=gpu)
    sa, sb = stored((M, K), ta), stored((K, N), tb)
    nt.matrix_mul_batched_strided(dev_tensor(a, gpu), ta, dev_tensor(b, gpu), tb, c, count, M * K, K * N, M * N,
                                  sa[0], sa[1], sb[0], sb[1], M, N, 0.75, 0.0)
    assert_fp32(c.cpu().numpy(), ref, K, what="odd strides")


def test_backward_of_the_ragged_vocabulary_projection(gpu, oracle):
    """The two gradient products of configuration 5's layer: dE/dh = dE/dc w (k = 30011, rows of dE/dc
    30011 long) and dE/dw = dE/dc^T h (m = 30011), beta = 1, checked on sampled rows in double precision."""
    torch = torch_()
    V = 30011
    dy = oracle.normal((4096, V), 8500, 0, 0.1)
    w = oracle.normal((V, 512), 8501, 0, 0.02)
    h = oracle.uniform((4096, 512), 8502)
    dh0, dw0 = oracle.uniform((4096, 512), 8503), oracle.uniform((V, 512), 8504)
    dh, dw = dev_tensor(dh0, gpu), dev_tensor(dw0, gpu)
    dyd = dev_tensor(dy, gpu)
    nt.matrix_mul(dyd, X_NOTRANS, dev_tensor(w, gpu), X_NOTRANS, dh, 1.0, 1.0)
    nt.matrix_mul(dyd, X_TRANS, dev_tensor(h, gpu), X_NOTRANS, dw, 1.0, 1.0)
    rows = np.array([0, 1, 127, 128, 2047, 4095])
    ref = dy[rows].astype(np.float64) @ w.astype(np.float64) + dh0[rows]
    assert_fp32(dh.cpu().numpy()[rows], ref, V, what="dE/dh")
    vr = np.array([0, 3, 127, 128, 30000, 30008, 30009, 30010])
    ref = dy[:, vr].astype(np.float64).T @ h.astype(np.float64) + dw0[vr]
    assert_fp32(dw.cpu().numpy()[vr], ref, 4096, what="dE/dw")


def test_unaligned_operands(gpu, oracle):
    """Base pointers and leading dimensions that are not multiples of 16 bytes (float: still the main
    path; half: 16-byte loads through registers from any even address)."""
    torch = torch_()
    M, N, K = 70, 52, 36
    for ta, tb in TRANS:
        a = oracle.uniform(stored((M, K), ta), 7)
        b = oracle.uniform(stored((K, N), tb), 8)
        ref = oracle.matmul2d(a, ta, b, tb)
        for half in (False, True):
            # shift both operands by one element inside a larger buffer
            abuf = torch.zeros(a.size + 1, device=gpu, dtype=torch.float16 if half else torch.float32)
            bbuf = torch.zeros(b.size + 1, device=gpu, dtype=abuf.dtype)
            abuf[1:] = dev_tensor(a.ravel(), gpu, half)
            bbuf[1:] = dev_tensor(b.ravel(), gpu, half)
            av = abuf[1:].view(a.shape)
            bv = bbuf[1:].view(b.shape)
            c = torch.empty((M, N), device=gpu, dtype=abuf.dtype)
            nt.matrix_mul(av, ta, bv, tb, c)
            if half:
                ah = oracle.from_f16_bits(oracle.to_f16_bits(a))
                bh = oracle.from_f16_bits(oracle.to_f16_bits(b))
                assert_fp16(c.float().cpu().numpy(), oracle.matmul2d(ah, ta, bh, tb))
            else:
                assert_fp32(c.cpu().numpy(), ref, K)

@pytest.mark.parametrize("ta,tb", TRANS)
@pytest.mark.parametrize("out_float", [False, True])
def test_half_rows_of_any_length_and_alignment(gpu, oracle, ta, tb, out_float):
    """Half operands whose rows are no multiple of 16 bytes, at bases that are only 2-byte aligned, in buffers
    that end with the matrix: they are fetched 16 bytes at a time all the same, and the piece that hangs over
    the end of a buffer (whose last dword the range check would drop with its valid half) is fetched half by
    half. Sizes that need the 128 x 128 tile, ragged in every dimension; the last row and column of the result
    are checked on their own, since that is where a lost element would show."""
    torch = torch_()
    # the two long ones run many turns of the straight-line loop (a ring of four slabs in registers between memory
    # and LDS), with a ragged last slab after a complete one and with a last slab that is complete
    for (M, N, K) in ((203, 301, 77), (131, 135, 259), (9, 7, 5), (1, 300, 1), (70, 67, 1003), (33, 141, 1056)):
        nt.tuning_set("NTSAMD_TILE_CFG", "1" if K == 1056 else "0")
        a = oracle.from_f16_bits(oracle.to_f16_bits(oracle.uniform(stored((M, K), ta), 31)))
        b = oracle.from_f16_bits(oracle.to_f16_bits(oracle.uniform(stored((K, N), tb), 32)))
        bias = oracle.from_f16_bits(oracle.to_f16_bits(oracle.uniform((N,), 33)))
        ref = oracle.matmul2d(a, ta, b, tb) + bias[None, :]
        odt = torch.float32 if out_float else torch.float16
        for off in (0, 1):
            # the matrices end exactly where their buffers end
            abuf = torch.zeros(a.size + off, device=gpu, dtype=torch.float16)
            bbuf = torch.zeros(b.size + off, device=gpu, dtype=torch.float16)
            abuf[off:] = dev_tensor(a.ravel(), gpu, True)
            bbuf[off:] = dev_tensor(b.ravel(), gpu, True)
            c = torch.full((M, N), float("nan"), device=gpu, dtype=odt)
            nt.matrix_mul(abuf[off:].view(a.shape), ta, bbuf[off:].view(b.shape), tb, c,
                          bias=dev_tensor(bias, gpu, True).to(odt))
            got = c.float().cpu().numpy()
            assert_fp16(got, ref, what="%dx%dx%d offset %d" % (M, N, K, off))
            assert_fp16(got[-1:, :], ref[-1:, :], what="last row")
            assert_fp16(got[:, -1:], ref[:, -1:], what="last column")


@pytest.mark.parametrize("ta,tb", TRANS)
@pytest.mark.parametrize("out_float", [False, True])
def test_half_rows_of_any_length_copied_to_padded_rows(gpu, oracle, ta, tb, out_float):
    """The same operands when the library copies them into its workspace with rows padded to whole 16-byte pieces
    (zeros in the padding) and runs the product on the kernels that move operands straight to LDS: forced here on
    small shapes (the library does it by itself where the operand is small beside the product), every tile shape,
    one operand odd and the other not, both odd, a k that is no multiple of 8, a batch with a shared b."""
    torch = torch_()
    odt = torch.float32 if out_float else torch.float16
    try:
        nt.tuning_set("NTSAMD_F16_REPITCH", 1)
        for (M, N, K), cfg in (((203, 301, 77), "0"), ((131, 135, 259), "1"), ((9, 7, 5), "1"), ((1, 300, 1), "0"),
                               ((70, 67, 1003), "0"), ((264, 301, 96), "2"), ((300, 520, 1056), "2"), ((256, 141, 64), "1")):
            nt.tuning_set("NTSAMD_TILE_CFG", cfg)
            a = oracle.from_f16_bits(oracle.to_f16_bits(oracle.uniform(stored((M, K), ta), 41)))
            b = oracle.from_f16_bits(oracle.to_f16_bits(oracle.uniform(stored((K, N), tb), 42)))
            bias = oracle.from_f16_bits(oracle.to_f16_bits(oracle.uniform((N,), 43)))
            ref = oracle.matmul2d(a, ta, b, tb) + bias[None, :]
            for off in (0, 1):
                abuf = torch.zeros(a.size + off, device=gpu, dtype=torch.float16)
                bbuf = torch.zeros(b.size + off, device=gpu, dtype=torch.float16)
                abuf[off:] = dev_tensor(a.ravel(), gpu, True)
                bbuf[off:] = dev_tensor(b.ravel(), gpu, True)
                c = torch.full((M, N), float("nan"), device=gpu, dtype=odt)
                nt.matrix_mul(abuf[off:].view(a.shape), ta, bbuf[off:].view(b.shape), tb, c,
                              bias=dev_tensor(bias, gpu, True).to(odt))
                got = c.float().cpu().numpy()
                assert_fp16(got, ref, what="%dx%dx%d offset %d" % (M, N, K, off))
                assert_fp16(got[-1:, :], ref[-1:, :], what="last row")
                assert_fp16(got[:, -1:], ref[:, -1:], what="last column")
        # a batch of five a's with rows of 77 against one shared b with rows of 301
        nt.tuning_set("NTSAMD_TILE_CFG", "1")
        batch, M, N, K = 5, 67, 301, 77
        a = oracle.from_f16_bits(oracle.to_f16_bits(oracle.uniform((batch,) + stored((M, K), ta), 44)))
        b = oracle.from_f16_bits(oracle.to_f16_bits(oracle.uniform(stored((K, N), tb), 45)))
        ga, gb = dev_tensor(a, gpu, True), dev_tensor(b, gpu, True)
        c = torch.full((batch, M, N), float("nan"), device=gpu, dtype=odt)
        na, ma = a.shape[1:]
        nb, mb = b.shape
        nt.matrix_mul_batched_strided(ga, ta, gb, tb, c, batch, na * ma, 0, M * N, na, ma, nb, mb, M, N, 0.5, 0.0)
        for item in range(batch):
            assert_fp16(c[item].float().cpu().numpy(), oracle.matmul2d(a[item], ta, b, tb, None, 0.5, 0.0), what="item %d" % item)
    finally:
        nt.tuning_set("NTSAMD_F16_REPITCH", None)


def test_lists_of_half_matrices_with_odd_rows(gpu, oracle):
    """Pointer lists of half matrices take the same 16-byte loads (no alignment to rely on)."""
    torch = torch_()
    M, N, K, count = 67, 45, 131, 5
    a = [oracle.from_f16_bits(oracle.to_f16_bits(oracle.uniform((M, K), 40 + i))) for i in range(count)]
    b = [oracle.from_f16_bits(oracle.to_f16_bits(oracle.uniform((N, K), 50 + i))) for i in range(count)]
    ad = [dev_tensor(x, gpu, True) for x in a]
    bd = [dev_tensor(x, gpu, True) for x in b]
    cd = [torch.full((M, N), float("nan"), device=gpu, dtype=torch.float16) for _ in range(count)]
    nt.matrix_mul_batched(ad, X_NOTRANS, bd, X_TRANS, cd, 0.5, 0.0)
    for i in range(count):
        assert_fp16(cd[i].float().cpu().numpy(), oracle.matmul2d(a[i], X_NOTRANS, b[i], X_TRANS, alpha=0.5), what="item %d" % i)


def test_beta_zero_ignores_old_contents_and_scaling_is_exact(gpu, oracle):
    torch = torch_()
    a = dev_tensor(oracle.uniform((200, 96), 11), gpu)
    b = dev_tensor(oracle.uniform((96, 136), 12), gpu)
    junk = torch.full((200, 136), float("nan"), device=gpu)
    junk[::2] = float("inf")
    c1 = torch.zeros((200, 136), device=gpu)
    nt.matrix_mul(a, X_NOTRANS, b, X_NOTRANS, c1)
    nt.matrix_mul(a, X_NOTRANS, b, X_NOTRANS, junk)
    assert torch.equal(c1, junk)
    c2 = torch.empty_like(c1)
    nt.matrix_mul(a, X_NOTRANS, b, X_NOTRANS, c2, 2.0, 0.0)
    assert torch.equal(c2, 2 * c1)                       # alpha = 2 only shifts exponents
    c3 = c1.clone()
    nt.matrix_mul(a, X_NOTRANS, b, X_NOTRANS, c3, 1.0, 1.0)
    assert torch.equal(c3, 2 * c1)                       # beta = 1 on top of the product doubles it
    # (A B)^T = B^T A^T through the transposed kernels
    ct = torch.empty((136, 200), device=gpu)
    nt.matrix_mul(b, X_TRANS, a, X_TRANS, ct)
    assert normwise(ct.t().cpu().numpy(), c1.cpu().numpy()) < 1e-6


# ---- batches --------------------------------------------------------------------

@pytest.mark.parametrize("half", (False, True))
def test_strided_batches(gpu, oracle, half):
    torch = torch_()
    check = assert_fp16 if half else (lambda g, r, what="": assert_fp32(g, r, 24, what=what))

    def prep(x):
        return oracle.from_f16_bits(oracle.to_f16_bits(x)) if half else x

    q = prep(oracle.normal((2, 5, 50, 24), 1))
    k = prep(oracle.normal((2, 5, 40, 24), 2))
    v = prep(oracle.normal((2, 5, 40, 24), 3))
    s_ref = oracle.matmul_batched(q, X_NOTRANS, k, X_TRANS, None, 0.125)
    dt = torch.float16 if half else torch.float32
    s = torch.full((2, 5, 50, 40), float("nan"), device=gpu, dtype=dt)
    nt.matrix_mul_batched_strided(dev_tensor(q, gpu, half), X_NOTRANS, dev_tensor(k, gpu, half), X_TRANS, s,
                                  10, 50 * 24, 40 * 24, 50 * 40, 50, 24, 40, 24, 50, 40, 0.125, 0.0)
    check(s.float().cpu().numpy(), s_ref, "QK^T")
    s_in = prep(s_ref)
    o_ref = oracle.matmul_batched(s_in, X_NOTRANS, v, X_NOTRANS)
    o = torch.empty((2, 5, 50, 24), device=gpu, dtype=dt)
    nt.matrix_mul_batched_strided(dev_tensor(s_in, gpu, half), X_NOTRANS, dev_tensor(v, gpu, half), X_NOTRANS, o,
                                  10, 50 * 40, 40 * 24, 50 * 24, 50, 40, 40, 24, 50, 24)
    check(o.float().cpu().numpy(), o_ref, "SV")
    # stride 0: one b shared by the whole batch (a transposed N-D a against one matrix)
    at = prep(oracle.uniform((7, 24, 33), 4))
    w = prep(oracle.uniform((24, 18), 5))
    ref = oracle.matmul(at, X_TRANS, w, X_NOTRANS)
    c = torch.empty((7, 33, 18), device=gpu, dtype=dt)
    nt.matrix_mul_batched_strided(dev_tensor(at, gpu, half), X_TRANS, dev_tensor(w, gpu, half), X_NOTRANS, c,
                                  7, 24 * 33, 0, 33 * 18, 24, 33, 24, 18, 33, 18)
    check(c.float().cpu().numpy(), ref, "shared b")
    # stride 0 on a, accumulate
    a1 = prep(oracle.uniform((20, 24), 6))
    bb = prep(oracle.uniform((6, 24, 10), 7))
    c0 = prep(oracle.uniform((6, 20, 10), 8))
    ref = np.stack([oracle.matmul2d(a1, X_NOTRANS, bb[i].copy(), X_NOTRANS, c0[i].copy(), 1.0, 1.0) for i in range(6)])
    c = dev_tensor(c0, gpu, half)
    nt.matrix_mul_batched_strided(dev_tensor(a1, gpu, half), X_NOTRANS, dev_tensor(bb, gpu, half), X_NOTRANS, c,
                                  6, 0, 240, 200, 20, 24, 24, 10, 20, 10, 1.0, 1.0)
    check(c.float().cpu().numpy(), ref, "shared a")


def test_pointer_lists(gpu, oracle):
    torch = torch_()
    # more items than one launch carries in its arguments (128), unequal spacing
    a = oracle.uniform((20, 9, 14), 1)
    b = oracle.uniform((15, 14, 6), 2)
    ga, gb = dev_tensor(a, gpu), dev_tensor(b, gpu)
    c = torch.full((20, 15, 9, 6), float("nan"), device=gpu)
    al, bl, cl = [], [], []
    for p in range(20):
        for q in range(15):
            al.append(ga[p]); bl.append(gb[q]); cl.append(c[p, q])
    assert len(al) == 300
    nt.matrix_mul_batched(al, X_NOTRANS, bl, X_NOTRANS, cl, 0.5, 0.0)
    assert_fp32(c.cpu().numpy(), oracle.matmul(a, X_NOTRANS, b, X_NOTRANS, None, 0.5), 14)
    # half, transposed items
    ah = oracle.from_f16_bits(oracle.to_f16_bits(oracle.normal((3, 16, 40), 3)))
    bh = oracle.from_f16_bits(oracle.to_f16_bits(oracle.normal((3, 24, 16), 4)))
    gah, gbh = dev_tensor(ah, gpu, True), dev_tensor(bh, gpu, True)
    ch = torch.empty((3, 40, 24), device=gpu, dtype=torch.float16)
    nt.matrix_mul_batched([gah[i] for i in (2, 0, 1)], X_TRANS, [gbh[i] for i in (2, 0, 1)], X_TRANS,
                          [ch[i] for i in (2, 0, 1)])
    assert_fp16(ch.float().cpu().numpy(), oracle.matmul_batched(ah, X_TRANS, bh, X_TRANS))


# ---- fused bias -------------------------------------------------------------------

@pytest.mark.parametrize("half", (False, True))
def test_fused_bias(gpu, oracle, half):
    torch = torch_()

    def prep(x):
        return oracle.from_f16_bits(oracle.to_f16_bits(x)) if half else x

    x = prep(oracle.uniform((6, 20, 48), 1))
    w = prep(oracle.normal((48, 72), 2, 0, 0.05))
    dt = torch.float16 if half else torch.float32
    for bshape in ((72,), (20,), (6, 1, 1)):
        bias = prep(oracle.normal(bshape, 3, 0, 0.05))
        ref, n = oracle.mulandshift(x, w, bias, 0.5)
        c = torch.full((120, 72), float("nan"), device=gpu, dtype=dt)
        if n == 2:
            mode, div = BIAS_COL, 1
        else:
            mode, div = BIAS_ROW, int(np.prod(ref.shape[n + 1:-1]))
        nt.matrix_mul(dev_tensor(x.reshape(120, 48), gpu, half), X_NOTRANS, dev_tensor(w, gpu, half), X_NOTRANS, c, 0.5, 0.0,
                      bias=dev_tensor(bias.ravel(), gpu, half), bias_mode=mode, bias_row_div=div)
        got = c.float().cpu().numpy().reshape(ref.shape)
        mag = 0.5 * oracle.matmul(np.abs(x), X_NOTRANS, np.abs(w), X_NOTRANS) + np.abs(ref - oracle.matmul(x, X_NOTRANS, w, X_NOTRANS, None, 0.5))
        if half and mode == BIAS_ROW:
            # a bias by row is added behind the product, as the reference adds it (_SumDim on the half result,
            # MulAndShift.cpp:69-88): the product is rounded to half before the sum is, so where the two nearly
            # cancel the error is a half ulp of the product, not of the sum
            assert np.isfinite(got).all()
            assert normwise(got, ref) <= FP16_LIMIT and scaled(got, ref, mag) <= FP16_LIMIT, str(bshape)
        elif half:
            assert_fp16(got, ref, what=str(bshape))
        else:
            assert_fp32(got, ref, 48, mag, what=str(bshape))


@pytest.mark.parametrize("half", (False, True))
def test_bias_by_row_on_many_rows_and_odd_columns(gpu, oracle, half):
    """The pass that adds a bias by row behind the product: more rows than its grid holds in one sweep (it strides),
    columns that are no whole 16-byte pieces (element by element), a row group of 3 and a rectifier; against float64."""
    torch = torch_()
    dt = torch.float16 if half else torch.float32
    for M, N, K, div in ((300000, 8, 8, 3), (1000, 37, 16, 1), (4100, 72, 24, 7)):
        g = torch.Generator(device="cpu").manual_seed(M + N)
        a = torch.randn(M, K, generator=g).to(dt).to(gpu)
        b = torch.randn(K, N, generator=g).to(dt).to(gpu)
        length = (M + div - 1) // div
        bias = torch.randn(length, generator=g).to(dt).to(gpu)
        c = torch.full((M, N), float("nan"), device=gpu, dtype=dt)
        nt.matrix_mul(a, X_NOTRANS, b, X_NOTRANS, c, 1.0, 0.0, bias=bias, bias_mode=BIAS_ROW, bias_row_div=div, act=nt.ACT_RECTIFY)
        assert "+row_bias_kernel" in nt.last_plan()
        rows = torch.arange(M, device=gpu) // div
        prod = a.double() @ b.double()
        if half:
            prod = prod.half().double()          # the product is rounded before the bias is added, as in the reference
        ref = (prod + bias.double()[rows][:, None]).clamp(min=0)
        err = float((c.double() - ref).abs().max() / ref.abs().max())
        assert err <= (2e-3 if half else 1e-5), (M, N, K, div, err)


@pytest.mark.parametrize("half", (False, True))
def test_fused_bias_and_rectify(gpu, oracle, half):
    """Rectify(MulAndShift(x, w, b)) in the epilogue (the first step of the reference's feed-forward block):
    against the oracle's product + broadcast add + rectify, on the main path and on the generic one
    (row-indexed bias), with beta, and with a NaN and a negative zero forced into the result."""
    torch = torch_()
    for cfg in ("0", "1", "2") if half else ("0", "1"):
        nt.tuning_set("NTSAMD_TILE_CFG", cfg)
        for i, (M, N, K) in enumerate([(64, 64, 32), (136, 264, 96), (257, 120, 64), (33, 35, 37) if not half else (40, 48, 56)]):
            x = oracle.normal((M, K), 9000 + i)
            w = oracle.normal((K, N), 9100 + i, 0, 0.3)
            b = oracle.normal((N,), 9200 + i)
            c0 = oracle.uniform((M, N), 9300 + i)
            if half:
                x, w, b, c0 = (oracle.from_f16_bits(oracle.to_f16_bits(t)) for t in (x, w, b, c0))
            for beta in (0.0, 0.5):
                pre = oracle.matmul2d(x, X_NOTRANS, w, X_NOTRANS, c0.copy(), 1.0, beta) + b[None, :]
                ref = oracle.rectify(np.ascontiguousarray(pre, np.float32))
                c = dev_tensor(c0, gpu, half) if beta != 0 else torch.full((M, N), float("nan"), device=gpu, dtype=torch.float16 if half else torch.float32)
                nt.matrix_mul(dev_tensor(x, gpu, half), X_NOTRANS, dev_tensor(w, gpu, half), X_NOTRANS, c, 1.0, beta,
                              bias=dev_tensor(b, gpu, half), act=nt.ACT_RECTIFY)
                got = c.float().cpu().numpy()
                assert (got >= 0).all() and (got[ref == 0] <= 1e-3).all()
                # elements whose pre-activation is within rounding of zero may fall on either side
                if half:
                    assert_fp16(got, ref, what="cfg%s %dx%dx%d beta=%g" % (cfg, M, N, K, beta))
                else:
                    assert_fp32(got, ref, K, what="cfg%s %dx%dx%d beta=%g" % (cfg, M, N, K, beta))
    nt.tuning_set("NTSAMD_TILE_CFG", None)
    if not half:
        # bias by row group (generic path) with the activation
        x, w, b = oracle.normal((60, 20), 9400), oracle.normal((20, 30), 9401), oracle.normal((6,), 9402)
        pre = oracle.matmul2d(x, X_NOTRANS, w, X_NOTRANS) + np.repeat(b, 10)[:, None]
        c = torch.full((60, 30), float("nan"), device=gpu)
        nt.matrix_mul(dev_tensor(x, gpu), X_NOTRANS, dev_tensor(w, gpu), X_NOTRANS, c, 1.0, 0.0,
                      bias=dev_tensor(b, gpu), bias_mode=nt.BIAS_ROW, bias_row_div=10, act=nt.ACT_RECTIFY)
        assert_fp32(c.cpu().numpy(), oracle.rectify(np.ascontiguousarray(pre, np.float32)), 20, what="row bias")
        # special values: NaN in, NaN out; an exact negative zero stays a negative zero
        x = np.zeros((8, 8), np.float32)
        x[0, 0] = np.nan
        w = np.eye(8, dtype=np.float32)
        b = np.full((8,), -0.0, np.float32)
        c = torch.full((8, 8), 7.0, device=gpu)
        nt.matrix_mul(dev_tensor(x, gpu), X_NOTRANS, dev_tensor(w, gpu), X_NOTRANS, c, 1.0, 0.0, bias=dev_tensor(b, gpu), act=nt.ACT_RECTIFY)
        got = c.cpu().numpy()
        assert np.isnan(got[0]).all() and not np.isnan(got[1:]).any() and (got[1:] == 0).all()
    L = nt.load()
    t = torch.zeros(64, device=gpu)
    p = t.data_ptr()
    assert L.ntsamd_matrix_mul_bias_act(0, None, p, 1, 2, p, 1, 2, p, 2, 8, 8, 8, 8, 8, 8, 1.0, 0.0, p, 1, 8, 1, 5) == 1


def test_runs_on_the_callers_stream(gpu, oracle):
    torch = torch_()
    a = dev_tensor(oracle.uniform((256, 128), 1), gpu)
    b = dev_tensor(oracle.uniform((128, 192), 2), gpu)
    c = torch.zeros((256, 192), device=gpu)
    side = torch.cuda.Stream()
    torch.cuda.synchronize()
    with torch.cuda.stream(side):
        nt.matrix_mul(a, X_NOTRANS, b, X_NOTRANS, c)
    side.synchronize()
    assert_fp32(c.cpu().numpy(), oracle.matmul2d(a.cpu().numpy(), X_NOTRANS, b.cpu().numpy(), X_NOTRANS), 128)
    assert torch.cuda.current_device() == 0


# ---- the benchmark configurations at full size ---------------------------------------

def sampled_f64(a, ta, b, tb, rows, alpha=1.0):
    A = (a.T if ta == X_TRANS else a)[rows].astype(np.float64)
    B = (b.T if tb == X_TRANS else b).astype(np.float64)
    return alpha * (A @ B)


def whole_f64(a, ta, b, tb):
    """op(a) op(b) in double precision on the host, the WHOLE result: a mistake in the mapping of workgroups to
    tiles (the renumbering by XCD, the last group of tile rows, an unwritten tile) cannot hide between samples."""
    A = (a.T if ta == X_TRANS else a).astype(np.float64)
    B = (b.T if tb == X_TRANS else b).astype(np.float64)
    return A @ B


def library_magnitude(gpu, a, ta, b, tb, half=False):
    """(|a| |b|)_ij for the component-wise measure, at sizes where the CPU oracle would take minutes: one more
    product of the library itself, on the absolute values (every term positive: no cancellation to get wrong)."""
    torch = torch_()
    ga, gb = dev_tensor(np.abs(a), gpu, half), dev_tensor(np.abs(b), gpu, half)
    rows = a.shape[1] if ta == X_TRANS else a.shape[0]
    cols = b.shape[0] if tb == X_TRANS else b.shape[1]
    m = torch.empty((rows, cols), device=gpu)
    nt.matrix_mul(ga, ta, gb, tb, m)
    return m.cpu().numpy().astype(np.float64)


def test_config1_and_2_linear_layer(gpu, oracle):
    """fp32 [4096x512] x [512x2048], plain and with the bias of MulAndShift."""
    torch = torch_()
    x = oracle.uniform((4096, 512), 1)
    w = oracle.normal((512, 2048), 2, 0, 0.02)
    bias = oracle.normal((2048,), 3, 0, 0.02)
    gx, gw, gb = dev_tensor(x, gpu), dev_tensor(w, gpu), dev_tensor(bias, gpu)
    c = torch.full((4096, 2048), float("nan"), device=gpu)
    nt.matrix_mul(gx, X_NOTRANS, gw, X_NOTRANS, c)
    got = c.cpu().numpy()
    # every element, against double precision, under both measures
    want = whole_f64(x, X_NOTRANS, w, X_NOTRANS)
    mag = library_magnitude(gpu, x, X_NOTRANS, w, X_NOTRANS)
    assert_fp32(got, want, 512, mag, what="configuration 2 without its bias, whole result")
    # configuration 1's own operands: both uniform
    w1 = oracle.uniform((512, 2048), 2)
    c1 = torch.full((4096, 2048), float("nan"), device=gpu)
    nt.matrix_mul(gx, X_NOTRANS, dev_tensor(w1, gpu), X_NOTRANS, c1)
    assert_fp32(c1.cpu().numpy(), whole_f64(x, X_NOTRANS, w1, X_NOTRANS), 512,
                library_magnitude(gpu, x, X_NOTRANS, w1, X_NOTRANS), what="configuration 1, whole result")
    # the oracle itself on a slab of rows (it needs ~1 s per 400 rows here)
    ref = oracle.matmul2d(x[:256].copy(), X_NOTRANS, w, X_NOTRANS)
    assert_fp32(got[:256], ref, 512, magnitude(oracle, x[:256].copy(), X_NOTRANS, w, X_NOTRANS, 1.0))
    cb = torch.full((4096, 2048), float("nan"), device=gpu)
    nt.matrix_mul(gx, X_NOTRANS, gw, X_NOTRANS, cb, bias=gb)
    # the epilogue adds bias[column] to the same accumulators
    assert normwise((cb - c).cpu().numpy(), np.broadcast_to(bias, (4096, 2048))) < 1e-5
    assert_fp32(cb.cpu().numpy(), want + bias.astype(np.float64), 512, mag + np.abs(bias),
                what="configuration 2, whole result")
    ref_b, n = oracle.mulandshift(x[:64].copy().reshape(1, 64, 512), w, bias)
    assert n == 2
    assert_fp32(cb.cpu().numpy()[:64], ref_b[0], 512)


def test_config3_attention_batches(gpu, oracle):
    torch = torch_()
    q = oracle.normal((256, 128, 64), 1)
    k = oracle.normal((256, 128, 64), 2)
    v = oracle.normal((256, 128, 64), 3)
    gq, gk, gv = dev_tensor(q, gpu), dev_tensor(k, gpu), dev_tensor(v, gpu)
    s = torch.full((256, 128, 128), float("nan"), device=gpu)
    nt.matrix_mul_batched_strided(gq, X_NOTRANS, gk, X_TRANS, s, 256, 8192, 8192, 16384, 128, 64, 128, 64, 128, 128, 0.125)
    s_ref = oracle.matmul_batched(q, X_NOTRANS, k, X_TRANS, None, 0.125)
    s_mag = oracle.matmul_batched(np.abs(q), X_NOTRANS, np.abs(k), X_TRANS, None, 0.125)
    assert_fp32(s.cpu().numpy(), s_ref, 64, s_mag, what="configuration 3, scores, all 256 items")
    assert_fp32(s.cpu().numpy(), 0.125 * np.einsum("bik,bjk->bij", q.astype(np.float64), k.astype(np.float64)), 64, s_mag,
                what="configuration 3, scores against double precision")
    o = torch.full((256, 128, 64), float("nan"), device=gpu)
    nt.matrix_mul_batched_strided(s, X_NOTRANS, gv, X_NOTRANS, o, 256, 16384, 8192, 8192, 128, 128, 128, 64, 128, 64)
    sh = s.cpu().numpy()
    o_ref = oracle.matmul_batched(sh, X_NOTRANS, v, X_NOTRANS)
    o_mag = oracle.matmul_batched(np.abs(sh), X_NOTRANS, np.abs(v), X_NOTRANS)
    assert_fp32(o.cpu().numpy(), o_ref, 128, o_mag, what="configuration 3, context, all 256 items")
    assert_fp32(o.cpu().numpy(), np.einsum("bik,bkj->bij", sh.astype(np.float64), v.astype(np.float64)), 128, o_mag,
                what="configuration 3, context against double precision")


def test_config4_half_tn(gpu, oracle):
    """fp16, a stored [1024x8192] with X_TRANS, b [1024x4096]: fp32 accumulation, half result."""
    torch = torch_()
    a = oracle.from_f16_bits(oracle.to_f16_bits(oracle.normal((1024, 8192), 1, 0, 0.02)))
    b = oracle.from_f16_bits(oracle.to_f16_bits(oracle.normal((1024, 4096), 2, 0, 0.02)))
    ga, gb = dev_tensor(a, gpu, True), dev_tensor(b, gpu, True)
    c = torch.full((8192, 4096), float("nan"), device=gpu, dtype=torch.float16)
    nt.matrix_mul(ga, X_TRANS, gb, X_NOTRANS, c)
    got = c.float().cpu().numpy()
    # every element against double precision (assert_fp16 also wants every element finite: c held NaN)
    assert_fp16(got, whole_f64(a, X_TRANS, b, X_NOTRANS), what="configuration 4, whole result")
    # the fp32 oracle on a block of result rows (columns of the stored a)
    sub = np.ascontiguousarray(a[:, :96])
    assert_fp16(got[:96], oracle.matmul2d(sub, X_TRANS, b, X_NOTRANS))
    # scaling by 2 is exact in half as well, for results that are normal halves
    c2 = torch.empty_like(c)
    nt.matrix_mul(ga, X_TRANS, gb, X_NOTRANS, c2, 2.0)
    normal = c.abs() > 2.0 ** -13      # above the first binade, where a value just below 2^-14 may round up into it
    assert normal.float().mean() > 0.9
    assert bool(torch.isfinite(c2).all())
    assert int((c2[normal] != (2 * c)[normal]).sum()) == 0
    assert torch.equal(c2[normal], (2 * c)[normal])
    # below that, doubling the fp32 sum before the one rounding can differ from doubling the rounded half by a
    # half's smallest step at most
    assert float((c2.float() - 2 * c.float())[~normal].abs().max()) <= 2.0 ** -24


@pytest.mark.parametrize("ta,tb", TRANS)
def test_half_walk_over_more_tiles_than_cus(gpu, oracle, ta, tb):
    """More 256 x 256 tiles than the part has CUs: one workgroup per CU walks over them, fetches the next tile while
    the finished one leaves, and requests k-contiguous operands two slabs at a time. Ragged edges in m and n, a k
    that ends inside a slab and inside a pair of slabs, odd and even numbers of slabs, batches; every element against
    double precision, and to the last half bit against the one-tile-per-workgroup kernels."""
    torch = torch_()
    knobs = ("NTSAMD_TILE_CFG", "NTSAMD_F16_PINGPONG", "NTSAMD_F16_PERSIST")
    try:
        for i, (M, N, K, batch) in enumerate(((4100, 4360, 264, 1), (4360, 4100, 1000, 1), (4352, 4352, 328, 1),
                                              (1100, 1300, 296, 9))):
            a = oracle.from_f16_bits(oracle.to_f16_bits(oracle.normal((batch,) + stored((M, K), ta), 7100 + i, 0, 0.05)))
            b = oracle.from_f16_bits(oracle.to_f16_bits(oracle.normal((batch,) + stored((K, N), tb), 7200 + i, 0, 0.05)))
            ga, gb = dev_tensor(a, gpu, True), dev_tensor(b, gpu, True)
            got = {}
            for walk in (1, 0):
                for key, val in zip(knobs, (2, walk, walk)):
                    nt.tuning_set(key, val)
                c = torch.full((batch, M, N), float("nan"), device=gpu, dtype=torch.float16)
                if batch == 1:
                    nt.matrix_mul(ga[0], ta, gb[0], tb, c[0], 0.75, 0.0)
                else:
                    na, ma = a.shape[1:]
                    nb, mb = b.shape[1:]
                    nt.matrix_mul_batched_strided(ga, ta, gb, tb, c, batch, na * ma, nb * mb, M * N, na, ma, nb, mb, M, N, 0.75, 0.0)
                got[walk] = c
            # the walk multiplies 16 x 16 x 32 blocks, the one-tile kernels 32 x 32 x 16: the same products summed in
            # another order inside the matrix pipe, so a sum next to a rounding boundary may come out one half apart
            w, o = got[1].float(), got[0].float()
            step = torch.maximum(w.abs(), o.abs()) * 2.0 ** -10 + 2.0 ** -24
            assert bool(((w - o).abs() <= step).all()), "%dx%dx%d x%d: the walk and the one-tile kernels differ" % (M, N, K, batch)
            assert float((w != o).float().mean()) < 1e-3
            res = got[1].float().cpu().numpy()
            for item in range(batch):
                assert_fp16(res[item], 0.75 * whole_f64(a[item], ta, b[item], tb), what="%dx%dx%d item %d" % (M, N, K, item))
    finally:
        for key in knobs:
            nt.tuning_set(key, None)


@pytest.mark.parametrize("ta,tb", TRANS)
def test_half_walk_with_a_bias_by_column(gpu, oracle, ta, tb):
    """The linear layer in half on more tiles than CUs (MulAndShift, source/tensor/core/arithmetic/MulAndShift.cpp:
    product, then the bias added along the last dimension), with and without Rectify behind it: the walking kernel
    takes the bias along; every element against double precision (the bias added before the one rounding), to the
    last half bit against the one-tile kernels, ragged edges included (columns past N read no bias)."""
    torch = torch_()
    knobs = ("NTSAMD_TILE_CFG", "NTSAMD_F16_PINGPONG", "NTSAMD_F16_PERSIST")
    try:
        for i, (M, N, K) in enumerate(((4100, 4360, 264), (4352, 4352, 1000))):
            a = oracle.from_f16_bits(oracle.to_f16_bits(oracle.normal(stored((M, K), ta), 7300 + i, 0, 0.05)))
            b = oracle.from_f16_bits(oracle.to_f16_bits(oracle.normal(stored((K, N), tb), 7400 + i, 0, 0.05)))
            bias = oracle.from_f16_bits(oracle.to_f16_bits(oracle.normal((N,), 7500 + i, 0, 0.5)))
            ga, gb, gbias = dev_tensor(a, gpu, True), dev_tensor(b, gpu, True), dev_tensor(bias, gpu, True)
            exact = 0.75 * whole_f64(a, ta, b, tb) + bias.astype(np.float64)[None, :]
            for act in (nt.ACT_NONE, nt.ACT_RECTIFY):
                got = {}
                for walk in (1, 0):
                    for key, val in zip(knobs, (2, walk, walk)):
                        nt.tuning_set(key, val)
                    c = torch.full((M, N), float("nan"), device=gpu, dtype=torch.float16)
                    nt.matrix_mul(ga, ta, gb, tb, c, 0.75, 0.0, bias=gbias, act=act)
                    got[walk] = c
                w, o = got[1].float(), got[0].float()
                step = torch.maximum(w.abs(), o.abs()) * 2.0 ** -10 + 2.0 ** -24
                assert bool(((w - o).abs() <= step).all()), "%dx%dx%d act %d: the walk and the one-tile kernels differ" % (M, N, K, act)
                assert float((w != o).float().mean()) < 1e-3
                want = np.maximum(exact, 0.0) if act == nt.ACT_RECTIFY else exact
                assert_fp16(got[1].float().cpu().numpy(), want, what="%dx%dx%d with bias, act %d" % (M, N, K, act))
    finally:
        for key in knobs:
            nt.tuning_set(key, None)


@pytest.mark.parametrize("tb", (X_NOTRANS, X_TRANS))
def test_half_walk_over_tiles_of_128_rows(gpu, oracle, tb):
    """Results with fewer 256 x 256 tiles than CUs but enough tiles of 128 x 256: the walking kernel on the lower tile
    (a stored row by row). Ragged edges, a k that ends inside a pair of slabs, with and without a bias, a batch;
    every element against double precision, and to the last half bit against the one-tile kernels."""
    torch = torch_()
    ta = X_NOTRANS
    try:
        for i, (M, N, K, batch, with_bias) in enumerate(((4096, 2048, 520, 1, False), (3900, 2100, 264, 1, True),
                                                         (4000, 1800, 1000, 1, True), (1000, 1100, 328, 9, False))):
            a = oracle.from_f16_bits(oracle.to_f16_bits(oracle.normal((batch,) + stored((M, K), ta), 7600 + i, 0, 0.05)))
            b = oracle.from_f16_bits(oracle.to_f16_bits(oracle.normal((batch,) + stored((K, N), tb), 7700 + i, 0, 0.05)))
            bias = oracle.from_f16_bits(oracle.to_f16_bits(oracle.normal((N,), 7800 + i, 0, 0.5)))
            ga, gb = dev_tensor(a, gpu, True), dev_tensor(b, gpu, True)
            gbias = dev_tensor(bias, gpu, True) if with_bias else None
            got = {}
            for walk in (4, 0):
                nt.tuning_set("NTSAMD_F16_PERSIST", walk)
                c = torch.full((batch, M, N), float("nan"), device=gpu, dtype=torch.float16)
                if batch == 1:
                    nt.matrix_mul(ga[0], ta, gb[0], tb, c[0], 0.75, 0.0, bias=gbias)
                else:
                    na, ma = a.shape[1:]
                    nb, mb = b.shape[1:]
                    nt.matrix_mul_batched_strided(ga, ta, gb, tb, c, batch, na * ma, nb * mb, M * N, na, ma, nb, mb, M, N, 0.75, 0.0)
                got[walk] = c
            w, o = got[4].float(), got[0].float()
            step = torch.maximum(w.abs(), o.abs()) * 2.0 ** -10 + 2.0 ** -24
            assert bool(((w - o).abs() <= step).all()), "%dx%dx%d x%d: the walk and the one-tile kernels differ" % (M, N, K, batch)
            assert float((w != o).float().mean()) < 1e-3
            res = w.cpu().numpy()
            for item in range(batch):
                want = 0.75 * whole_f64(a[item], ta, b[item], tb) + (bias.astype(np.float64)[None, :] if with_bias else 0.0)
                assert_fp16(res[item], want, what="%dx%dx%d item %d" % (M, N, K, item))
    finally:
        nt.tuning_set("NTSAMD_F16_PERSIST", None)


@pytest.mark.parametrize("ta,tb", TRANS)
def test_half_walk_that_adds_to_the_old_result(gpu, oracle, ta, tb):
    """beta != 0 on more tiles than CUs (the gradient products of source/network/XBackwardMath.cpp all add to what the
    gradient tensor holds): the walking kernel reads the old c on its way out and adds it in fp32 before the one
    rounding. Tiles of 256 rows in every layout and of 128 rows where a is stored row by row; every element against
    double precision, and to the last half bit against the one-tile kernels."""
    torch = torch_()
    try:
        cases = [(4100, 4360, 264, 2, 1.0), (4352, 4352, 1000, 2, 0.5)]
        if ta == X_NOTRANS:
            cases.append((3900, 2100, 1032, 4, 1.0))
        for i, (M, N, K, walk, beta) in enumerate(cases):
            a = oracle.from_f16_bits(oracle.to_f16_bits(oracle.normal(stored((M, K), ta), 9300 + i, 0, 0.05)))
            b = oracle.from_f16_bits(oracle.to_f16_bits(oracle.normal(stored((K, N), tb), 9400 + i, 0, 0.05)))
            c0 = oracle.from_f16_bits(oracle.to_f16_bits(oracle.normal((M, N), 9500 + i, 0, 0.5)))
            ga, gb = dev_tensor(a, gpu, True), dev_tensor(b, gpu, True)
            got = {}
            for knob in (walk, 0):
                nt.tuning_set("NTSAMD_F16_PERSIST", knob)
                nt.tuning_set("NTSAMD_TILE_CFG", 2 if knob else None)
                c = dev_tensor(c0, gpu, True)
                nt.matrix_mul(ga, ta, gb, tb, c, 0.75, beta)
                got[knob] = c
            w, o = got[walk].float(), got[0].float()
            step = torch.maximum(w.abs(), o.abs()) * 2.0 ** -10 + 2.0 ** -24
            assert bool(((w - o).abs() <= step).all()), "%dx%dx%d: the walk and the one-tile kernels differ" % (M, N, K)
            assert float((w != o).float().mean()) < 1e-3
            assert_fp16(w.cpu().numpy(), 0.75 * whole_f64(a, ta, b, tb) + beta * c0.astype(np.float64), what="%dx%dx%d beta %g" % (M, N, K, beta))
    finally:
        nt.tuning_set("NTSAMD_F16_PERSIST", None)
        nt.tuning_set("NTSAMD_TILE_CFG", None)


def test_config5_ragged_vocab_projection(gpu, oracle):
    """fp32 H[4096x512] x W[30011x512]^T accumulated into C[4096x30011] with beta = 1."""
    torch = torch_()
    h = oracle.uniform((4096, 512), 1)
    w = oracle.normal((30011, 512), 2, 0, 0.02)
    c0 = oracle.uniform((4096, 30011), 3)
    gh, gw = dev_tensor(h, gpu), dev_tensor(w, gpu)
    c = dev_tensor(c0, gpu)
    nt.matrix_mul(gh, X_NOTRANS, gw, X_TRANS, c, 1.0, 1.0)
    got = c.cpu().numpy()
    # every element against double precision, under both measures
    prod = whole_f64(h, X_NOTRANS, w, X_TRANS)
    mag = library_magnitude(gpu, h, X_NOTRANS, w, X_TRANS) + np.abs(c0)
    assert_fp32(got, prod + c0, 512, mag, what="configuration 5, whole result")
    # the oracle on the last rows (the ragged right edge is in every row)
    ref = oracle.matmul2d(h[-24:].copy(), X_NOTRANS, w, X_TRANS, c0[-24:].copy(), 1.0, 1.0)
    assert_fp32(got[-24:], ref, 512)
    # accumulate once more: c + h w^T again = c0 + 2 h w^T
    nt.matrix_mul(gh, X_NOTRANS, gw, X_TRANS, c, 1.0, 1.0)
    assert_fp32(c.cpu().numpy(), 2 * prod + c0, 512, 2 * mag, what="configuration 5 accumulated twice, whole result")


def test_a_batch_with_too_many_tiles_is_refused(gpu):
    """Workgroups are numbered with 32-bit integers: a batch that would not fit is an argument error, found
    before anything is launched (the strides below lie about the size of the tensors; nothing reads them)."""
    torch = torch_()
    t = torch.zeros(1024, device=gpu)
    with pytest.raises(nt.NtsAmdError, match="too many tiles"):
        nt.matrix_mul_batched_strided(t, X_NOTRANS, t, X_NOTRANS, t, 1 << 27, 0, 0, 1024, 32, 32, 32, 32, 32, 32)


def test_rectified_linear_layer_at_full_size(gpu, oracle):
    """Configuration 2's layer with the activation in the epilogue: bit for bit the maximum of zero and the
    layer without it (the activation is applied to the same fp32 value the plain epilogue stores)."""
    torch = torch_()
    x = dev_tensor(oracle.uniform((4096, 512), 1), gpu)
    w = dev_tensor(oracle.normal((512, 2048), 2, 0, 0.02), gpu)
    b = dev_tensor(oracle.normal((2048,), 3, 0, 0.02), gpu)
    plain = torch.empty((4096, 2048), device=gpu)
    rect = torch.full((4096, 2048), float("nan"), device=gpu)
    nt.matrix_mul(x, X_NOTRANS, w, X_NOTRANS, plain, bias=b)
    nt.matrix_mul(x, X_NOTRANS, w, X_NOTRANS, rect, bias=b, act=nt.ACT_RECTIFY)
    torch.cuda.synchronize()
    assert torch.equal(rect, torch.clamp_min(plain, 0.0))
    assert 0.3 < (rect == 0).float().mean().item() < 0.7



@pytest.mark.parametrize("half,M,N,K,tb,beta", [
    (True, 70000, 32768, 256, X_NOTRANS, 0.5),      # c: 4.6 GB, the walking kernel with the old c
    (True, 2200000, 1024, 64, X_TRANS, 0.0),        # 2.2 million rows: the last rows start past 2^32 bytes
    (False, 40000, 30011, 64, X_TRANS, 1.0),        # c: 4.8 GB of rows that are only 4-byte aligned
])
def test_results_of_more_than_four_gigabytes(gpu, half, M, N, K, tb, beta):
    """A tile's base is a 64-bit address and only the offsets inside the tile's window are 32-bit: rows at the start,
    in the middle and at the very end of a result of more than 2^32 bytes against float64 (the size-independent
    check: the oracle would take minutes here), and no element of the first and the last 4096 rows left unwritten."""
    torch = torch_()
    dt = torch.float16 if half else torch.float32
    gen = torch.Generator(device=gpu).manual_seed(5)
    a = torch.randn((M, K), device=gpu, generator=gen).to(dt)
    b = torch.randn((N, K) if tb == X_TRANS else (K, N), device=gpu, generator=gen).to(dt)
    c = torch.randn((M, N), device=gpu, generator=gen).to(dt) if beta else torch.full((M, N), float("nan"), device=gpu, dtype=dt)
    rows = torch.tensor([0, 1, M // 2, M // 2 + 77, M - 2, M - 1], device=gpu)
    old = c[rows].double() if beta else 0.0
    nt.matrix_mul(a, X_NOTRANS, b, tb, c, 1.0, beta)
    torch.cuda.synchronize()
    ref = a[rows].double() @ (b.double().t() if tb == X_TRANS else b.double()) + beta * old
    err = float((c[rows].double() - ref).abs().max() / ref.abs().max())
    assert err <= (FP16_LIMIT if half else fp32_limit(K)), (err, nt.last_plan())
    assert bool(torch.isfinite(c[:4096]).all()) and bool(torch.isfinite(c[M - 4096:]).all())
