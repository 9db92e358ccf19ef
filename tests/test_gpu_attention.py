"""Parity of the one-kernel attention (ntsamd_attention) with the CPU oracle's restatement of
the reference's operator chain (Split, Scale, BMMul(q, k^T), Sum with the mask, Softmax,
BMMul with v, Merge), through the C ABI.

Limit: fp32, normwise error at most 1e-5 sqrt(K) with K = dh + lk (the two contractions a
result element passes through); the probabilities come from expf on both sides.
"""
import numpy as np
import pytest

import niutensor_amd as nt
from niutensor_amd import X_NOTRANS
from tolerance import FP16_LIMIT, assert_fp32, normwise, scaled

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


def run(gpu, q, k, v, heads, scale, mask=None):
    torch = torch_()
    out = torch.full(q.shape, float("nan"), device=gpu)
    nt.attention(dev(q, gpu), dev(k, gpu), dev(v, gpu), out, heads, scale, mask=dev(mask, gpu) if mask is not None else None)
    torch.cuda.synchronize()
    return out.cpu().numpy()


def test_fixtures_of_the_compiled_reference(gpu, generated_attention):
    names = generated_attention.of_kind("attention")
    assert len(names) == 9
    for name in names:
        d = generated_attention.case(name)
        heads, scale = int(d["params"][0]), float(d["scal"][0])
        dh = d["q"].shape[2] // heads
        if dh % 4 != 0 or dh > 128:
            pytest.fail("fixture %s has a head size the kernel refuses" % name)
        got = run(gpu, d["q"], d["k"], d["v"], heads, scale, d.get("mask"))
        assert_fp32(got, d["out"], dh + d["k"].shape[1], what=name)


@pytest.mark.parametrize("B,lq,lk,H,nh,masked", [
    (2, 128, 128, 128, 2, False),      # one key block, head size 64
    (3, 100, 77, 96, 3, True),         # ragged rows and keys, head size 32
    (1, 300, 513, 64, 1, True),        # several query tiles and key blocks
    (2, 40, 260, 256, 2, False),       # head size 128
    (2, 33, 65, 192, 2, True),         # head size 96 inside the 128 kernel
    (4, 9, 5, 8, 2, False),            # head size 4
    (1, 1, 1, 12, 1, False),           # a single score
    (3, 70, 64, 192, 3, True),         # short sentences: the second half of the key block holds no key
    (2, 50, 33, 64, 2, False),
])
def test_against_oracle(gpu, oracle, B, lq, lk, H, nh, masked):
    q, k, v = oracle.normal((B, lq, H), 11), oracle.normal((B, lk, H), 12), oracle.normal((B, lk, H), 13)
    mask = None
    if masked:
        mask = np.where(oracle.uniform((nh, B, lq, lk), 14, 0.0, 1.0) < 0.3, -1e9, 0.0).astype(np.float32)
        mask[..., lk // 2] = 0.0
    scale = float(np.float32(1.0 / np.sqrt(H // nh)))
    ref = oracle.attention(q, k, v, nh, scale, mask)
    got = run(gpu, q, k, v, nh, scale, mask)
    assert_fp32(got, ref, H // nh + lk, what=str((B, lq, lk, H, nh, masked)))


def test_rows_with_every_key_masked_and_large_scores(gpu, oracle):
    """A row whose mask is -1e9 everywhere comes out as the mean of v (scores below 32 vanish
    beside -1e9 in fp32, on both sides); scores of a few hundred do not overflow."""
    B, lq, lk, H, nh = 1, 70, 140, 64, 2
    q, k, v = oracle.normal((B, lq, H), 21), oracle.normal((B, lk, H), 22), oracle.normal((B, lk, H), 23)
    mask = np.zeros((nh, B, lq, lk), np.float32)
    mask[:, :, 3, :] = -1e9
    mask[:, :, 69, 1:] = -1e9
    ref = oracle.attention(q, k, v, nh, 0.5, mask)
    got = run(gpu, q, k, v, nh, 0.5, mask)
    assert_fp32(got, ref, 32 + lk, what="masked rows")
    assert np.abs(got[0, 3] - v[0].mean(0)).max() <= 1e-5
    assert np.array_equal(got[0, 69], v[0, 0])
    q, k = oracle.normal((B, lq, H), 24, 0.0, 3.0), oracle.normal((B, lk, H), 25, 0.0, 3.0)
    ref = oracle.attention(q, k, v, nh, 1.0)
    got = run(gpu, q, k, v, nh, 1.0)
    assert_fp32(got, ref, 32 + lk, what="large scores")


def test_split_layout_and_stream(gpu, oracle):
    """Tensors stored [heads][batch][rows][dh], as after the reference's Split, on a stream of the
    caller: same numbers as the merged layout."""
    torch = torch_()
    B, lq, lk, H, nh = 3, 50, 70, 64, 4
    dh = H // nh
    q, k, v = oracle.normal((B, lq, H), 31), oracle.normal((B, lk, H), 32), oracle.normal((B, lk, H), 33)
    ref = oracle.attention(q, k, v, nh, 0.25)
    sp = lambda x: np.ascontiguousarray(x.reshape(x.shape[0], x.shape[1], nh, dh).transpose(2, 0, 1, 3))
    s = torch.cuda.Stream()
    with torch.cuda.stream(s):
        qd, kd, vd = dev(sp(q), gpu), dev(sp(k), gpu), dev(sp(v), gpu)
        out = torch.full((nh, B, lq, dh), float("nan"), device=gpu)
        nt.attention(qd, kd, vd, out, nh, 0.25, split=True)
    s.synchronize()
    got = out.cpu().numpy().transpose(1, 2, 0, 3).reshape(B, lq, H)
    assert_fp32(got, ref, dh + lk, what="split layout")


def test_attention_shape_of_the_benchmark(gpu, oracle):
    """32 sentences x 8 heads, 128 positions, head size 64: against the oracle, and against the
    two batched products with torch's softmax between them."""
    torch = torch_()
    B, L, H, nh = 32, 128, 512, 8
    q, k, v = oracle.normal((B, L, H), 41), oracle.normal((B, L, H), 42), oracle.normal((B, L, H), 43)
    ref = oracle.attention(q, k, v, nh, 0.125)
    got = run(gpu, q, k, v, nh, 0.125)
    assert_fp32(got, ref, 64 + L, what="benchmark shape")
    # properties at full size: rows of v all equal -> the output repeats that row exactly enough
    vc = np.broadcast_to(oracle.normal((B, 1, H), 44), (B, L, H)).copy()
    got = run(gpu, q, k, vc, nh, 0.125)
    assert np.abs(got - vc).max() <= 1e-5 * np.abs(vc).max() * 4


@pytest.mark.parametrize("B,lq,lk,H,nh,masked", [
    (2, 128, 128, 128, 2, False),      # one key block: one pass
    (3, 100, 77, 96, 3, True),         # ragged rows and keys: scalar stores
    (1, 300, 516, 64, 1, True),        # several key blocks: two passes, 16-byte stores
    (2, 40, 261, 256, 2, False),       # head size 128, ragged
    (4, 9, 5, 8, 2, False),            # head size 4
    (1, 1, 1, 12, 1, False),
    (3, 70, 64, 192, 3, True),         # short sentences: blocks of 64 keys, 16-byte stores
    (2, 50, 33, 64, 2, False),         # the same, ragged
])
def test_probabilities_against_oracle(gpu, oracle, B, lq, lk, H, nh, masked):
    """The first half on its own (what the training path keeps): softmax(scale q k^T + mask) as a
    [heads][batch][lq][lk] tensor, against the oracle's Split, Scale, BMMul, Sum, Softmax."""
    torch = torch_()
    q, k = oracle.normal((B, lq, H), 71), oracle.normal((B, lk, H), 72)
    mask = None
    if masked:
        mask = np.where(oracle.uniform((nh, B, lq, lk), 73, 0.0, 1.0) < 0.3, -1e9, 0.0).astype(np.float32)
        mask[..., lk // 2] = 0.0
    scale = float(np.float32(1.0 / np.sqrt(H // nh)))
    ref = oracle.attention_probs(q, k, nh, scale, mask)
    probs = torch.full((nh, B, lq, lk), float("nan"), device=gpu)
    nt.attention_probs(dev(q, gpu), dev(k, gpu), probs, nh, scale, mask=dev(mask, gpu) if masked else None)
    torch.cuda.synchronize()
    got = probs.cpu().numpy()
    # probabilities: absolute error against a largest value of at most 1, and rows that sum to 1
    assert np.isfinite(got).all()
    assert np.abs(got - ref).max() <= 1e-5 * np.sqrt(H // nh)
    assert np.abs(got.sum(-1, dtype=np.float64) - 1).max() <= 1e-5
    if masked:
        assert (got[mask < 0] == 0).all()
    # followed by the second product it gives the attention of the one-kernel path
    v = oracle.normal((B, lk, H), 74)
    whole = run(gpu, q, k, v, nh, scale, mask)
    vh = v.reshape(B, lk, nh, H // nh).transpose(2, 0, 1, 3).astype(np.float64)
    two_step = (got.astype(np.float64) @ vh).transpose(1, 2, 0, 3).reshape(B, lq, H)
    assert np.abs(whole - two_step).max() <= 1e-5 * np.sqrt(H // nh + lk) * np.abs(two_step).max()


@pytest.mark.parametrize("B,lq,lk,H,nh,masked,dropout", [
    (2, 128, 128, 128, 2, False, True),     # one key block, 16-byte moves
    (3, 100, 77, 96, 3, True, True),        # ragged rows and keys: scalar moves
    (1, 300, 516, 64, 1, True, True),       # several key blocks: a first pass for the maxima and sums
    (2, 40, 261, 256, 2, False, True),      # head size 128, ragged
    (4, 9, 5, 8, 2, False, False),          # head size 4, no dropout
    (2, 70, 200, 128, 4, True, False),
    (3, 70, 64, 192, 3, True, True),        # short sentences: blocks of 64 keys
    (2, 50, 33, 64, 2, False, True),
])
def test_training_path_in_one_launch(gpu, oracle, B, lq, lk, H, nh, masked, dropout):
    """ntsamd_attention_train against the operator chain of the reference's training path put together from the
    oracle's pieces: probabilities from the oracle's Split, Scale, BMMul, Sum, Softmax (oracle_attention_probs);
    Dropout as the element-wise product with a mask of 0 and 1 / (1 - p) (the reference's Dropout is exactly that
    product); the oracle's batched product with the split values; the merge. The probabilities must also be what
    ntsamd_attention_probs writes, bit for bit where both make one pass."""
    torch = torch_()
    print("\n[gpu-case] attention_train B=%d lq=%d lk=%d H=%d heads=%d mask=%d dropout=%d" % (B, lq, lk, H, nh, masked, dropout), flush=True)
    q, k, v = oracle.normal((B, lq, H), 81), oracle.normal((B, lk, H), 82), oracle.normal((B, lk, H), 83)
    mask = None
    if masked:
        mask = np.where(oracle.uniform((nh, B, lq, lk), 84, 0.0, 1.0) < 0.3, -1e9, 0.0).astype(np.float32)
        mask[..., lk // 2] = 0.0
    drop = None
    if dropout:
        drop = np.where(oracle.uniform((nh, B, lq, lk), 85, 0.0, 1.0) < 0.1, 0.0, 1.0 / 0.9).astype(np.float32)
    scale = float(np.float32(1.0 / np.sqrt(H // nh)))
    dh = H // nh
    p_ref = oracle.attention_probs(q, k, nh, scale, mask)
    d_ref = p_ref * drop if dropout else p_ref
    vh = np.ascontiguousarray(v.reshape(B, lk, nh, dh).transpose(2, 0, 1, 3))
    c_ref = oracle.matmul_batched(d_ref.reshape(nh * B, lq, lk), X_NOTRANS, vh.reshape(nh * B, lk, dh), X_NOTRANS)
    o_ref = c_ref.reshape(nh, B, lq, dh).transpose(1, 2, 0, 3).reshape(B, lq, H)

    nan = lambda *shape: torch.full(shape, float("nan"), device=gpu)
    probs, dropped, out = nan(nh, B, lq, lk), (nan(nh, B, lq, lk) if dropout else None), nan(B, lq, H)
    nt.attention_train(dev(q, gpu), dev(k, gpu), dev(v, gpu), probs, out, nh, scale, mask=dev(mask, gpu) if masked else None,
                       drop_mask=dev(drop, gpu) if dropout else None, dropped=dropped)
    torch.cuda.synchronize()
    got_p, got_o = probs.cpu().numpy(), out.cpu().numpy()
    assert np.isfinite(got_p).all() and np.isfinite(got_o).all()
    assert np.abs(got_p - p_ref).max() <= 1e-5 * np.sqrt(dh)
    assert np.abs(got_p.sum(-1, dtype=np.float64) - 1).max() <= 1e-5
    if dropout:
        got_d = dropped.cpu().numpy()
        assert np.isfinite(got_d).all()
        assert np.array_equal(got_d, got_p * drop)              # one fp32 product per element, as Multiply does it
        assert (got_d[drop == 0] == 0).all()
    assert np.abs(got_o - o_ref).max() <= 1e-5 * np.sqrt(dh + lk) * np.abs(o_ref).max()
    # the probabilities on their own: the same kernel arithmetic
    alone = nan(nh, B, lq, lk)
    nt.attention_probs(dev(q, gpu), dev(k, gpu), alone, nh, scale, mask=dev(mask, gpu) if masked else None)
    assert np.abs(alone.cpu().numpy() - got_p).max() <= 2e-7
    # without dropout the result is the attention of the one-kernel path
    if not dropout:
        whole = run(gpu, q, k, v, nh, scale, mask)
        assert np.abs(whole - got_o).max() <= 1e-5 * np.sqrt(dh + lk) * np.abs(o_ref).max()


def halfed(oracle, x):
    return oracle.from_f16_bits(oracle.to_f16_bits(x))


def assert_half(got, ref, mag, what):
    """Limit 1e-2 (half against the fp32 reference), measured norm-wise and component-wise against
    mag = sum_k p_k |v_k|: a result element is a sum of probabilities times values, each probability
    enters the second product rounded to half (as in the reference's half path), so its error is a
    multiple of 2^-11 mag however much of the sum cancels."""
    assert np.isfinite(got).all(), what
    e = normwise(got, ref)
    assert e <= FP16_LIMIT, "%s: normwise error %.3g > %.3g" % (what, e, FP16_LIMIT)
    e = scaled(got, ref, mag)
    assert e <= FP16_LIMIT, "%s: component-wise error %.3g > %.3g" % (what, e, FP16_LIMIT)


def run_half(gpu, q, k, v, heads, scale, mask=None):
    torch = torch_()
    out = torch.full(q.shape, float("nan"), device=gpu, dtype=torch.float16)
    nt.attention(dev(q, gpu).half(), dev(k, gpu).half(), dev(v, gpu).half(), out, heads, scale,
                 mask=dev(mask, gpu) if mask is not None else None)
    torch.cuda.synchronize()
    return out.float().cpu().numpy()


@pytest.mark.parametrize("B,lq,lk,H,nh,masked", [
    (2, 128, 128, 128, 2, False),      # head size 64, one key block
    (3, 100, 77, 96, 3, True),         # head size 32, ragged rows and keys
    (1, 300, 513, 64, 1, True),        # several query tiles and key blocks
    (2, 40, 260, 256, 2, False),       # head size 128
    (2, 33, 65, 80, 2, True),          # head size 40 inside the 64 kernel
    (4, 9, 5, 16, 2, False),           # head size 8
    (1, 1, 1, 8, 1, False),            # a single score
    (3, 70, 64, 192, 3, True),         # short sentences: blocks of 64 keys
    (2, 50, 33, 256, 2, False),        # the same with heads of 128, ragged
])
def test_half_against_oracle(gpu, oracle, B, lq, lk, H, nh, masked):
    """Half tensors: the fp32 oracle on the half-rounded inputs, result within 1e-2 (the limit the
    task statement sets for half against the fp32 reference)."""
    q, k, v = (halfed(oracle, oracle.normal(s, seed)) for s, seed in (((B, lq, H), 51), ((B, lk, H), 52), ((B, lk, H), 53)))
    mask = None
    if masked:
        mask = np.where(oracle.uniform((nh, B, lq, lk), 54, 0.0, 1.0) < 0.3, -1e9, 0.0).astype(np.float32)
        mask[..., lk // 2] = 0.0
    scale = float(np.float32(1.0 / np.sqrt(H // nh)))
    ref = oracle.attention(q, k, v, nh, scale, mask)
    mag = oracle.attention(q, k, np.abs(v), nh, scale, mask)
    got = run_half(gpu, q, k, v, nh, scale, mask)
    assert_half(got, ref, mag, str((B, lq, lk, H, nh, masked)))


@pytest.mark.parametrize("B,lq,lk,H,nh,masked", [
    (4, 1000, 136, 1024, 16, True),    # head size 64, 512 workgroups of 128 rows, a ragged last block of 64 keys
    (32, 520, 70, 128, 4, False),      # head size 32, a last workgroup with 8 live rows
    (8, 1000, 136, 1024, 8, True),     # head size 128
    (8, 900, 200, 832, 8, False),      # head size 104 in the kernel built for 128
])
def test_half_with_two_blocks_of_query_rows_per_wave(gpu, oracle, B, lq, lk, H, nh, masked):
    """Long sequences in half run with 128 query rows per workgroup, two blocks of 16 per wave against blocks of 64
    keys (taken when such workgroups still give every CU two): against the oracle like the other half cases, and
    bit for bit the same rows when the sentences are fed in two halves that are too few for that form."""
    q, k, v = (halfed(oracle, oracle.normal(s, seed)) for s, seed in (((B, lq, H), 71), ((B, lk, H), 72), ((B, lk, H), 73)))
    mask = None
    if masked:
        mask = np.where(oracle.uniform((nh, B, lq, lk), 74, 0.0, 1.0) < 0.3, -1e9, 0.0).astype(np.float32)
        mask[..., lk // 2] = 0.0
    scale = float(np.float32(1.0 / np.sqrt(H // nh)))
    assert nh * B * ((lq + 127) // 128) >= 512
    ref = oracle.attention(q, k, v, nh, scale, mask)
    mag = oracle.attention(q, k, np.abs(v), nh, scale, mask)
    got = run_half(gpu, q, k, v, nh, scale, mask)
    assert_half(got, ref, mag, str((B, lq, lk, H, nh, masked)))
    # the one-block form on a part of the batch: the same arithmetic per row up to the order of the key blocks, so the
    # rows agree to the limit as well
    part = run_half(gpu, q[:1], k[:1], v[:1], nh, scale, None if mask is None else np.ascontiguousarray(mask[:, :1]))
    assert_half(part, ref[:1], mag[:1], "one sentence of " + str((B, lq, lk, H, nh, masked)))


def test_half_exact_cases_and_benchmark_shape(gpu, oracle):
    torch = torch_()
    # one key: probabilities exactly 1, the result is v's row, bit for bit
    B, lq, H, nh = 2, 70, 64, 2
    q, k1, v1 = halfed(oracle, oracle.normal((B, lq, H), 61)), halfed(oracle, oracle.normal((B, 1, H), 62)), halfed(oracle, oracle.normal((B, 1, H), 63))
    got = run_half(gpu, q, k1, v1, nh, 0.3)
    assert np.array_equal(got, np.broadcast_to(v1, (B, lq, H)))
    # scale 0: uniform probabilities (1/64 is exact in half), the result is the mean of v's rows
    k, v = halfed(oracle, oracle.normal((B, 64, H), 64)), halfed(oracle, oracle.normal((B, 64, H), 65))
    got = run_half(gpu, q, k, v, nh, 0.0)
    mean = v.astype(np.float64).mean(1, keepdims=True)
    assert np.abs(got - mean).max() <= 2e-3 * np.abs(mean).max() + 1e-3
    # 32 sentences x 8 heads x 128 positions, head size 64; and the split layout gives the same bits
    B, L, H, nh = 32, 128, 512, 8
    q, k, v = (halfed(oracle, oracle.normal((B, L, H), s)) for s in (66, 67, 68))
    ref = oracle.attention(q, k, v, nh, 0.125)
    got = run_half(gpu, q, k, v, nh, 0.125)
    assert_half(got, ref, oracle.attention(q, k, np.abs(v), nh, 0.125), "benchmark shape, half")
    sp = lambda x: np.ascontiguousarray(x.reshape(B, L, nh, 64).transpose(2, 0, 1, 3))
    out = torch.full((nh, B, L, 64), float("nan"), device=gpu, dtype=torch.float16)
    nt.attention(dev(sp(q), gpu).half(), dev(sp(k), gpu).half(), dev(sp(v), gpu).half(), out, nh, 0.125, split=True)
    torch.cuda.synchronize()
    assert np.array_equal(out.float().cpu().numpy().transpose(1, 2, 0, 3).reshape(B, L, H), got)


def test_bad_arguments_are_refused(gpu):
    torch = torch_()
    L = nt.load()
    import ctypes as C
    t = torch.zeros(4096, device=gpu)
    st = (C.c_longlong * 12)(*([8, 64, 8] * 4))
    p = t.data_ptr()
    assert L.ntsamd_attention(0, None, p, p, p, None, p, 4, 1, 1, 8, 8, 8, st, 1.0) == 2           # double: not served
    st4 = (C.c_longlong * 12)(*([4, 64, 4] * 4))
    assert L.ntsamd_attention(0, None, p, p, p, None, p, 3, 1, 1, 8, 8, 4, st4, 1.0) != 0          # half: head size 4
    assert L.ntsamd_attention(0, None, p, p, p, None, p, 2, 1, 1, 8, 8, 6, st, 1.0) != 0           # head size 6
    assert L.ntsamd_attention(0, None, p, p, p, None, p, 2, 1, 1, 8, 8, 132, st, 1.0) != 0         # head size 132
    assert L.ntsamd_attention(0, None, p, p, p, None, p, 2, 1, 1, 8, 0, 8, st, 1.0) != 0           # no keys
    assert L.ntsamd_attention(0, None, p, p, p, None, p, 2, 0, 1, 8, 8, 8, st, 1.0) == 0           # nothing to do
    bad = (C.c_longlong * 12)(*([8, 64, 6] * 4))
    assert L.ntsamd_attention(0, None, p, p, p, None, p, 2, 1, 1, 8, 8, 8, bad, 1.0) != 0          # unaligned rows


def test_probabilities_at_the_benchmark_shape(gpu, oracle):
    """32 sentences x 8 heads, 128 x 128 scores per head: every row sums to 1, the probabilities times v equal
    the one-kernel attention (two independent kernels for the same chain), and one head against the oracle."""
    torch = torch_()
    B, L, H, nh = 32, 128, 512, 8
    q, k, v = oracle.normal((B, L, H), 91), oracle.normal((B, L, H), 92), oracle.normal((B, L, H), 93)
    qd, kd, vd = dev(q, gpu), dev(k, gpu), dev(v, gpu)
    probs = torch.full((nh, B, L, L), float("nan"), device=gpu)
    nt.attention_probs(qd, kd, probs, nh, 0.125)
    torch.cuda.synchronize()
    p = probs.cpu().numpy()
    assert np.isfinite(p).all() and (p >= 0).all()
    assert np.abs(p.sum(-1) - 1.0).max() <= 1e-5
    out = torch.empty((B, L, H), device=gpu)
    nt.attention(qd, kd, vd, out, nh, 0.125)
    ctx = torch.empty((B, L, H), device=gpu)
    dh = H // nh
    nt.matrix_mul_batched_grid(probs, nt.X_NOTRANS, L, (L * L, B * L * L), vd, nt.X_NOTRANS, H, (L * H, dh),
                               ctx, H, (L * H, dh), B, nh, L, L, L, dh, L, dh)
    torch.cuda.synchronize()
    assert_fp32(ctx.cpu().numpy(), out.cpu().numpy(), dh + L, what="probabilities x v against the one kernel")
    ref = oracle.attention_probs(q[3:4], k[3:4], nh, 0.125)
    assert_fp32(p[:, 3:4], ref, dh, what="sentence 3")


@pytest.mark.parametrize("B,lq,lk,H,nh,masked", [
    (16, 1, 100, 512, 8, False),       # one new position against 100 cached ones
    (5, 1, 1, 64, 2, False),           # the first step: one key
    (3, 8, 77, 96, 3, True),           # eight rows (the most this kernel takes), ragged keys, masked
    (2, 4, 700, 256, 2, True),         # head size 128, more keys than lanes
    (7, 3, 33, 24, 2, False),          # head size 12: lanes without columns
])
def test_a_handful_of_query_rows(gpu, oracle, B, lq, lk, H, nh, masked):
    """Up to eight query rows per head (a decoding step) run on the kernel that reads k and v once and
    multiplies in the vector ALU; the same inputs through the MFMA kernel (NTSAMD_ATTN_ROWS=0) must meet
    the same limit against the oracle."""
    q, k, v = oracle.normal((B, lq, H), 61), oracle.normal((B, lk, H), 62), oracle.normal((B, lk, H), 63)
    mask = None
    if masked:
        mask = np.where(oracle.uniform((nh, B, lq, lk), 64, 0.0, 1.0) < 0.3, -1e9, 0.0).astype(np.float32)
        mask[..., 0] = 0.0
    scale = 1.0 / np.sqrt(H // nh)
    ref = oracle.attention(q, k, v, nh, scale, mask)
    for rows in ("1", "0"):
        nt.tuning_set("NTSAMD_ATTN_ROWS", rows)
        try:
            got = run(gpu, q, k, v, nh, scale, mask)
        finally:
            nt.tuning_set("NTSAMD_ATTN_ROWS", None)
        assert_fp32(got, ref, H // nh + lk, what="rows kernel" if rows == "1" else "MFMA kernel")

