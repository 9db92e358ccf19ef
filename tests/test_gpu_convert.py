"""Parity of ntsamd_convert_data_type with the CPU oracle, through the C ABI: bit-exact for all
four conversions, at every alignment, for every half pattern; and the pipeline of the
reference's TConvertDataType case 3 (convert, half product, convert back) with its known answer."""
import ctypes as C

import numpy as np
import pytest

import niutensor_amd as nt
from oracle.binding import X_FLOAT, X_FLOAT16, X_INT

pytestmark = pytest.mark.gpu

TORCH_OF = {X_FLOAT: "float32", X_FLOAT16: "float16", X_INT: "int32"}


def torch_():
    import torch
    return torch


@pytest.fixture(autouse=True)
def name_the_case(request):
    print("\n[gpu-case] %s" % request.node.nodeid, flush=True)
    yield


def to_dev(x, gpu):
    """numpy float32 / int32 / uint16 (half bit patterns) -> device tensor of the matching torch type"""
    torch = torch_()
    if x.dtype == np.uint16:
        return torch.from_numpy(x.view(np.int16).copy()).to(gpu).view(torch.float16)
    return torch.from_numpy(np.ascontiguousarray(x)).to(gpu)


def to_host(t):
    torch = torch_()
    if t.dtype == torch.float16:
        return t.view(torch.int16).cpu().numpy().view(np.uint16)
    return t.cpu().numpy()


def run(gpu, x, type_t, offset=0):
    """convert on the GPU; offset (elements) moves both arrays off their 16-byte alignment"""
    torch = torch_()
    src_full = to_dev(np.concatenate([np.zeros(offset, x.dtype), x.ravel()]), gpu)
    dst_full = torch.zeros(offset + x.size + 8, dtype=getattr(torch, TORCH_OF[type_t]), device=gpu)
    nt.convert_data_type(src_full[offset:offset + x.size], dst_full[offset:offset + x.size])
    torch.cuda.synchronize()
    out = to_host(dst_full)
    assert not out[:offset].any() and not out[offset + x.size:].any(), "wrote outside the array"
    return out[offset:offset + x.size].reshape(x.shape)


def test_every_half_pattern_and_back(gpu, oracle):
    bits = np.arange(65536, dtype=np.uint16)
    wide = run(gpu, bits, X_FLOAT)
    ref = oracle.convert(bits, X_FLOAT)
    assert np.array_equal(wide.view(np.uint32)[~np.isnan(ref)], ref.view(np.uint32)[~np.isnan(ref)])
    assert np.isnan(wide[np.isnan(ref)]).all()
    finite = ~np.isnan(ref)
    back = run(gpu, ref, X_FLOAT16)
    assert np.array_equal(back[finite], bits[finite])


@pytest.mark.parametrize("n,offset", [(1, 0), (7, 0), (8, 0), (1000003, 0), (4099, 1), (65536, 3), (257, 5)])
def test_four_conversions_against_oracle(gpu, oracle, n, offset):
    rng = np.random.default_rng(n + offset)
    x = (rng.standard_normal(n) * np.exp(rng.uniform(-18, 12, n))).astype(np.float32)
    x[:: 97] = np.float32(65520.0)                   # rounds to infinity in half
    x[1:: 89] = np.float32(3.1e-8)                   # below half's smallest sub-normal / 2
    x[2:: 83] = np.arange(len(x[2:: 83]), dtype=np.float32) + 2048.5     # ties
    got = run(gpu, x, X_FLOAT16, offset)
    assert np.array_equal(got, oracle.convert(x, X_FLOAT16))
    h = rng.integers(0, 65536, n).astype(np.uint16)
    h[(h & 0x7c00) == 0x7c00] = 0x3c00                # NaN payloads are not compared
    assert np.array_equal(run(gpu, h, X_FLOAT, offset).view(np.uint32), oracle.convert(h, X_FLOAT).view(np.uint32))
    f = (rng.standard_normal(n) * 10 ** rng.uniform(0, 11, n)).astype(np.float32)
    f[:: 101] = np.nan
    f[1:: 103] = np.inf
    f[2:: 107] = -np.inf
    assert np.array_equal(run(gpu, f, X_INT, offset), oracle.convert(f, X_INT))
    i = rng.integers(-2**31, 2**31 - 1, n).astype(np.int32)
    assert np.array_equal(run(gpu, i, X_FLOAT, offset).view(np.uint32), oracle.convert(i, X_FLOAT).view(np.uint32))


def test_pipeline_of_the_reference_test(gpu):
    """TConvertDataType.cpp:214-268: float -> half, half product, half -> float, answer :243-245."""
    torch = torch_()
    d1 = torch.tensor([[1.0, -2.0], [0.5, -4.0], [0.0, 6.0]], device=gpu)
    d2 = torch.tensor([[1.0, 2.0, 3.0], [0.0, 4.0, 5.0]], device=gpu)
    answer = np.array([[1.0, -6.0, -7.0], [0.5, -15.0, -18.5], [0.0, 24.0, 30.0]], np.float32)
    c16, dd16 = torch.empty((3, 2), dtype=torch.float16, device=gpu), torch.empty((2, 3), dtype=torch.float16, device=gpu)
    nt.convert_data_type(d1, c16)
    nt.convert_data_type(d2, dd16)
    e16 = torch.empty((3, 3), dtype=torch.float16, device=gpu)
    nt.matrix_mul(c16, nt.X_NOTRANS, dd16, nt.X_NOTRANS, e16)
    f = torch.empty((3, 3), device=gpu)
    nt.convert_data_type(e16, f)
    assert np.array_equal(f.cpu().numpy(), answer)


def test_equal_types_do_nothing_and_bad_pairs_are_refused(gpu):
    torch = torch_()
    L = nt.load()
    a = torch.ones(16, device=gpu)
    b = torch.zeros(16, device=gpu)
    assert L.ntsamd_convert_data_type(0, None, a.data_ptr(), 2, b.data_ptr(), 2, 16) == 0
    torch.cuda.synchronize()
    assert not b.cpu().numpy().any()                                  # ConvertDataType.cu:81-82: returns at once
    assert L.ntsamd_convert_data_type(0, None, a.data_ptr(), 0, b.data_ptr(), 3, 16) == 2
    assert L.ntsamd_last_error().decode() == "Unsupported data types for conversion!"
    assert L.ntsamd_convert_data_type(0, None, a.data_ptr(), 4, b.data_ptr(), 2, 16) == 2
    assert L.ntsamd_convert_data_type(0, None, a.data_ptr(), 2, b.data_ptr(), 3, -1) == 1
    assert L.ntsamd_convert_data_type(0, None, None, 2, b.data_ptr(), 3, 4) == 1
    assert L.ntsamd_convert_data_type(0, None, a.data_ptr(), 2, b.data_ptr(), 3, 0) == 0


@pytest.mark.parametrize("ta", (nt.X_NOTRANS, nt.X_TRANS))
@pytest.mark.parametrize("tb", (nt.X_NOTRANS, nt.X_TRANS))
def test_float_a_is_rounded_to_half_inside_the_product(gpu, oracle, ta, tb):
    """A half product whose a is stored as float (the probabilities after the softmax,
    source/sample/transformer/submodel/Attention.cpp:231-237: ConvertDataType, then BMMul with the half values):
    the result is that of oracle_convert_data_type followed by the half product, and the same bits as the
    library's own conversion pass followed by its product on the same kernel."""
    torch = torch_()
    from tolerance import assert_fp16
    for i, (M, N, K) in enumerate(((128, 64, 128), (100, 72, 50), (257, 129, 333), (40, 30011, 96))):
        sa = (K, M) if ta == nt.X_TRANS else (M, K)
        sb = (N, K) if tb == nt.X_TRANS else (K, N)
        a = ((oracle.uniform(sa, 8100 + i) + 0.5) / 3.0).astype(np.float32)       # values that do not fit a half exactly
        b = oracle.from_f16_bits(oracle.to_f16_bits(oracle.normal(sb, 8200 + i, 0, 0.5)))
        a_half = oracle.from_f16_bits(oracle.convert(a, X_FLOAT16))    # what the reference multiplies
        ga, gb = to_dev(a, gpu), to_dev(b, gpu).half()
        for out_float in (False, True):
            ref = oracle.matmul2d(a_half, ta, b, tb, None, 0.5, 0.0)
            c = torch.full((M, N), float("nan"), device=gpu, dtype=torch.float32 if out_float else torch.float16)
            nt.matrix_mul(ga, ta, gb, tb, c, 0.5, 0.0)
            assert_fp16(c.float().cpu().numpy(), ref, what="%dx%dx%d float a, %s result" % (M, N, K, "float" if out_float else "half"))
            # the library's two steps: a conversion pass, then the product through the same register-staged kernel
            nt.tuning_set("NTSAMD_F16_FETCH", 2)
            try:
                ah = torch.empty(sa, device=gpu, dtype=torch.float16)
                nt.convert_data_type(ga, ah)
                c2 = torch.full_like(c, float("nan"))
                nt.matrix_mul(ah, ta, gb, tb, c2, 0.5, 0.0)
            finally:
                nt.tuning_set("NTSAMD_F16_FETCH", None)
            assert torch.equal(c, c2), "%dx%dx%d: fused rounding and conversion pass differ" % (M, N, K)


def test_float_probabilities_times_half_values_in_batches(gpu, oracle):
    """The attention context of the half training path: probabilities (float, after softmax and dropout) times the
    heads' values (half), as a strided batch; and the same on merged tensors through the grid entry point."""
    torch = torch_()
    from tolerance import assert_fp16
    batch, lq, lk, dh = 6, 40, 50, 64
    p = np.abs(oracle.normal((batch, lq, lk), 8300, 0, 1.0)).astype(np.float32)
    p /= p.sum(axis=-1, keepdims=True)
    v = oracle.from_f16_bits(oracle.to_f16_bits(oracle.normal((batch, lk, dh), 8301, 0, 0.5)))
    p_half = oracle.from_f16_bits(oracle.convert(p, X_FLOAT16))
    ref = oracle.matmul_batched(p_half, nt.X_NOTRANS, v, nt.X_NOTRANS, None, 1.0)
    gp, gv = to_dev(p, gpu), to_dev(v, gpu).half()
    c = torch.full((batch, lq, dh), float("nan"), device=gpu, dtype=torch.float16)
    nt.matrix_mul_batched_strided(gp, nt.X_NOTRANS, gv, nt.X_NOTRANS, c, batch, lq * lk, lk * dh, lq * dh, lq, lk, lk, dh, lq, dh, 1.0, 0.0)
    assert_fp16(c.float().cpu().numpy(), ref, what="float probabilities x half values, strided batch")


def test_long_products_round_a_in_a_pass_of_their_own_with_the_same_bits(gpu, oracle):
    """Where the library rounds a float a in a pass of its own before a long product (into its workspace), the
    result is the one its conversion entry point followed by the all-half product gives, bit for bit; forced on
    small shapes and on a batch whose matrices stand apart, and left to the library's own choice at
    2048 x 2048 x 1024."""
    torch = torch_()
    from tolerance import assert_fp16
    T, NT = nt.X_TRANS, nt.X_NOTRANS
    for i, (M, N, K, ta, forced) in enumerate(((128, 64, 128, NT, 1), (100, 72, 56, T, 1), (257, 136, 328, NT, 1),
                                               (2048, 2048, 1024, NT, None), (2048, 2048, 1024, T, None))):
        sa = (K, M) if ta == T else (M, K)
        a = ((oracle.uniform(sa, 8400 + i) + 0.5) / 3.0).astype(np.float32)
        b = oracle.from_f16_bits(oracle.to_f16_bits(oracle.normal((K, N), 8500 + i, 0, 0.5)))
        ga, gb = to_dev(a, gpu), to_dev(b, gpu).half()
        ah = torch.empty(sa, device=gpu, dtype=torch.float16)
        nt.convert_data_type(ga, ah)
        for out_float in (False, True):
            c = torch.full((M, N), float("nan"), device=gpu, dtype=torch.float32 if out_float else torch.float16)
            c2 = torch.full_like(c, float("nan"))
            nt.tuning_set("NTSAMD_A32_CONVERT", forced)
            try:
                nt.matrix_mul(ga, ta, gb, NT, c, 0.5, 0.0)
            finally:
                nt.tuning_set("NTSAMD_A32_CONVERT", None)
            nt.matrix_mul(ah, ta, gb, NT, c2, 0.5, 0.0)
            assert torch.equal(c, c2), "%dx%dx%d: a rounded before the product differs from convert + product" % (M, N, K)
            if M <= 300:
                a_half = oracle.from_f16_bits(oracle.convert(a, X_FLOAT16))
                assert_fp16(c.float().cpu().numpy(), oracle.matmul2d(a_half, ta, b, NT, None, 0.5, 0.0),
                            what="%dx%dx%d float a rounded first" % (M, N, K))
    # a strided batch whose probabilities stand 24 floats apart: the pass covers the gaps too, the product skips them
    batch, lq, lk, dh, gap = 5, 40, 48, 64, 24
    p = np.abs(oracle.normal((batch, lq * lk + gap), 8600, 0, 1.0)).astype(np.float32)
    v = oracle.from_f16_bits(oracle.to_f16_bits(oracle.normal((batch, lk, dh), 8601, 0, 0.5)))
    p_half = oracle.from_f16_bits(oracle.convert(np.ascontiguousarray(p[:, :lq * lk]).reshape(batch, lq, lk), X_FLOAT16))
    ref = oracle.matmul_batched(p_half, NT, v, NT, None, 1.0)
    gp, gv = to_dev(p, gpu), to_dev(v, gpu).half()
    c = torch.full((batch, lq, dh), float("nan"), device=gpu, dtype=torch.float16)
    nt.tuning_set("NTSAMD_A32_CONVERT", 1)
    try:
        nt.matrix_mul_batched_strided(gp, NT, gv, NT, c, batch, lq * lk + gap, lk * dh, lq * dh, lq, lk, lk, dh, lq, dh, 1.0, 0.0)
    finally:
        nt.tuning_set("NTSAMD_A32_CONVERT", None)
    assert_fp16(c.float().cpu().numpy(), ref, what="float probabilities rounded first, strided batch with gaps")


def test_mixed_types_that_are_not_offered_are_refused(gpu):
    torch = torch_()
    a = torch.zeros((8, 8), device=gpu, dtype=torch.float16)
    b = torch.zeros((8, 8), device=gpu, dtype=torch.float32)
    c = torch.zeros((8, 8), device=gpu, dtype=torch.float16)
    with pytest.raises(nt.NtsAmdError):
        nt.matrix_mul(a, nt.X_NOTRANS, b, nt.X_NOTRANS, c)          # half a, float b
    with pytest.raises(nt.NtsAmdError):
        nt.matrix_mul(b, nt.X_NOTRANS, b, nt.X_NOTRANS, c)          # float operands, half result
