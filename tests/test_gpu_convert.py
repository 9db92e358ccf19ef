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
