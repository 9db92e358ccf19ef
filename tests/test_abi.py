"""The C-ABI boundary without a GPU: the library loads, exports what include/ntsamd_gemm.h
declares, and rejects bad calls with the reference's messages before touching a device.
Also the fatal-error behaviour of the nts:: host layer (message to stderr, then abort)."""
import ctypes as C
import os
import re
import signal
import subprocess

import pytest

import niutensor_amd as nt

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HEADER = os.path.join(ROOT, "include", "ntsamd_gemm.h")
NTS_TESTS = os.path.join(ROOT, "tests", "cpp", "build", "nts_tests")


def declared_functions():
    text = open(HEADER).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(ntsamd_\w+)\s*\(", text)))


def test_library_exports_every_declared_symbol():
    names = declared_functions()
    assert len(names) == 17
    assert sorted(nt.EXPORTS) == names
    lib = C.CDLL(nt.LIB_PATH)
    for name in names:
        assert hasattr(lib, name), name


def test_measurement_knobs_are_set_by_name_and_not_declared_in_the_header():
    """The knobs for measurements and tests are exported but no part of the documented interface; they are read
    from the environment once and changed by name afterwards (no getenv on the way to a launch)."""
    assert "ntsamd_tuning_set" not in declared_functions()
    nt.tuning_set("NTSAMD_SPLIT_K", 4)
    nt.tuning_set("SPLIT_K", None)
    with pytest.raises(nt.NtsAmdError, match="no knob named"):
        nt.tuning_set("NTSAMD_NO_SUCH_KNOB", 1)
    src = open(os.path.join(ROOT, "niutensor_amd", "csrc", "ntsamd_capi.hip")).read()
    assert src.count("getenv(") == 1          # the one inside the call_once
    for name in os.listdir(os.path.join(ROOT, "niutensor_amd", "csrc")):
        if name.endswith((".h", ".hip")) and name != "ntsamd_capi.hip":
            assert "getenv" not in open(os.path.join(ROOT, "niutensor_amd", "csrc", name)).read(), name


def test_no_vendor_blas_is_linked():
    out = subprocess.run(["ldd", nt.LIB_PATH], capture_output=True, text=True).stdout
    for banned in ("rocblas", "hipblas", "cublas", "MIOpen", "torch"):
        assert banned not in out, out
    out = subprocess.run(["ldd", nt.HOST_LIB_PATH], capture_output=True, text=True).stdout
    for banned in ("rocblas", "hipblas", "cublas", "nts_oracle", "torch"):
        assert banned not in out, out


def test_version_and_empty_error():
    L = nt.load()
    assert L.ntsamd_version().decode() == "0.1"


# Every call below must be rejected (or found empty) BEFORE a device is involved: the
# pointers are made up, so none of these argument lists may describe a runnable product.
def call_mm(L, ta=nt.X_NOTRANS, tb=nt.X_NOTRANS, types=(2, 2, 2), dims=(2, 3, 3, 2, 2, 2), ptr=0x1000):
    return L.ntsamd_matrix_mul(0, None, ptr, ta, types[0], ptr, tb, types[1], ptr, types[2], *dims, 1.0, 0.0)


def test_argument_errors_need_no_device():
    L = nt.load()
    # unsupported data types: X_INT, X_DOUBLE, mixed
    for types in ((0, 0, 0), (4, 4, 4), (3, 2, 2), (3, 2, 3), (2, 2, 3)):
        assert call_mm(L, types=types) == 2
        assert L.ntsamd_last_error().decode() == "Unsupported data type!"
    # transpose flags are the enum values 0 / 1, nothing else
    assert call_mm(L, ta=2) == 1
    assert "X_TRANS (0) or X_NOTRANS (1)" in L.ntsamd_last_error().decode()
    # shapes that do not multiply, in each transpose layout
    assert call_mm(L, dims=(2, 3, 2, 3, 2, 3)) == 1
    assert L.ntsamd_last_error().decode() == "Unmatched matrices in multiplication!"
    assert call_mm(L, ta=nt.X_TRANS, dims=(2, 3, 3, 2, 2, 2)) == 1
    assert call_mm(L, dims=(2, 3, 3, 2, 2, 3)) == 1
    assert call_mm(L, dims=(-2, 3, 3, 2, 2, 2)) == 1
    # the entry point that allocates nothing checks its arguments the same way, and its number of pieces
    args = (0, None, 0x1000, 1, 2, 0x1000, 1, 2, 0x1000, 2)
    assert L.ntsamd_matrix_mul_static(*args, 2, 3, 3, 2, 2, 2, 1.0, 0.0, -1) == 1
    assert L.ntsamd_matrix_mul_static(*args, 2, 3, 2, 3, 2, 3, 1.0, 0.0, 0) == 1
    assert L.ntsamd_matrix_mul_static(*args, 0, 3, 3, 2, 0, 2, 1.0, 0.0, 0) == 0       # no rows: nothing to do
    assert L.ntsamd_release_workspaces(1000) == 3
    assert L.ntsamd_release_workspaces(-1) == 0                                        # none allocated: nothing to do
    # null pointers
    assert call_mm(L, ptr=None) == 1
    assert L.ntsamd_last_error().decode() == "Empty matrices in multiplication!"
    # batch errors
    rc = L.ntsamd_matrix_mul_batched_strided(0, None, 0x1000, 1, 2, 6, 0x1000, 1, 2, 6, 0x1000, 2, 1,
                                             3, 2, 3, 3, 2, 2, 2, 1.0, 0.0)
    assert rc == 1 and "overlap" in L.ntsamd_last_error().decode()
    rc = L.ntsamd_matrix_mul_batched_strided(0, None, 0x1000, 1, 2, 6, 0x1000, 1, 2, 6, 0x1000, 2, 4,
                                             -1, 2, 3, 3, 2, 2, 2, 1.0, 0.0)
    assert rc == 1
    # bias errors
    rc = L.ntsamd_matrix_mul_bias(0, None, 0x1000, 1, 2, 0x1000, 1, 2, 0x1000, 2, 2, 3, 3, 2, 2, 2, 1.0, 0.0,
                                  0x1000, nt.BIAS_COL, 3, 1)
    assert rc == 1 and L.ntsamd_last_error().decode() == "Wrong tensor size!"
    rc = L.ntsamd_matrix_mul_bias(0, None, 0x1000, 1, 2, 0x1000, 1, 2, 0x1000, 2, 2, 3, 3, 2, 2, 2, 1.0, 0.0,
                                  None, nt.BIAS_COL, 2, 1)
    assert rc == 1


def test_column_sum_and_reduction_argument_errors_need_no_device():
    L = nt.load()
    cs = L.ntsamd_matrix_mul_colsum
    # missing column-sum buffer; half inputs with a float result; shapes that do not multiply
    assert cs(0, None, 0x1000, 1, 2, 0x1000, 1, 2, 0x1000, 2, 2, 3, 3, 2, 2, 2, 1.0, 0.0, None, 0.0) == 1
    assert "column sums" in L.ntsamd_last_error().decode()
    assert cs(0, None, 0x1000, 1, 3, 0x1000, 1, 3, 0x1000, 2, 2, 3, 3, 2, 2, 2, 1.0, 0.0, 0x1000, 0.0) == 2
    assert cs(0, None, 0x1000, 1, 2, 0x1000, 1, 2, 0x1000, 2, 2, 3, 2, 3, 2, 3, 1.0, 0.0, 0x1000, 0.0) == 1
    assert cs(0, None, None, 1, 2, 0x1000, 1, 2, 0x1000, 2, 2, 3, 3, 2, 2, 2, 1.0, 0.0, 0x1000, 0.0) == 1
    # no columns: nothing to do
    assert cs(0, None, 0x1000, 1, 2, 0x1000, 1, 2, 0x1000, 2, 2, 3, 3, 0, 2, 0, 1.0, 0.0, 0x1000, 0.0) == 0
    rs = L.ntsamd_reduce_sum_xz
    assert rs(0, None, 0x1000, 4, 2, 3, 1, 0x1000, 0.0) == 2              # X_DOUBLE
    assert L.ntsamd_last_error().decode() == "Unsupported data type!"
    assert rs(0, None, 0x1000, 2, -2, 3, 1, 0x1000, 0.0) == 1
    assert rs(0, None, None, 2, 2, 3, 1, 0x1000, 0.0) == 1
    assert rs(0, None, 0x1000, 2, 2, 3, 1, None, 0.0) == 1
    assert rs(0, None, 0x1000, 2, 70000, 70000, 1, 0x1000, 0.0) == 1
    assert rs(0, None, 0x1000, 2, 5, 0, 1, 0x1000, 0.0) == 0              # no output elements


def test_empty_products_succeed_without_a_device():
    L = nt.load()
    # zero rows, zero columns, zero batch items: nothing to do, no device needed
    assert call_mm(L, dims=(0, 3, 3, 2, 0, 2)) == 0
    assert call_mm(L, dims=(2, 3, 3, 0, 2, 0)) == 0
    rc = L.ntsamd_matrix_mul_batched_strided(0, None, 0x1000, 1, 2, 6, 0x1000, 1, 2, 6, 0x1000, 2, 4,
                                             0, 2, 3, 3, 2, 2, 2, 1.0, 0.0)
    assert rc == 0


def test_convert_and_attention_argument_errors_need_no_device():
    L = nt.load()
    p = 0x1000
    assert L.ntsamd_convert_data_type(0, None, p, 2, p, 4, 8) == 2
    assert L.ntsamd_last_error().decode() == "Unsupported data types for conversion!"
    assert L.ntsamd_convert_data_type(0, None, p, 3, p, 0, 8) == 2                # half -> int: refused like the reference
    assert L.ntsamd_convert_data_type(0, None, p, 2, p, 2, 8) == 0                # equal types: nothing to do
    assert L.ntsamd_convert_data_type(0, None, p, 2, p, 3, -5) == 1
    assert L.ntsamd_convert_data_type(0, None, None, 2, p, 3, 5) == 1
    assert L.ntsamd_convert_data_type(0, None, p + 2, 2, p, 3, 5) == 1            # a float array on an odd half
    st = (C.c_longlong * 12)(*([8, 64, 8] * 4))
    assert L.ntsamd_attention(0, None, p, p, p, None, p, 4, 1, 1, 8, 8, 8, st, 1.0) == 2
    assert L.ntsamd_last_error().decode() == "Unsupported data type!"
    assert L.ntsamd_attention(0, None, p, p, p, None, p, 2, 1, 1, 8, 8, 132, st, 1.0) == 1
    assert L.ntsamd_attention(0, None, p, p, p, None, p, 2, 1, 1, 8, 0, 8, st, 1.0) == 1
    assert "no keys" in L.ntsamd_last_error().decode()
    assert L.ntsamd_attention(0, None, p, p, p, None, p, 2, -1, 1, 8, 8, 8, st, 1.0) == 1
    assert L.ntsamd_attention(0, None, p, p, p, None, p, 2, 0, 1, 8, 8, 8, st, 1.0) == 0            # no heads: nothing to do
    assert L.ntsamd_attention(0, None, p + 4, p, p, None, p, 2, 1, 1, 8, 8, 8, st, 1.0) == 1        # q not 16-byte aligned
    assert L.ntsamd_attention(0, None, p, p, p, None, p, 2, 1, 1, 8, 8, 8, None, 1.0) == 1
    big = (C.c_longlong * 12)(*([8, 64, 8, 8, 64, 1 << 24, 8, 64, 8, 8, 64, 8]))
    assert L.ntsamd_attention(0, None, p, p, p, None, p, 2, 1, 1, 8, 1000, 8, big, 1.0) == 1
    assert "2 GiB" in L.ntsamd_last_error().decode()
    # an unknown activation
    assert L.ntsamd_matrix_mul_bias_act(0, None, p, 1, 2, p, 1, 2, p, 2, 8, 8, 8, 8, 8, 8, 1.0, 0.0, p, 1, 8, 1, 7) == 1


def test_grid_batch_argument_errors_need_no_device():
    L = nt.load()
    p = 0x1000
    g = L.ntsamd_matrix_mul_batched_grid

    def call(lda=8, sa=(64, 0), ldb=8, sb=(64, 0), ldc=8, sc=(64, 128), counts=(2, 2), types=(2, 2, 2), a=p):
        return g(0, None, a, 1, types[0], lda, sa[0], sa[1], p, 1, types[1], ldb, sb[0], sb[1],
                 p, types[2], ldc, sc[0], sc[1], counts[0], counts[1], 8, 8, 8, 8, 8, 8, 1.0, 0.0)

    assert call(lda=7) == 1 and "leading dimension" in L.ntsamd_last_error().decode()
    assert call(ldc=4) == 1
    assert call(sa=(-1, 0)) == 1 and "negative" in L.ntsamd_last_error().decode()
    assert call(counts=(-2, 2)) == 1
    assert call(counts=(1 << 16, 1 << 16)) == 1 and "too many" in L.ntsamd_last_error().decode()
    assert call(counts=(0, 2)) == 0                                       # nothing to do
    assert call(a=None) == 1
    assert call(types=(3, 2, 2)) == 2                                     # half times float
    # results: two items in the same place; heads side by side but rows too short for both; heads side by
    # side with the next batch item starting inside the last row
    assert call(sc=(0, 128)) == 1 and "overlap" in L.ntsamd_last_error().decode()
    assert call(ldc=12, sc=(8, 128)) == 1
    assert call(ldc=16, sc=(8, 7 * 16 + 8)) == 1


def test_invalid_device_is_an_error():
    L = nt.load()
    rc = L.ntsamd_init(12345)
    assert rc == 3 and "device" in L.ntsamd_last_error().decode()
    rc = L.ntsamd_init(-1)
    assert rc == 3


@pytest.mark.parametrize("case,message", [
    ("unmatched", "Unmatched tensors in multiplication!"),
    ("datatype", "Input tensors should have the same data type!"),
    ("order", "Input tensor and output tensor must have same order!"),
    ("wrongorder", "wrong tensor order"),
    ("empty", "Empty input tensors!"),
    ("host", "does not replace"),
    ("biasshape", "TODO!"),
    ("nograd", "No gradient found!"),
    ("gradtodo", "TODO!"),
    ("converthost", "does not replace"),
    ("convertsize", "Unmatched tensors!"),
    ("attentionheads", "The hidden size must be a multiple of the number of heads!"),
    ("attentiontype", "Input tensors should have the same data type!"),
])
def test_nts_layer_fatal_errors(case, message):
    """CheckNTErrors / ShowNTErrors of the reference: '[ERROR] ...' on stderr, then std::terminate."""
    assert os.path.exists(NTS_TESTS), "build tests/cpp first (__graft_entry__.build())"
    p = subprocess.run([NTS_TESTS, "--abort", case], capture_output=True, text=True, timeout=60)
    assert p.returncode == -signal.SIGABRT, (p.returncode, p.stderr)
    assert p.stderr.startswith("[ERROR]"), p.stderr
    assert message in p.stderr
