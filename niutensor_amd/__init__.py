"""MI355X (gfx950) matrix multiplication for NiuTensor: Python plumbing.

The product is the C-ABI library `lib/libntsamd.so` (hand-written HIP kernels,
declared in `include/ntsamd_gemm.h`) and the C++ `nts::` host layer in `nts/`.
This module only loads the library through ctypes so that tests and the
benchmark can call the C ABI on buffers that PyTorch owns. There is no CPU
fallback: if the library is missing, or there is no gfx950 device, calls fail.
"""
import ctypes as C
import os
import subprocess

HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(HERE, "lib", "libntsamd.so")
HOST_LIB_PATH = os.path.join(HERE, "lib", "libnts_amd.so")

X_TRANS, X_NOTRANS = 0, 1           # MATRIX_TRANS_TYPE, source/tensor/XDataType.h:36
X_INT, X_FLOAT, X_FLOAT16 = 0, 2, 3  # TENSOR_DATA_TYPE, source/tensor/XDataType.h:33
BIAS_NONE, BIAS_COL, BIAS_ROW = 0, 1, 2
ACT_NONE, ACT_RECTIFY = 0, 1

EXPORTS = (
    "ntsamd_last_error",
    "ntsamd_version",
    "ntsamd_init",
    "ntsamd_matrix_mul",
    "ntsamd_matrix_mul_bias",
    "ntsamd_matrix_mul_bias_act",
    "ntsamd_matrix_mul_batched_strided",
    "ntsamd_matrix_mul_batched",
    "ntsamd_matrix_mul_batched_grid",
    "ntsamd_matrix_mul_colsum",
    "ntsamd_reduce_sum_xz",
    "ntsamd_attention",
    "ntsamd_attention_probs",
    "ntsamd_attention_train",
    "ntsamd_convert_data_type",
    "ntsamd_release_workspaces",
    "ntsamd_matrix_mul_static",
)


class NtsAmdError(RuntimeError):
    pass


def build(jobs=8):
    """Compile every HIP source for gfx950 (hipcc cross-compiles without a GPU)."""
    subprocess.run(["make", "-s", "-C", os.path.join(HERE, "csrc"), "-j%d" % jobs], check=True)
    subprocess.run(["make", "-s", "-C", os.path.join(HERE, "nts"), "-j%d" % jobs], check=True)


_lib = None


def load():
    """Load libntsamd.so; raises if it has not been built."""
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(LIB_PATH):
        raise NtsAmdError("%s is missing: run niutensor_amd.build() (or make -C niutensor_amd/csrc)" % LIB_PATH)
    L = C.CDLL(LIB_PATH)
    vp, ci, cf, ll = C.c_void_p, C.c_int, C.c_float, C.c_longlong
    L.ntsamd_last_error.restype = C.c_char_p
    L.ntsamd_version.restype = C.c_char_p
    L.ntsamd_init.argtypes = [ci]
    L.ntsamd_matrix_mul.argtypes = [ci, vp, vp, ci, ci, vp, ci, ci, vp, ci] + [ci] * 6 + [cf, cf]
    L.ntsamd_matrix_mul_bias.argtypes = [ci, vp, vp, ci, ci, vp, ci, ci, vp, ci] + [ci] * 6 + [cf, cf, vp, ci, ci, ci]
    L.ntsamd_matrix_mul_bias_act.argtypes = L.ntsamd_matrix_mul_bias.argtypes + [ci]
    L.ntsamd_matrix_mul_batched_strided.argtypes = [ci, vp, vp, ci, ci, ll, vp, ci, ci, ll, vp, ci, ll,
                                                    ci] + [ci] * 6 + [cf, cf]
    L.ntsamd_matrix_mul_batched_grid.argtypes = [ci, vp, vp, ci, ci, ci, ll, ll, vp, ci, ci, ci, ll, ll,
                                                 vp, ci, ci, ll, ll, ci, ci] + [ci] * 6 + [cf, cf]
    L.ntsamd_matrix_mul_batched.argtypes = [ci, vp, C.POINTER(vp), ci, ci, C.POINTER(vp), ci, ci, C.POINTER(vp), ci,
                                            ci] + [ci] * 6 + [cf, cf]
    L.ntsamd_matrix_mul_colsum.argtypes = [ci, vp, vp, ci, ci, vp, ci, ci, vp, ci] + [ci] * 6 + [cf, cf, vp, cf]
    L.ntsamd_reduce_sum_xz.argtypes = [ci, vp, vp, ci, ci, ci, ci, vp, cf]
    L.ntsamd_attention.argtypes = [ci, vp, vp, vp, vp, vp, vp, ci, ci, ci, ci, ci, ci, C.POINTER(ll), cf]
    L.ntsamd_attention_probs.argtypes = [ci, vp, vp, vp, vp, vp, ci, ci, ci, ci, ci, ci, C.POINTER(ll), cf]
    L.ntsamd_attention_train.argtypes = [ci, vp, vp, vp, vp, vp, vp, vp, vp, vp, ci, ci, ci, ci, ci, ci, C.POINTER(ll), cf]
    L.ntsamd_convert_data_type.argtypes = [ci, vp, vp, ci, vp, ci, ll]
    L.ntsamd_release_workspaces.argtypes = [ci]
    L.ntsamd_matrix_mul_static.argtypes = L.ntsamd_matrix_mul.argtypes + [ci]
    # measurement knobs: exported, but no part of the interface include/ntsamd_gemm.h documents
    L.ntsamd_tuning_set.argtypes = [C.c_char_p, ci]
    L.ntsamd_tuning_set.restype = ci
    L.ntsamd_last_plan.restype = C.c_char_p
    L.ntsamd_plan_only.argtypes = [ci]
    L.ntsamd_plan_only.restype = None
    for name in EXPORTS[2:]:
        getattr(L, name).restype = ci
    _lib = L
    return L


_plan_log = None


def record_plans(on):
    """Start (True) or stop (False) keeping what every call through this module was planned as; stopping returns
    the list. For the benchmark, which prints the kernels of a configuration beside its timings."""
    global _plan_log
    log, _plan_log = _plan_log, ([] if on else None)
    return log


def _check(rc):
    if rc != 0:
        raise NtsAmdError("ntsamd error %d: %s" % (rc, load().ntsamd_last_error().decode()))
    if _plan_log is not None:
        _plan_log.append(load().ntsamd_last_plan().decode())


def _dtype_code(t):
    import torch
    if t.dtype == torch.float32:
        return X_FLOAT
    if t.dtype == torch.float16:
        return X_FLOAT16
    if t.dtype == torch.int32:
        return X_INT
    raise NtsAmdError("Unsupported data type!")


def _stream_ptr(t):
    import torch
    return torch.cuda.current_stream(t.device).cuda_stream


def _mat(t):
    """Stored rows, columns of the last two dimensions of a dense tensor."""
    assert t.is_contiguous()
    return int(t.shape[-2]), int(t.shape[-1])


def matrix_mul(a, transA, b, transB, c, alpha=1.0, beta=0.0, bias=None, bias_mode=BIAS_COL, bias_row_div=1, act=ACT_NONE):
    """c = f(alpha * op(a) op(b) + beta * c (+ bias)) on 2-D device tensors, through the C ABI;
    f is the identity or, with act=ACT_RECTIFY (needs a bias), max(0, .)."""
    L = load()
    na, ma = _mat(a)
    nb, mb = _mat(b)
    nc, mc = _mat(c)
    dev = a.device.index
    if bias is None:
        rc = L.ntsamd_matrix_mul(dev, _stream_ptr(a), a.data_ptr(), transA, _dtype_code(a),
                                 b.data_ptr(), transB, _dtype_code(b), c.data_ptr(), _dtype_code(c),
                                 na, ma, nb, mb, nc, mc, alpha, beta)
    else:
        rc = L.ntsamd_matrix_mul_bias_act(dev, _stream_ptr(a), a.data_ptr(), transA, _dtype_code(a),
                                          b.data_ptr(), transB, _dtype_code(b), c.data_ptr(), _dtype_code(c),
                                          na, ma, nb, mb, nc, mc, alpha, beta,
                                          bias.data_ptr(), bias_mode, bias.numel(), bias_row_div, act)
    _check(rc)
    return c


def matrix_mul_static(a, transA, b, transB, c, alpha=1.0, beta=0.0, splits=0):
    """matrix_mul through the entry point that allocates nothing (partial products of a cut k in the static scratch)."""
    na, ma = _mat(a)
    nb, mb = _mat(b)
    nc, mc = _mat(c)
    rc = load().ntsamd_matrix_mul_static(a.device.index, _stream_ptr(a), a.data_ptr(), transA, _dtype_code(a),
                                         b.data_ptr(), transB, _dtype_code(b), c.data_ptr(), _dtype_code(c),
                                         na, ma, nb, mb, nc, mc, alpha, beta, splits)
    _check(rc)
    return c


def release_workspaces(device=-1):
    """Free the workspaces of products cut along k (every device if device < 0)."""
    _check(load().ntsamd_release_workspaces(device))


def tuning_set(name, value):
    """Set a measurement knob ("NTSAMD_TILE_CFG", "NTSAMD_SPLIT_K", ...) in the running library; None or a negative
    value hands the decision back to the library. For tests and measurements only."""
    v = -1 if value is None else int(value)
    _check(load().ntsamd_tuning_set(name.encode(), v))


def last_plan():
    """What the last product or attention call of this thread was planned as: kernel family, tile shape, layout,
    fetch route, pieces of k, the passes around it. For measurements and tests."""
    return load().ntsamd_last_plan().decode()


def plan_only(on):
    """While on, calls from this thread stop after planning: no device is looked up, nothing is allocated or
    launched, no pointer is followed; last_plan() then tells what would have run. For tests of the dispatcher."""
    load().ntsamd_plan_only(1 if on else 0)


def matrix_mul_batched_strided(a, transA, b, transB, c, count, strideA, strideB, strideC,
                               na, ma, nb, mb, nc, mc, alpha=1.0, beta=0.0):
    L = load()
    rc = L.ntsamd_matrix_mul_batched_strided(a.device.index, _stream_ptr(a),
                                             a.data_ptr(), transA, _dtype_code(a), strideA,
                                             b.data_ptr(), transB, _dtype_code(b), strideB,
                                             c.data_ptr(), _dtype_code(c), strideC,
                                             count, na, ma, nb, mb, nc, mc, alpha, beta)
    _check(rc)
    return c


def matrix_mul_batched_grid(a, transA, lda, stridesA, b, transB, ldb, stridesB, c, ldc, stridesC,
                            count0, count1, na, ma, nb, mb, nc, mc, alpha=1.0, beta=0.0):
    """count0 x count1 products whose matrices stand inside larger tensors: item (i0, i1) of an operand starts
    at i0 * strides[0] + i1 * strides[1] elements and has rows ld elements apart."""
    L = load()
    rc = L.ntsamd_matrix_mul_batched_grid(a.device.index, _stream_ptr(a),
                                          a.data_ptr(), transA, _dtype_code(a), lda, stridesA[0], stridesA[1],
                                          b.data_ptr(), transB, _dtype_code(b), ldb, stridesB[0], stridesB[1],
                                          c.data_ptr(), _dtype_code(c), ldc, stridesC[0], stridesC[1],
                                          count0, count1, na, ma, nb, mb, nc, mc, alpha, beta)
    _check(rc)
    return c


def matrix_mul_batched(a_list, transA, b_list, transB, c_list, alpha=1.0, beta=0.0):
    """Pointer-list batch over same-shaped 2-D device tensors."""
    L = load()
    n = len(a_list)
    arr = C.c_void_p * n
    pa = arr(*[t.data_ptr() for t in a_list])
    pb = arr(*[t.data_ptr() for t in b_list])
    pc = arr(*[t.data_ptr() for t in c_list])
    a, b, c = a_list[0], b_list[0], c_list[0]
    na, ma = _mat(a)
    nb, mb = _mat(b)
    nc, mc = _mat(c)
    rc = L.ntsamd_matrix_mul_batched(a.device.index, _stream_ptr(a), pa, transA, _dtype_code(a),
                                     pb, transB, _dtype_code(b), pc, _dtype_code(c),
                                     n, na, ma, nb, mb, nc, mc, alpha, beta)
    _check(rc)
    return c_list


def matrix_mul_colsum(a, transA, b, transB, c, col_sum, alpha=1.0, beta=0.0, col_sum_beta=0.0):
    """c = alpha * op(a) op(b) + beta * c and col_sum = col_sum_beta * col_sum + column sums of op(b)."""
    L = load()
    na, ma = _mat(a)
    nb, mb = _mat(b)
    nc, mc = _mat(c)
    rc = L.ntsamd_matrix_mul_colsum(a.device.index, _stream_ptr(a), a.data_ptr(), transA, _dtype_code(a),
                                    b.data_ptr(), transB, _dtype_code(b), c.data_ptr(), _dtype_code(c),
                                    na, ma, nb, mb, nc, mc, alpha, beta, col_sum.data_ptr(), col_sum_beta)
    _check(rc)
    return c, col_sum


def reduce_sum_xz(t, out, beta=0.0):
    """out[y] = beta * out[y] + sum over x and z of a dense [x][y][z] device tensor."""
    L = load()
    assert t.is_contiguous() and t.dim() == 3
    x, y, z = (int(v) for v in t.shape)
    rc = L.ntsamd_reduce_sum_xz(t.device.index, _stream_ptr(t), t.data_ptr(), _dtype_code(t), x, y, z,
                                out.data_ptr(), beta)
    _check(rc)
    return out


def attention(q, k, v, out, heads, scale, mask=None, split=False):
    """out = softmax(scale q k^T + mask) v per head. q, k, v, out are [batch][rows][heads*dh] device
    tensors (split=False: the layout before Split / after Merge) or [heads][batch][rows][dh] (split=True);
    mask is None or a dense float [heads][batch][lq][lk] tensor."""
    L = load()
    if split:
        _, batch, lq, dh = (int(x) for x in q.shape)
        lk = int(k.shape[2])
        st = lambda rows: (batch * rows * dh, rows * dh, dh)
    else:
        batch, lq, hd = (int(x) for x in q.shape)
        lk = int(k.shape[1])
        dh = hd // heads
        st = lambda rows: (dh, rows * hd, hd)
    for t in (q, k, v, out):
        assert t.is_contiguous()
    strides = (C.c_longlong * 12)(*(st(lq) + st(lk) + st(lk) + st(lq)))
    rc = L.ntsamd_attention(q.device.index, _stream_ptr(q), q.data_ptr(), k.data_ptr(), v.data_ptr(),
                            mask.data_ptr() if mask is not None else None, out.data_ptr(), _dtype_code(q),
                            heads, batch, lq, lk, dh, strides, scale)
    _check(rc)
    return out


def attention_probs(q, k, probs, heads, scale, mask=None):
    """probs[h][b] = softmax(scale q_h k_h^T + mask[h][b]); q [batch][lq][heads*dh], k [batch][lk][heads*dh],
    probs and mask dense float [heads][batch][lq][lk]."""
    batch, lq, hd = (int(x) for x in q.shape)
    lk = int(k.shape[1])
    dh = hd // heads
    for t in (q, k, probs):
        assert t.is_contiguous()
    strides = (C.c_longlong * 6)(dh, lq * hd, hd, dh, lk * hd, hd)
    rc = load().ntsamd_attention_probs(q.device.index, _stream_ptr(q), q.data_ptr(), k.data_ptr(),
                                       mask.data_ptr() if mask is not None else None, probs.data_ptr(), _dtype_code(q),
                                       heads, batch, lq, lk, dh, strides, scale)
    _check(rc)
    return probs


def attention_train(q, k, v, probs, out, heads, scale, mask=None, drop_mask=None, dropped=None):
    """The training path in one launch: probs = softmax(scale q k^T + mask) ([heads][batch][lq][lk]),
    dropped = probs * drop_mask (written if given), out = (dropped or probs) v in the merged layout of q."""
    batch, lq, hd = (int(x) for x in q.shape)
    lk = int(k.shape[1])
    dh = hd // heads
    for t in (q, k, v, probs, out):
        assert t.is_contiguous()
    st = lambda rows: (dh, rows * hd, hd)
    strides = (C.c_longlong * 12)(*(st(lq) + st(lk) + st(lk) + st(lq)))
    ptr = lambda t: t.data_ptr() if t is not None else None
    rc = load().ntsamd_attention_train(q.device.index, _stream_ptr(q), q.data_ptr(), k.data_ptr(), v.data_ptr(), ptr(mask),
                                       ptr(drop_mask), probs.data_ptr(), ptr(dropped), out.data_ptr(), _dtype_code(q),
                                       heads, batch, lq, lk, dh, strides, scale)
    _check(rc)
    return out


def convert_data_type(s, t):
    """t[i] = (type of t) s[i] for dense device tensors of equal size (float32, float16, int32)."""
    assert s.is_contiguous() and t.is_contiguous() and s.numel() == t.numel()
    rc = load().ntsamd_convert_data_type(s.device.index, _stream_ptr(s), s.data_ptr(), _dtype_code(s),
                                         t.data_ptr(), _dtype_code(t), s.numel())
    _check(rc)
    return t
