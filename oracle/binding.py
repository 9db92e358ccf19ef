"""TEST INFRASTRUCTURE: ctypes bindings of the CPU checker.

`Oracle` wraps libnts_oracle.so (the C restatement, nts_oracle.c);
`Reference` wraps _ref/libnts_ref.so (the real NiuTensor CPU sources compiled
by the Makefile beside this file) when that library has been built.
Arrays are numpy, C-contiguous; fp32 unless stated.
"""
import ctypes as C
import os
import subprocess

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))

X_TRANS, X_NOTRANS = 0, 1          # source/tensor/XDataType.h:36
X_FLOAT, X_FLOAT16 = 2, 3          # source/tensor/XDataType.h:33
X_INT = 0
# numpy carriers of the three types: half travels as its bit pattern
NP_TYPE_CODE = {np.float32: X_FLOAT, np.int32: X_INT, np.uint16: X_FLOAT16}
TYPE_CODE_NP = {X_FLOAT: np.float32, X_INT: np.int32, X_FLOAT16: np.uint16}

_fp = C.POINTER(C.c_float)
_ip = C.POINTER(C.c_int)


def _f(a):
    assert a.dtype == np.float32 and a.flags["C_CONTIGUOUS"]
    return a.ctypes.data_as(_fp)


def _dims(shape):
    arr = (C.c_int * max(len(shape), 1))(*shape)
    return arr


def build(native=True):
    """Compile the C restatement (and the reference itself where its tree exists)."""
    subprocess.run(["make", "-s", "-C", HERE, "-j8", "oracle", "ref"], check=True)


def mm_shape(a_shape, transA, b_shape, transB):
    """Result shape of the N-D product, MatrixMul.cpp:279-294."""
    an = a_shape[-1] if transA == X_TRANS else a_shape[-2]
    bm = b_shape[-2] if transB == X_TRANS else b_shape[-1]
    return tuple(a_shape[:-2]) + tuple(b_shape[:-2]) + (an, bm)


def bmm_shape(a_shape, transA, b_shape, transB):
    """Result shape of the same-order batched product, MatrixMulBatched.cpp:305-311."""
    an = a_shape[-1] if transA == X_TRANS else a_shape[-2]
    bm = b_shape[-2] if transB == X_TRANS else b_shape[-1]
    return tuple(a_shape[:-2]) + (an, bm)


class Oracle:
    def __init__(self, native=False):
        name = "libnts_oracle_native.so" if native else "libnts_oracle.so"
        path = os.path.join(HERE, name)
        if not os.path.exists(path):
            build()
        self.lib = L = C.CDLL(path)
        L.oracle_matmul2d.argtypes = [_fp, C.c_int, _fp, C.c_int, _fp] + [C.c_int] * 6 + [C.c_float] * 2
        L.oracle_matmul2d.restype = C.c_int
        L.oracle_matmul_batched.argtypes = [_fp, C.c_int, _ip, _fp, C.c_int, _ip, _fp, _ip, C.c_int,
                                            C.c_float, C.c_float]
        L.oracle_matmul_batched.restype = C.c_int
        L.oracle_matmul.argtypes = [_fp, C.c_int, _ip, C.c_int, _fp, C.c_int, _ip, C.c_int,
                                    _fp, _ip, C.c_int, C.c_float, C.c_float]
        L.oracle_matmul.restype = C.c_int
        L.oracle_broadcast_dim_index.argtypes = [_ip, C.c_int, _ip, C.c_int]
        L.oracle_broadcast_dim_index.restype = C.c_int
        L.oracle_sumdim.argtypes = [_fp, _ip, C.c_int, _fp, C.c_int, _fp, C.c_int, C.c_float]
        L.oracle_sumdim.restype = C.c_int
        L.oracle_mulandshift.argtypes = [_fp, C.c_int, _ip, C.c_int, _fp, C.c_int, _ip, C.c_int,
                                         _fp, _ip, C.c_int, _fp, _ip, _ip, C.c_float]
        L.oracle_mulandshift.restype = C.c_int
        L.oracle_reduce_sum.argtypes = [_fp, _ip, C.c_int, C.c_int, _fp]
        L.oracle_reduce_sum.restype = C.c_int
        L.oracle_grad_matmul.argtypes = [_fp, _fp, C.c_int, _ip, C.c_int, _fp, _fp, C.c_int, _ip, C.c_int, _fp, C.c_float]
        L.oracle_grad_matmul.restype = C.c_int
        L.oracle_grad_matmul_batched.argtypes = [_fp, _fp, C.c_int, _ip, _fp, _fp, C.c_int, _ip, _fp, _ip, C.c_int, C.c_float]
        L.oracle_grad_matmul_batched.restype = C.c_int
        L.oracle_grad_mulandshift.argtypes = [_fp, _fp, C.c_int, _ip, C.c_int, _fp, _fp, C.c_int, _ip, C.c_int,
                                              _fp, C.c_int, _fp, _ip, C.c_int, C.c_int, C.c_float]
        L.oracle_grad_mulandshift.restype = C.c_int
        L.oracle_softmax.argtypes = [_fp, C.c_long, C.c_int, _fp]
        L.oracle_softmax.restype = C.c_int
        L.oracle_attention.argtypes = [_fp, _fp, _fp, _fp, _fp] + [C.c_int] * 5 + [C.c_float]
        L.oracle_attention.restype = C.c_int
        L.oracle_attention_probs.argtypes = [_fp, _fp, _fp, _fp] + [C.c_int] * 5 + [C.c_float]
        L.oracle_attention_probs.restype = C.c_int
        L.oracle_rectify.argtypes = [_fp, C.c_long, _fp]
        L.oracle_convert_data_type.argtypes = [C.c_void_p, C.c_int, C.c_void_p, C.c_int, C.c_long]
        L.oracle_convert_data_type.restype = C.c_int
        L.oracle_is_float_equal.argtypes = [C.c_float] * 4
        L.oracle_is_float_equal.restype = C.c_int
        L.oracle_check_data.argtypes = [_fp, _fp, C.c_int, C.c_float]
        L.oracle_check_data.restype = C.c_int
        L.oracle_f32_to_f16.argtypes = [C.c_float]
        L.oracle_f32_to_f16.restype = C.c_uint16
        L.oracle_f16_to_f32.argtypes = [C.c_uint16]
        L.oracle_f16_to_f32.restype = C.c_float
        L.oracle_f32_to_f16_array.argtypes = [_fp, C.POINTER(C.c_uint16), C.c_long]
        L.oracle_f16_to_f32_array.argtypes = [C.POINTER(C.c_uint16), _fp, C.c_long]
        L.oracle_fill_uniform.argtypes = [_fp, C.c_long, C.c_uint64, C.c_float, C.c_float]
        L.oracle_fill_normal.argtypes = [_fp, C.c_long, C.c_uint64, C.c_float, C.c_float]

    # -- products ---------------------------------------------------------
    def matmul2d(self, a, transA, b, transB, c=None, alpha=1.0, beta=0.0):
        na, ma = a.shape
        nb, mb = b.shape
        nc = ma if transA == X_TRANS else na
        mc = nb if transB == X_TRANS else mb
        if c is None:
            c = np.zeros((nc, mc), np.float32)
        r = self.lib.oracle_matmul2d(_f(a), transA, _f(b), transB, _f(c), na, ma, nb, mb,
                                     c.shape[0], c.shape[1], alpha, beta)
        if r != 0:
            raise ValueError("Unmatched tensors in multiplication!")
        return c

    def matmul(self, a, transA, b, transB, c=None, alpha=1.0, beta=0.0):
        if c is None:
            c = np.zeros(mm_shape(a.shape, transA, b.shape, transB), np.float32)
        r = self.lib.oracle_matmul(_f(a), transA, _dims(a.shape), a.ndim, _f(b), transB, _dims(b.shape), b.ndim,
                                   _f(c), _dims(c.shape), c.ndim, alpha, beta)
        if r != 0:
            raise ValueError("Unmatched tensors in multiplication!")
        return c

    def matmul_batched(self, a, transA, b, transB, c=None, alpha=1.0, beta=0.0):
        if c is None:
            c = np.zeros(bmm_shape(a.shape, transA, b.shape, transB), np.float32)
        if not (a.ndim == b.ndim == c.ndim):
            raise ValueError("Input tensor and output tensor must have same order!")
        r = self.lib.oracle_matmul_batched(_f(a), transA, _dims(a.shape), _f(b), transB, _dims(b.shape),
                                           _f(c), _dims(c.shape), a.ndim, alpha, beta)
        if r != 0:
            raise ValueError("Unmatched tensors in multiplication!")
        return c

    def broadcast_dim_index(self, a_shape, b_shape):
        return self.lib.oracle_broadcast_dim_index(_dims(a_shape), len(a_shape), _dims(b_shape), len(b_shape))

    def sumdim(self, a, b, n, beta=1.0):
        c = np.empty_like(a)
        r = self.lib.oracle_sumdim(_f(a), _dims(a.shape), a.ndim, _f(b), b.size, _f(c), n, beta)
        if r != 0:
            raise ValueError("Wrong tensor size!")
        return c

    def mulandshift(self, x, w, bias, alpha=1.0, transX=X_NOTRANS, transW=X_NOTRANS):
        shape = mm_shape(x.shape, transX, w.shape, transW)
        c = np.zeros(shape, np.float32)
        cd = (C.c_int * 8)()
        co = C.c_int(0)
        n = self.lib.oracle_mulandshift(_f(x), transX, _dims(x.shape), x.ndim, _f(w), transW, _dims(w.shape), w.ndim,
                                        _f(bias), _dims(bias.shape), bias.ndim, _f(c), cd, C.byref(co), alpha)
        if n < 0:
            raise ValueError("the reference aborts on this bias shape")
        assert tuple(cd[i] for i in range(co.value)) == shape
        return c, n

    # -- helpers ----------------------------------------------------------
    # -- backward ---------------------------------------------------------
    def reduce_sum(self, x, dim):
        out = np.zeros(x.shape[:dim] + x.shape[dim + 1:], np.float32)
        if self.lib.oracle_reduce_sum(_f(x), _dims(x.shape), x.ndim, dim, _f(out)) != 0:
            raise ValueError("Illegal dimension to reduce!")
        return out

    @staticmethod
    def _opt(g):
        return _f(g) if g is not None else None

    def grad_matmul(self, a, transA, b, transB, dedc, alpha=1.0, deda=None, dedb=None):
        """deda, dedb: starting values of the gradients (updated in place and returned); None = not wanted."""
        r = self.lib.oracle_grad_matmul(_f(a), self._opt(deda), transA, _dims(a.shape), a.ndim,
                                        _f(b), self._opt(dedb), transB, _dims(b.shape), b.ndim, _f(dedc), alpha)
        if r != 0:
            raise ValueError("TODO!" if r == -2 else "Unmatched tensors in multiplication!")
        return deda, dedb

    def grad_matmul_batched(self, a, transA, b, transB, dedc, alpha=1.0, deda=None, dedb=None):
        r = self.lib.oracle_grad_matmul_batched(_f(a), self._opt(deda), transA, _dims(a.shape),
                                                _f(b), self._opt(dedb), transB, _dims(b.shape),
                                                _f(dedc), _dims(dedc.shape), a.ndim, alpha)
        if r != 0:
            raise ValueError("Unmatched tensors in multiplication!")
        return deda, dedb

    def grad_mulandshift(self, x, w, dedc, n, alpha=1.0, dedx=None, dedw=None, dedbias=None,
                         transX=X_NOTRANS, transW=X_NOTRANS):
        r = self.lib.oracle_grad_mulandshift(_f(x), self._opt(dedx), transX, _dims(x.shape), x.ndim,
                                             _f(w), self._opt(dedw), transW, _dims(w.shape), w.ndim,
                                             self._opt(dedbias), 0 if dedbias is None else dedbias.size,
                                             _f(dedc), _dims(dedc.shape), dedc.ndim, n, alpha)
        if r != 0:
            raise ValueError("TODO!" if r == -2 else "Wrong tensor size!")
        return dedx, dedw, dedbias

    # -- attention ---------------------------------------------------------
    def softmax(self, x):
        y = np.empty_like(x)
        if self.lib.oracle_softmax(_f(x), x.size // x.shape[-1], x.shape[-1], _f(y)) != 0:
            raise ValueError("empty softmax")
        return y

    def attention(self, q, k, v, heads, scale, mask=None):
        """q [batch][lq][hidden], k and v [batch][lk][hidden], mask None or [heads][batch][lq][lk]."""
        batch, lq, hidden = q.shape
        out = np.zeros_like(q)
        r = self.lib.oracle_attention(_f(q), _f(k), _f(v), _f(mask) if mask is not None else None, _f(out),
                                      batch, lq, k.shape[1], hidden, heads, scale)
        if r != 0:
            raise ValueError("Unmatched tensors in attention")
        return out

    def rectify(self, x):
        y = np.empty_like(x)
        self.lib.oracle_rectify(_f(x), x.size, _f(y))
        return y

    # -- data type conversion ------------------------------------------------
    def convert(self, x, type_t):
        """x: float32 (X_FLOAT), int32 (X_INT) or uint16 holding half bit patterns (X_FLOAT16);
        returns the same for type_t."""
        type_s = NP_TYPE_CODE[x.dtype.type]
        x = np.ascontiguousarray(x)
        out = np.empty(x.shape, TYPE_CODE_NP[type_t])
        if type_s == type_t:
            return x.copy()
        if self.lib.oracle_convert_data_type(x.ctypes.data, type_s, out.ctypes.data, type_t, x.size) != 0:
            raise ValueError("Unsupported data types for conversion!")
        return out

    def attention_probs(self, q, k, heads, scale, mask=None):
        """Softmax(scale q_h k_h^T + mask) as [heads][batch][lq][lk]; q [batch][lq][hidden], k [batch][lk][hidden]."""
        batch, lq, hidden = q.shape
        probs = np.zeros((heads, batch, lq, k.shape[1]), np.float32)
        r = self.lib.oracle_attention_probs(_f(q), _f(k), _f(mask) if mask is not None else None, _f(probs),
                                            batch, lq, k.shape[1], hidden, heads, scale)
        if r != 0:
            raise ValueError("Unmatched tensors in attention")
        return probs

    def is_float_equal(self, a, b, abs_err, rel_err=1e-4):
        return bool(self.lib.oracle_is_float_equal(a, b, abs_err, rel_err))

    def check_data(self, value, answer, tol=1e-4):
        v = np.ascontiguousarray(value, np.float32).ravel()
        w = np.ascontiguousarray(answer, np.float32).ravel()
        return v.size == w.size and bool(self.lib.oracle_check_data(_f(v), _f(w), v.size, tol))

    def to_f16_bits(self, x):
        x = np.ascontiguousarray(x, np.float32)
        out = np.empty(x.shape, np.uint16)
        self.lib.oracle_f32_to_f16_array(_f(x), out.ctypes.data_as(C.POINTER(C.c_uint16)), x.size)
        return out

    def from_f16_bits(self, h):
        h = np.ascontiguousarray(h, np.uint16)
        out = np.empty(h.shape, np.float32)
        self.lib.oracle_f16_to_f32_array(h.ctypes.data_as(C.POINTER(C.c_uint16)), _f(out), h.size)
        return out

    def uniform(self, shape, seed, lo=-1.0, hi=1.0):
        x = np.empty(shape, np.float32)
        self.lib.oracle_fill_uniform(_f(x), x.size, seed, lo, hi)
        return x

    def normal(self, shape, seed, mean=0.0, std=1.0):
        x = np.empty(shape, np.float32)
        self.lib.oracle_fill_normal(_f(x), x.size, seed, mean, std)
        return x


class Reference:
    """The real NiuTensor CPU implementation (only where _ref/libnts_ref.so exists)."""

    PATH = os.path.join(HERE, "_ref", "libnts_ref.so")

    @classmethod
    def available(cls):
        return os.path.exists(cls.PATH)

    def __init__(self):
        self.lib = L = C.CDLL(self.PATH)
        L.ref_matmul2d.argtypes = [_fp, C.c_int, _fp, C.c_int, _fp] + [C.c_int] * 6 + [C.c_float] * 2
        L.ref_matmul.argtypes = [_fp, C.c_int, _ip, C.c_int, _fp, C.c_int, _ip, C.c_int,
                                 _fp, _ip, C.c_int, C.c_float, C.c_float]
        L.ref_matmul_batched.argtypes = [_fp, C.c_int, _ip, _fp, C.c_int, _ip, _fp, _ip, C.c_int,
                                         C.c_float, C.c_float]
        L.ref_matmul_alloc.argtypes = [_fp, C.c_int, _ip, C.c_int, _fp, C.c_int, _ip, C.c_int, _fp, _ip, C.c_float]
        L.ref_broadcast_dim_index.argtypes = [_ip, C.c_int, _ip, C.c_int]
        L.ref_sumdim.argtypes = [_fp, _ip, C.c_int, _fp, _ip, C.c_int, _fp, C.c_int, C.c_float]
        L.ref_mulandshift.argtypes = [C.c_int, _fp, C.c_int, _ip, C.c_int, _fp, C.c_int, _ip, C.c_int,
                                      _fp, _ip, C.c_int, _fp, _ip, C.c_float]
        L.ref_enum_values.argtypes = [_ip]
        L.ref_reduce_sum.argtypes = [_fp, _ip, C.c_int, C.c_int, _fp]
        L.ref_attention_probs.argtypes = [_fp, _fp, _fp, _fp] + [C.c_int] * 5 + [C.c_float]
        L.ref_rectify.argtypes = [_fp, C.c_int, _fp]
        L.ref_convert.argtypes = [C.c_void_p, C.c_int, C.c_void_p, C.c_int, C.c_int]
        L.ref_softmax.argtypes = [_fp, _ip, C.c_int, _fp]
        L.ref_attention.argtypes = [_fp, _fp, _fp, _fp, _fp] + [C.c_int] * 5 + [C.c_float]
        L.ref_grad.argtypes = [C.c_int, _fp, _ip, C.c_int, C.c_int, _fp, _ip, C.c_int, C.c_int,
                               _fp, _ip, C.c_int, C.c_float, _fp, _fp, _fp, _fp]

    def matmul2d(self, a, transA, b, transB, c=None, alpha=1.0, beta=0.0):
        na, ma = a.shape
        nb, mb = b.shape
        if c is None:
            c = np.zeros((ma if transA == X_TRANS else na, nb if transB == X_TRANS else mb), np.float32)
        self.lib.ref_matmul2d(_f(a), transA, _f(b), transB, _f(c), na, ma, nb, mb, c.shape[0], c.shape[1], alpha, beta)
        return c

    def matmul(self, a, transA, b, transB, c=None, alpha=1.0, beta=0.0):
        if c is None:
            c = np.zeros(mm_shape(a.shape, transA, b.shape, transB), np.float32)
        self.lib.ref_matmul(_f(a), transA, _dims(a.shape), a.ndim, _f(b), transB, _dims(b.shape), b.ndim,
                            _f(c), _dims(c.shape), c.ndim, alpha, beta)
        return c

    def matmul_alloc(self, a, transA, b, transB, alpha=1.0):
        shape = mm_shape(a.shape, transA, b.shape, transB)
        c = np.zeros(shape, np.float32)
        cd = (C.c_int * 8)()
        order = self.lib.ref_matmul_alloc(_f(a), transA, _dims(a.shape), a.ndim, _f(b), transB, _dims(b.shape), b.ndim,
                                          _f(c), cd, alpha)
        return c, tuple(cd[i] for i in range(order))

    def matmul_batched(self, a, transA, b, transB, c=None, alpha=1.0, beta=0.0):
        if c is None:
            c = np.zeros(bmm_shape(a.shape, transA, b.shape, transB), np.float32)
        self.lib.ref_matmul_batched(_f(a), transA, _dims(a.shape), _f(b), transB, _dims(b.shape),
                                    _f(c), _dims(c.shape), a.ndim, alpha, beta)
        return c

    def broadcast_dim_index(self, a_shape, b_shape):
        return self.lib.ref_broadcast_dim_index(_dims(a_shape), len(a_shape), _dims(b_shape), len(b_shape))

    def sumdim(self, a, b, n, beta=1.0):
        c = np.empty_like(a)
        self.lib.ref_sumdim(_f(a), _dims(a.shape), a.ndim, _f(b), _dims(b.shape), b.ndim, _f(c), n, beta)
        return c

    def mulandshift(self, x, w, bias, alpha=1.0, transX=None, transW=None):
        overload = 1 if transX is None else 2
        tx = X_NOTRANS if transX is None else transX
        tw = X_NOTRANS if transW is None else transW
        shape = mm_shape(x.shape, tx, w.shape, tw)
        c = np.zeros(shape, np.float32)
        cd = (C.c_int * 8)()
        order = self.lib.ref_mulandshift(overload, _f(x), tx, _dims(x.shape), x.ndim, _f(w), tw, _dims(w.shape), w.ndim,
                                         _f(bias), _dims(bias.shape), bias.ndim, _f(c), cd, alpha)
        assert tuple(cd[i] for i in range(order)) == shape
        return c

    def reduce_sum(self, x, dim):
        out = np.zeros(x.shape[:dim] + x.shape[dim + 1:], np.float32)
        self.lib.ref_reduce_sum(_f(x), _dims(x.shape), x.ndim, dim, _f(out))
        return out

    def grad(self, kind, a, transA, b, transB, dedc, alpha, deda, dedb, bias=None, dedbias=None):
        """Forward with the reference's operator (0 MatrixMul, 1 MatrixMulBatched, 2 MulAndShift), then
        its autograd step on the recorded edge; the gradients are updated in place."""
        self.lib.ref_grad(kind, _f(a), _dims(a.shape), a.ndim, transA, _f(b), _dims(b.shape), b.ndim, transB,
                          _f(bias) if bias is not None else None,
                          _dims(bias.shape) if bias is not None else None, 0 if bias is None else bias.ndim,
                          alpha, _f(dedc), _f(deda), _f(dedb), _f(dedbias) if dedbias is not None else None)
        return deda, dedb, dedbias

    def softmax(self, x):
        y = np.empty_like(x)
        self.lib.ref_softmax(_f(x), _dims(x.shape), x.ndim, _f(y))
        return y

    def attention(self, q, k, v, heads, scale, mask=None):
        batch, lq, hidden = q.shape
        out = np.zeros_like(q)
        self.lib.ref_attention(_f(q), _f(k), _f(v), _f(mask) if mask is not None else None, _f(out),
                               batch, lq, k.shape[1], hidden, heads, scale)
        return out

    def attention_probs(self, q, k, heads, scale, mask=None):
        batch, lq, hidden = q.shape
        probs = np.zeros((heads, batch, lq, k.shape[1]), np.float32)
        self.lib.ref_attention_probs(_f(q), _f(k), _f(mask) if mask is not None else None, _f(probs),
                                     batch, lq, k.shape[1], hidden, heads, scale)
        return probs

    def rectify(self, x):
        y = np.empty_like(x)
        self.lib.ref_rectify(_f(x), x.size, _f(y))
        return y

    def convert(self, x, type_t):
        type_s = NP_TYPE_CODE[x.dtype.type]
        x = np.ascontiguousarray(x)
        out = np.empty(x.shape, TYPE_CODE_NP[type_t])
        self.lib.ref_convert(x.ctypes.data, type_s, out.ctypes.data, type_t, x.size)
        return out

    def run_matmul_tests(self):
        return self.lib.ref_run_matmul_tests()

    def enum_values(self):
        out = (C.c_int * 5)()
        self.lib.ref_enum_values(out)
        return dict(X_TRANS=out[0], X_NOTRANS=out[1], X_FLOAT=out[2], X_FLOAT16=out[3], sizeof_XTensor=out[4])
