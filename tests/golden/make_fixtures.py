"""Writes tests/golden/ref_generated.npz from the COMPILED reference (oracle/_ref/libnts_ref.so).

Run in a container that holds the NiuTensor tree (`make -C oracle ref` first):

    python tests/golden/make_fixtures.py

The file holds inputs and the outputs the real NiuTensor CPU implementation
produced for them, for the parts of the path its own tests do not cover:
NT/TT products, alpha/beta, N-D dispatch (flatten rule, (p,q) pairing, a
transposed N-D a against a shared 2-D b), the allocating wrapper's result
shape, GetBroadcastDimIndex, and MulAndShift (no TMulAndShift exists in the
reference). Only data is stored; the tests compare the C restatement and the
GPU path against it.
"""
import itertools
import os
import sys

import numpy as np

ROOT = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
sys.path.insert(0, ROOT)
from oracle.binding import Oracle, Reference, X_TRANS, X_NOTRANS, mm_shape, bmm_shape  # noqa: E402


def main():
    o = Oracle()
    r = Reference()
    out = {}
    index = []

    def put(name, **arrays):
        index.append(name)
        for k, v in arrays.items():
            out["%s/%s" % (name, k)] = np.asarray(v)

    seed = 1000

    # 2-D products: every transpose pair, alpha/beta, ragged sizes
    for (M, N, K) in ((5, 7, 3), (19, 13, 21), (1, 9, 4), (9, 1, 40)):
        for ta, tb in itertools.product((X_NOTRANS, X_TRANS), repeat=2):
            for alpha, beta in ((1.0, 0.0), (0.5, 1.0)):
                seed += 3
                a = o.uniform((K, M) if ta == X_TRANS else (M, K), seed)
                b = o.uniform((N, K) if tb == X_TRANS else (K, N), seed + 1)
                c0 = o.uniform((M, N), seed + 2)
                c = r.matmul2d(a, ta, b, tb, c0.copy(), alpha, beta)
                put("mm2d_%dx%dx%d_%d%d_a%g_b%g" % (M, N, K, ta, tb, alpha, beta), kind="matmul2d",
                    a=a, b=b, c0=c0, c=c, params=[ta, tb], scal=[alpha, beta])

    # N-D dispatch of _MatrixMul
    nd_cases = [
        ((3, 2, 3), X_NOTRANS, (3, 4), X_NOTRANS),          # flatten rule
        ((2, 3, 5, 4), X_NOTRANS, (6, 4), X_TRANS),         # flatten rule, b transposed
        ((3, 4, 5), X_TRANS, (4, 6), X_NOTRANS),            # transposed N-D a, shared b: no flattening
        ((3, 2, 3), X_NOTRANS, (2, 3, 2), X_NOTRANS),       # (p,q) pairing
        ((2, 4, 3), X_TRANS, (3, 5, 4), X_TRANS),           # (p,q) pairing, both transposed
        ((2, 2, 3, 4), X_NOTRANS, (2, 4, 5), X_NOTRANS),    # order 4 x order 3
        ((6, 5), X_NOTRANS, (3, 5, 2), X_NOTRANS),          # 2-D a against N-D b
    ]
    for i, (sa, ta, sb, tb) in enumerate(nd_cases):
        for alpha, beta in ((1.0, 0.0), (0.75, 1.0)):
            seed += 3
            a = o.uniform(sa, seed)
            b = o.uniform(sb, seed + 1)
            calloc, shape = r.matmul_alloc(a, ta, b, tb, alpha)
            c0 = o.uniform(shape, seed + 2)
            c = r.matmul(a, ta, b, tb, c0.copy(), alpha, beta)
            put("mmnd_%d_a%g_b%g" % (i, alpha, beta), kind="matmul", a=a, b=b, c0=c0, c=c, calloc=calloc,
                params=[ta, tb], scal=[alpha, beta])

    # same-order batched products
    for i, (sa, ta, sb, tb) in enumerate([
        ((4, 6, 5), X_NOTRANS, (4, 7, 5), X_TRANS),
        ((2, 3, 5, 6), X_TRANS, (2, 3, 5, 4), X_NOTRANS),
        ((3, 8, 8), X_NOTRANS, (3, 8, 8), X_NOTRANS),
        ((5, 4, 9), X_TRANS, (5, 3, 4), X_TRANS),
    ]):
        for alpha, beta in ((0.125, 0.0), (1.0, 1.0)):
            seed += 3
            a = o.uniform(sa, seed)
            b = o.uniform(sb, seed + 1)
            c = r.matmul_batched(a, ta, b, tb, None, alpha, 0.0)
            c0 = o.uniform(c.shape, seed + 2)
            c = r.matmul_batched(a, ta, b, tb, c0.copy(), alpha, beta)
            put("bmm_%d_a%g_b%g" % (i, alpha, beta), kind="matmul_batched", a=a, b=b, c0=c0, c=c,
                params=[ta, tb], scal=[alpha, beta])

    # GetBroadcastDimIndex over small shapes
    rows = []
    dims = (1, 2, 3)
    for ao in (1, 2, 3):
        for ashape in itertools.product(dims, repeat=ao):
            for bo in (1, 2, 3):
                for bshape in itertools.product(dims, repeat=bo):
                    n = r.broadcast_dim_index(ashape, bshape)
                    rows.append(list(ashape) + [0] * (3 - ao) + [ao] + list(bshape) + [0] * (3 - bo) + [bo] + [n])
    put("broadcast_dim_index", kind="broadcast", table=np.array(rows, np.int32))

    # MulAndShift: both overloads; bias on the last dimension and on an earlier one
    mas = [
        (1, (6, 5), None, (5, 4), None, (4,), 1.0),
        (1, (3, 4, 5), None, (5, 7), None, (7,), 1.0),
        (1, (3, 4, 5), None, (5, 7), None, (1, 7), 0.5),
        (1, (2, 3, 4, 5), None, (5, 6), None, (6,), 2.0),
        (1, (3, 4, 5), None, (5, 7), None, (4,), 1.0),            # bias matches dim 1: column broadcast
        (1, (3, 4, 5), None, (5, 7), None, (3, 1, 1), 1.0),        # bias matches dim 0
        (1, (7, 7, 5), None, (5, 7), None, (7,), 1.0),             # several dims of size 7: the last one wins
        (2, (6, 5), X_NOTRANS, (4, 5), X_TRANS, (4,), 1.0),
        (2, (5, 6), X_TRANS, (5, 4), X_NOTRANS, (4,), 0.5),
        (2, (3, 4, 5), X_NOTRANS, (7, 5), X_TRANS, (7,), 1.0),
        (2, (5, 6), X_TRANS, (4, 5), X_TRANS, (6,), 1.0),          # bias matches the row dimension
    ]
    for i, (ov, sx, tx, sw, tw, sb, alpha) in enumerate(mas):
        seed += 3
        x = o.uniform(sx, seed)
        w = o.normal(sw, seed + 1, 0.0, 0.5)
        bias = o.normal(sb, seed + 2, 0.0, 0.5)
        c = r.mulandshift(x, w, bias, alpha, tx, tw)
        put("mas_%d" % i, kind="mulandshift", x=x, w=w, bias=bias, c=c,
            params=[ov, X_NOTRANS if tx is None else tx, X_NOTRANS if tw is None else tw], scal=[alpha])

    out["index"] = np.array(index)
    path = os.path.join(os.path.dirname(os.path.abspath(__file__)), "ref_generated.npz")
    np.savez_compressed(path, **out)
    print("wrote", path, len(index), "cases", os.path.getsize(path), "bytes")


def backward():
    o = Oracle()
    r = Reference()
    out = {}
    index = []

    def put(name, **arrays):
        index.append(name)
        for k, v in arrays.items():
            out["%s/%s" % (name, k)] = np.asarray(v)

    seed = 5000

    # _ReduceSum: scalar loop, column buffers, and the 32-lane fold over a contiguous last dimension
    for i, (shape, dim) in enumerate([((7, 5), 0), ((9, 64), 0), ((5, 96), 1), ((6, 160), 1), ((4, 6, 32), 2),
                                      ((4, 6, 33), 2), ((3, 5, 7), 1), ((70, 128), 0), ((4, 6, 32), 0)]):
        seed += 1
        x = o.uniform(shape, seed)
        put("reduce_%d" % i, kind="reduce_sum", x=x, y=r.reduce_sum(x, dim), params=[dim])

    # GradMatrixMul: 2-D, all transposes; flatten rule
    mm = [((9, 7), (7, 5)), ((33, 20), (20, 17))]
    for i, (sa, sb) in enumerate(mm):
        for ta, tb in itertools.product((X_NOTRANS, X_TRANS), repeat=2):
            seed += 6
            M, K = sa
            N = sb[1]
            a = o.uniform((K, M) if ta == X_TRANS else (M, K), seed)
            b = o.uniform((N, K) if tb == X_TRANS else (K, N), seed + 1)
            dedc = o.uniform((M, N), seed + 2)
            deda0, dedb0 = o.uniform(a.shape, seed + 3), o.uniform(b.shape, seed + 4)
            deda, dedb, _ = r.grad(0, a, ta, b, tb, dedc, 0.75, deda0.copy(), dedb0.copy())
            put("gmm_%d_%d%d" % (i, ta, tb), kind="grad_matmul", a=a, b=b, dedc=dedc, deda0=deda0, dedb0=dedb0,
                deda=deda, dedb=dedb, params=[ta, tb], scal=[0.75])
    for i, (sa, sb, tb) in enumerate([((3, 4, 6), (6, 5), X_NOTRANS), ((2, 3, 4, 6), (5, 6), X_TRANS)]):
        seed += 6
        a, b = o.uniform(sa, seed), o.uniform(sb, seed + 1)
        dedc = o.uniform(mm_shape(sa, X_NOTRANS, sb, tb), seed + 2)
        deda0, dedb0 = o.uniform(sa, seed + 3), o.uniform(sb, seed + 4)
        deda, dedb, _ = r.grad(0, a, X_NOTRANS, b, tb, dedc, 1.0, deda0.copy(), dedb0.copy())
        put("gmm_flat_%d" % i, kind="grad_matmul", a=a, b=b, dedc=dedc, deda0=deda0, dedb0=dedb0,
            deda=deda, dedb=dedb, params=[X_NOTRANS, tb], scal=[1.0])

    # GradMatrixMulBatched
    for ta, tb in itertools.product((X_NOTRANS, X_TRANS), repeat=2):
        seed += 6
        M, K, N = 6, 9, 5
        a = o.uniform((4, K, M) if ta == X_TRANS else (4, M, K), seed)
        b = o.uniform((4, N, K) if tb == X_TRANS else (4, K, N), seed + 1)
        dedc = o.uniform(bmm_shape(a.shape, ta, b.shape, tb), seed + 2)
        deda0, dedb0 = o.uniform(a.shape, seed + 3), o.uniform(b.shape, seed + 4)
        deda, dedb, _ = r.grad(1, a, ta, b, tb, dedc, 0.125, deda0.copy(), dedb0.copy())
        put("gbmm_%d%d" % (ta, tb), kind="grad_matmul_batched", a=a, b=b, dedc=dedc, deda0=deda0, dedb0=dedb0,
            deda=deda, dedb=dedb, params=[ta, tb], scal=[0.125])

    # GradMulAndShift (first overload): bias on the last dimension (with and without the 32-lane
    # buffers), on a middle one and on the first
    for i, (sx, sw, sb) in enumerate([((4, 6, 8), (8, 64), (64,)), ((4, 6, 8), (8, 5), (5,)), ((12, 8), (8, 32), (32,)),
                                      ((5, 6, 8), (8, 7), (6,)), ((4, 32, 8), (8, 32), (4,)), ((3, 6, 8), (8, 6), (6,))]):
        seed += 8
        x, w, bias = o.uniform(sx, seed), o.normal(sw, seed + 1, 0, 0.5), o.normal(sb, seed + 2, 0, 0.5)
        cshape = mm_shape(sx, X_NOTRANS, sw, X_NOTRANS)
        dedc = o.uniform(cshape, seed + 3)
        dedx0, dedw0, dedb0 = o.uniform(sx, seed + 4), o.uniform(sw, seed + 5), o.uniform(sb, seed + 6)
        dedx, dedw, dedb = r.grad(2, x, X_NOTRANS, w, X_NOTRANS, dedc, 0.5, dedx0.copy(), dedw0.copy(), bias, dedb0.copy())
        put("gmas_%d" % i, kind="grad_mulandshift", x=x, w=w, bias=bias, dedc=dedc, dedx0=dedx0, dedw0=dedw0,
            dedb0=dedb0, dedx=dedx, dedw=dedw, dedb=dedb, params=[r.broadcast_dim_index(cshape, sb)], scal=[0.5])

    out["index"] = np.array(index)
    path = os.path.join(os.path.dirname(os.path.abspath(__file__)), "ref_generated_backward.npz")
    np.savez_compressed(path, **out)
    print("wrote", path, len(index), "cases", os.path.getsize(path), "bytes")


def attention():
    o = Oracle()
    r = Reference()
    out = {}
    index = []

    def put(name, **arrays):
        index.append(name)
        for k, v in arrays.items():
            out["%s/%s" % (name, k)] = np.asarray(v)

    seed = 9000
    # _Softmax over the last dimension: scalar sums, 32-lane sums, a constant row, large magnitudes
    for i, (shape, std) in enumerate([((5, 7), 1.0), ((3, 32), 3.0), ((4, 96), 3.0), ((2, 3, 40), 1.0), ((6, 128), 0.5),
                                      ((2, 1), 1.0), ((3, 33), 30.0), ((2, 64), 0.0)]):
        seed += 1
        x = o.normal(shape, seed, 0.0, std) if std > 0 else np.full(shape, 2.5, np.float32)
        put("softmax_%d" % i, kind="softmax", x=x, y=r.softmax(x))

    # attention: (batch, lq, lk, hidden, heads, masked)
    cases = [(2, 5, 7, 8, 2, 0), (2, 9, 9, 16, 4, 1), (3, 33, 64, 32, 2, 1), (1, 40, 32, 24, 3, 0), (2, 64, 100, 128, 2, 1),
             (1, 130, 200, 64, 1, 1), (2, 16, 300, 96, 1, 0), (1, 1, 1, 4, 1, 0), (2, 20, 50, 256, 2, 2)]
    for i, (B, lq, lk, H, nh, masked) in enumerate(cases):
        seed += 4
        q, k, v = o.normal((B, lq, H), seed), o.normal((B, lk, H), seed + 1), o.normal((B, lk, H), seed + 2)
        mask = None
        if masked == 1:
            # the sample's masks hold 0 and -1e9 (Model.cpp:249-258, 310-337)
            mask = np.where(o.uniform((nh, B, lq, lk), seed + 3, 0.0, 1.0) < 0.3, -1e9, 0.0).astype(np.float32)
            mask[..., 0] = 0.0                                  # every row keeps one key
        elif masked == 2:
            # causal: row i sees keys 0..i
            mask = np.broadcast_to(np.where(np.arange(lk)[None, :] > np.arange(lq)[:, None], -1e9, 0.0),
                                   (nh, B, lq, lk)).astype(np.float32).copy()
        scale = float(np.float32(1.0 / np.sqrt(H / nh)))
        y = r.attention(q, k, v, nh, scale, mask)
        arrays = dict(kind="attention", q=q, k=k, v=v, out=y, params=[nh], scal=[scale])
        if mask is not None:
            arrays["mask"] = mask
        put("attention_%d" % i, **arrays)

    out["index"] = np.array(index)
    path = os.path.join(os.path.dirname(os.path.abspath(__file__)), "ref_generated_attention.npz")
    np.savez_compressed(path, **out)
    print("wrote", path, len(index), "cases", os.path.getsize(path), "bytes")


if __name__ == "__main__":
    main()
    backward()
    attention()
