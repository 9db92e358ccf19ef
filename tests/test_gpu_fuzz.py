"""A bounded random walk over what the dispatcher of the C ABI can be asked for: 320 cases from one fixed seed, drawn
over the data type triple, the four layouts, rows that are whole 16-byte pieces or not, bases that are 16-byte aligned
or not, alpha and beta, the bias modes and the activation, the kinds of batch (none, strided with or without a shared
operand, a list of pointers, a grid inside merged tensors), the column-sum by-product, and plans left to the library or
forced through its measurement knobs. Every case is printed before it is launched and compared with a float64
evaluation of the same operands (torch on the device); the first failure stops the test. About 20 s on one MI355X."""
import math

import numpy as np
import pytest

import niutensor_amd as nt
from niutensor_amd import X_NOTRANS, X_TRANS

pytestmark = pytest.mark.gpu

CASES = 320
KNOBS = {
    "NTSAMD_TILE_CFG": (None, None, None, 0, 1, 2, 3, 4),
    "NTSAMD_SPLIT_K": (None, None, None, 1, 2, 4, 8),
    "NTSAMD_F16_FETCH": (None, None, None, None, 2, 0),
    "NTSAMD_F16_PERSIST": (None, None, 0, 2, 3, 4),
    "NTSAMD_F16_PINGPONG": (None, None, 0),
    "NTSAMD_F16_REPITCH": (None, 0, 1),
    "NTSAMD_A32_CONVERT": (None, 0, 1),
    "NTSAMD_F32_R16": (None, None, 0),
    "NTSAMD_STORE_HINT": (None, None, 0, 1),
    "NTSAMD_GROUP_M": (None, None, 1, 3),
    "NTSAMD_F16_SLAB64": (None, None, 0, 1),
}


def draw_dim(rng, big):
    d = int(rng.integers(1, 1100 if big else 200))
    r = rng.random()
    if r < 0.5:
        d = max(8, d // 8 * 8)          # rows of whole 16-byte pieces in either type
    elif r < 0.6:
        d = max(4, d // 4 * 4)
    return d


def test_random_products_agree_with_float64(gpu):
    import torch
    rng = np.random.default_rng(20251125)
    T, NT = X_TRANS, X_NOTRANS
    dd = lambda t: t.double()

    def device(shape, dtype, off, lo=-1.0, hi=1.0):
        """a dense device tensor of that shape whose first element stands `off` elements into its allocation"""
        n = int(np.prod(shape))
        host = torch.from_numpy(rng.uniform(lo, hi, n + off).astype(np.float32))
        return host.to(gpu).to(dtype)[off:].view(*shape)

    families = {}
    for case in range(CASES):
        kind = str(rng.choice(["single", "single", "single", "strided", "list", "grid", "colsum"]))
        types = str(rng.choice(["f32", "f32", "f16", "f16", "f16_f32out", "a32_f16", "a32_f32out"]))
        if kind in ("list", "colsum") and types in ("a32_f16", "a32_f32out", "f16_f32out"):
            types = "f16"
        ta_t = torch.float32 if types in ("f32", "a32_f16", "a32_f32out") else torch.float16
        tb_t = torch.float32 if types == "f32" else torch.float16
        tc_t = torch.float32 if types in ("f32", "f16_f32out", "a32_f32out") else torch.float16
        big = rng.random() < 0.35
        M, N = draw_dim(rng, big), draw_dim(rng, big)
        K = draw_dim(rng, False) if rng.random() < 0.6 else int(rng.integers(256, 2300)) // 8 * 8
        ta, tb = (T if rng.random() < 0.5 else NT for _ in range(2))
        alpha = float(rng.choice([1.0, 1.0, 0.5, -1.25]))
        beta = float(rng.choice([0.0, 0.0, 0.0, 1.0, 0.5]))
        off = int(rng.choice([0, 0, 0, 1, 3, 4]))
        knobs = {k: v[int(rng.integers(0, len(v)))] for k, v in KNOBS.items()}
        if rng.random() < 0.45:
            knobs = dict.fromkeys(knobs)                          # everything left to the library
        if case % 12 == 5:
            # a directed draw: the kernel that walks over tiles needs many tiles or its knob, whole 16-byte pieces
            # and a half result, which the free draw above meets too rarely
            kind, types = str(rng.choice(["single", "strided"])), "f16"
            ta_t = tb_t = tc_t = torch.float16
            M, N, K = int(rng.integers(1, 120)) * 8, int(rng.integers(1, 120)) * 8, int(rng.integers(32, 200)) * 8
            off = int(rng.choice([0, 0, 8]))
            if rng.random() < 0.5:
                knobs = dict(dict.fromkeys(knobs), NTSAMD_F16_PERSIST=2, NTSAMD_TILE_CFG=2)
            else:
                knobs = dict(dict.fromkeys(knobs), NTSAMD_F16_PERSIST=4)
                ta = NT
        sa = (K, M) if ta == T else (M, K)
        sb = (N, K) if tb == T else (K, N)
        count = 1 if kind in ("single", "colsum") else int(rng.integers(2, 5))
        shared_b = kind == "strided" and rng.random() < 0.3
        bias_mode = None
        act = nt.ACT_NONE
        if kind == "single" and rng.random() < 0.45:
            bias_mode = nt.BIAS_COL if rng.random() < 0.75 else nt.BIAS_ROW
            act = nt.ACT_RECTIFY if rng.random() < 0.4 else nt.ACT_NONE
        what = "case %d %s %s M=%d N=%d K=%d ta=%d tb=%d count=%d sharedB=%d alpha=%g beta=%g off=%d bias=%s act=%d knobs=%s" % (
            case, kind, types, M, N, K, ta, tb, count, shared_b, alpha, beta, off, bias_mode, act,
            {k[7:]: v for k, v in knobs.items() if v is not None})
        print("[gpu-case] " + what, flush=True)

        if kind == "grid":
            # heads of merged tensors, as the attention context: a [h][b][lq][lk], b [b][lk][h * dh], c [b][lq][h * dh]
            h, b = int(rng.integers(1, 4)), int(rng.integers(1, 3))
            lq, lk, dh = min(M, 300), min(K, 400), int(rng.choice([8, 16, 64, 72]))
            hid = h * dh
            a = device((h, b, lq, lk), ta_t, off, 0.0, 1.0)
            bm = device((b, lk, hid), tb_t, off)
            c0 = device((b, lq, hid), tc_t, off)
            c = c0.clone() if beta != 0 else torch.full_like(c0, float("nan"))
        else:
            a = device((count,) + sa, ta_t, off)
            bm = device(((1 if shared_b else count),) + sb, tb_t, off)
            c0 = device((count, M, N), tc_t, off)
            c = c0.clone() if beta != 0 else torch.full_like(c0, float("nan"))
        bias = None
        if bias_mode == nt.BIAS_COL:
            bias = device((N,), tc_t, off if tc_t == torch.float32 else 0)
        elif bias_mode == nt.BIAS_ROW:
            bias = device((M,), tc_t, 0)
        col_sum0 = device((N,), tc_t, 0) if kind == "colsum" else None
        col_sum = col_sum0.clone() if col_sum0 is not None else None
        col_beta = float(rng.choice([0.0, 1.0]))

        for k, v in knobs.items():
            nt.tuning_set(k, v)
        try:
            if kind == "single":
                nt.matrix_mul(a[0], ta, bm[0], tb, c[0], alpha, beta, bias=bias, bias_mode=bias_mode or nt.BIAS_COL, act=act)
            elif kind == "colsum":
                nt.matrix_mul_colsum(a[0], ta, bm[0], tb, c[0], col_sum, alpha, beta, col_beta)
            elif kind == "strided":
                nt.matrix_mul_batched_strided(a, ta, bm, tb, c, count, sa[0] * sa[1], 0 if shared_b else sb[0] * sb[1], M * N,
                                              sa[0], sa[1], sb[0], sb[1], M, N, alpha, beta)
            elif kind == "list":
                order = [int(i) for i in rng.permutation(count)]
                nt.matrix_mul_batched([a[i] for i in order], ta, [bm[i] for i in order], tb, [c[i] for i in order], alpha, beta)
            else:
                nt.matrix_mul_batched_grid(a, NT, lk, (lq * lk, b * lq * lk), bm, NT, hid, (lk * hid, dh),
                                           c, hid, (lq * hid, dh), b, h, lq, lk, lk, dh, lq, dh, alpha, beta)
            plan = nt.last_plan()
        finally:
            for k in knobs:
                nt.tuning_set(k, None)
        families[plan.split(" tile=")[0].split("+")[-1]] = families.get(plan.split(" tile=")[0].split("+")[-1], 0) + 1

        a64 = dd(a.half()) if tb_t == torch.float16 else dd(a)        # a float a with a half b is rounded to half first
        if kind == "grid":
            ref = torch.empty_like(c0, dtype=torch.float64)
            for bi in range(b):
                for hi in range(h):
                    ref[bi, :, hi * dh:(hi + 1) * dh] = a64[hi, bi] @ dd(bm[bi, :, hi * dh:(hi + 1) * dh])
            ref = alpha * ref
            kk = lk
        else:
            opa = a64.transpose(1, 2) if ta == T else a64
            opb = dd(bm).transpose(1, 2) if tb == T else dd(bm)
            ref = alpha * (opa @ opb)
            kk = K
        if beta != 0:
            ref = ref + beta * dd(c0)
        if bias_mode == nt.BIAS_COL:
            ref = ref + dd(bias)[None, None, :]
        elif bias_mode == nt.BIAS_ROW:
            ref = ref + dd(bias)[None, :, None]
        if act == nt.ACT_RECTIFY:
            ref = ref.clamp(min=0)
        limit = 1e-2 if tc_t == torch.float16 else 1e-5 * math.sqrt(max(kk, 16))
        assert bool(torch.isfinite(c).all()), what + " -> " + plan
        err = float((dd(c) - ref).abs().max() / ref.abs().max().clamp(min=1e-30))
        assert err <= limit, "%s -> %s: error %.3g, limit %.3g" % (what, plan, err, limit)
        if col_sum is not None:
            sums = (dd(bm[0]).sum(1) if tb == T else dd(bm[0]).sum(0)) + col_beta * dd(col_sum0)
            lim_s = 1e-2 if tc_t == torch.float16 else 1e-5 * math.sqrt(max(K, 16))
            err_s = float((dd(col_sum) - sums).abs().max() / sums.abs().max().clamp(min=1e-30))
            assert err_s <= lim_s, "%s -> %s: column sums off by %.3g, limit %.3g" % (what, plan, err_s, lim_s)
    print("kernel families reached: %s" % sorted(families.items()), flush=True)
    for family in ("gemm_f32_kernel", "gemm_f16_direct_kernel", "gemm_f16_kernel", "gemm_f16_persistent_kernel"):
        assert any(family in k for k in families), (family, families)
