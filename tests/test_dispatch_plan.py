"""The dispatcher of the C ABI without a GPU: in planning-only mode (ntsamd_plan_only, a test aid that is exported
but not declared in include/ntsamd_gemm.h) a call stops before it touches a device and ntsamd_last_plan tells
what it would have launched. Checked here: the baseline's configurations land on the kernels written for them, and
over a few thousand random shapes no product that the 16-byte routes accept is ever sent to the element-wise
fallback (the kernel that is an order of magnitude slower), whatever tile shape and number of pieces the estimate
picks."""
import random

import pytest

import niutensor_amd as nt
from niutensor_amd import X_NOTRANS, X_TRANS

F32, F16 = nt.X_FLOAT, nt.X_FLOAT16


@pytest.fixture()
def planning():
    nt.load()
    for knob in ("NTSAMD_TILE_CFG", "NTSAMD_SPLIT_K", "NTSAMD_F16_FETCH", "NTSAMD_F16_PERSIST", "NTSAMD_F16_REPITCH",
                 "NTSAMD_A32_CONVERT", "NTSAMD_F32_SPLIT_ATOMIC", "NTSAMD_F16_SLAB64"):
        nt.tuning_set(knob, None)
    nt.plan_only(True)
    yield nt.load()
    nt.plan_only(False)
    nt.tuning_set("NTSAMD_TILE_CFG", None)
    nt.tuning_set("NTSAMD_SPLIT_K", None)


def plan_mm(L, M, N, K, ta, tb, types=(F32, F32, F32), beta=0.0, pa=0x100000, pb=0x200000, pc=0x300000, bias=None,
            bias_mode=nt.BIAS_COL, static_splits=None):
    na, ma = (M, K) if ta == X_NOTRANS else (K, M)
    nb, mb = (K, N) if tb == X_NOTRANS else (N, K)
    head = (0, None, pa, ta, types[0], pb, tb, types[1], pc, types[2], na, ma, nb, mb, M, N, 1.0, beta)
    if static_splits is not None:
        rc = L.ntsamd_matrix_mul_static(*head, static_splits)
    elif bias is not None:
        rc = L.ntsamd_matrix_mul_bias(*head, bias, bias_mode, N if bias_mode == nt.BIAS_COL else M, 1)
    else:
        rc = L.ntsamd_matrix_mul(*head)
    return rc, nt.last_plan()


def test_the_baseline_configurations_land_on_their_kernels(planning):
    L = planning
    rc, plan = plan_mm(L, 4096, 2048, 512, X_NOTRANS, X_NOTRANS)
    assert rc == 0 and plan == "gemm_f32_kernel tile=128x128 layout=NN fetch=vec16 splits=1"
    rc, plan = plan_mm(L, 4096, 2048, 512, X_NOTRANS, X_NOTRANS, bias=0x400000)
    assert rc == 0 and plan == "gemm_f32_kernel tile=128x128 layout=NN fetch=vec16 splits=1 bias=col"
    rc = L.ntsamd_matrix_mul_batched_strided(0, None, 0x100000, X_NOTRANS, F32, 8192, 0x200000, X_TRANS, F32, 8192,
                                             0x300000, F32, 16384, 256, 128, 64, 128, 64, 128, 128, 0.125, 0.0)
    assert rc == 0 and nt.last_plan() == "gemm_f32_kernel tile=64x64 layout=NT fetch=vec16 splits=1 strided"
    rc, plan = plan_mm(L, 8192, 4096, 1024, X_TRANS, X_NOTRANS, (F16, F16, F16))
    assert rc == 0 and plan == "gemm_f16_persistent_kernel tile=256x256,walk layout=TN fetch=lds-direct splits=1"
    rc, plan = plan_mm(L, 4096, 30011, 512, X_NOTRANS, X_TRANS, beta=1.0)
    assert rc == 0 and plan == "gemm_f32_kernel tile=128x128 layout=NT fetch=vec16 splits=1 beta"


def test_plans_name_the_passes_around_the_product(planning):
    L = planning
    # a half weight gradient: k cut into pieces that a second kernel adds up
    rc, plan = plan_mm(L, 512, 512, 4096, X_TRANS, X_NOTRANS, (F16, F16, F16), beta=1.0)
    assert rc == 0 and "gemm_f16_direct_kernel" in plan and "+split_reduce_kernel" in plan
    # rows of 30011 halves in the small operand: copied with padded rows, then the main path
    rc, plan = plan_mm(L, 4096, 30011, 512, X_NOTRANS, X_NOTRANS, (F16, F16, F16))
    assert rc == 0 and plan.startswith("repitch_f16_kernel(b)+gemm_f16_direct_kernel") and "fetch=lds-direct" in plan
    # a long product with a float a: rounded once, then all half
    rc, plan = plan_mm(L, 8192, 4096, 1024, X_NOTRANS, X_NOTRANS, (F32, F16, F16))
    assert rc == 0 and plan.startswith("convert_kernel(a to half)+gemm_f16_persistent_kernel")
    # few tiles of the small half shape: slabs of 64 along k; four workgroups to a CU: slabs of 32
    rc, plan = plan_mm(L, 1024, 1024, 4096, X_NOTRANS, X_TRANS, (F16, F16, F16))
    assert rc == 0 and plan.startswith("gemm_f16_direct_kernel tile=64x64,slab64 ")
    nt.tuning_set("NTSAMD_TILE_CFG", 1)
    rc, plan = plan_mm(L, 4096, 1024, 512, X_NOTRANS, X_TRANS, (F16, F16, F16))
    assert rc == 0 and plan.startswith("gemm_f16_direct_kernel tile=64x64 ")
    nt.tuning_set("NTSAMD_TILE_CFG", None)
    # a short one: rounded where it is fetched
    rc, plan = plan_mm(L, 128, 64, 128, X_NOTRANS, X_NOTRANS, (F32, F16, F16))
    assert rc == 0 and plan == "gemm_f16_kernel tile=64x64 layout=NN fetch=staged16,a float splits=1"


def test_an_explicit_number_of_pieces_is_honoured_or_refused(planning):
    L = planning
    rc, plan = plan_mm(L, 512, 512, 4096, X_TRANS, X_NOTRANS, (F16, F16, F16), static_splits=8)
    assert rc == 0 and "splits=8+split_reduce_kernel" in plan
    # half operands at odd addresses with odd rows can be cut too (the register-staged fetch)
    rc, plan = plan_mm(L, 500, 510, 4100, X_TRANS, X_NOTRANS, (F16, F16, F16), pa=0x100002, static_splits=4)
    assert rc == 0 and "gemm_f16_kernel" in plan and "splits=4+split_reduce_kernel" in plan
    # the big half tile has no kernel for pieces: asked for both, the call is refused, not run in one piece
    nt.tuning_set("NTSAMD_TILE_CFG", 2)
    rc, plan = plan_mm(L, 512, 512, 4096, X_TRANS, X_NOTRANS, (F16, F16, F16), static_splits=8)
    assert rc == 1 and "cannot be cut into 8 pieces" in L.ntsamd_last_error().decode()
    nt.tuning_set("NTSAMD_TILE_CFG", None)


def test_no_product_the_16_byte_routes_accept_goes_element_wise(planning):
    L = planning
    rng = random.Random(20251)
    seen = {}
    for case in range(4000):
        half = rng.random() < 0.5
        M = rng.choice((1, 7, 16, 33, 64, 100, 128, 257, 512, 1000, 2048, 4096, 8192))
        N = rng.choice((1, 8, 31, 64, 120, 128, 256, 500, 512, 2048, 4096, 30011))
        K = rng.choice((1, 5, 32, 64, 100, 128, 256, 512, 1024, 4096, 30011))
        ta, tb = rng.choice((X_TRANS, X_NOTRANS)), rng.choice((X_TRANS, X_NOTRANS))
        beta = rng.choice((0.0, 0.0, 1.0, 0.5))
        if half:
            types = rng.choice(((F16, F16, F16), (F16, F16, F16), (F16, F16, F32), (F32, F16, F16), (F32, F16, F32)))
            odd = rng.choice((0, 0, 2, 6))       # bases that are only 2-byte aligned
        else:
            types = (F32, F32, F32)
            odd = rng.choice((0, 0, 4, 12))      # bases that are only 4-byte aligned
        bias = 0x400000 if rng.random() < 0.3 else None
        rc, plan = plan_mm(L, M, N, K, ta, tb, types, beta, pa=0x100000 + odd, pb=0x200000 + odd, pc=0x300000 + odd, bias=bias)
        what = "case %d: %s %dx%dx%d %d%d beta=%g odd=%d bias=%s -> %s" % (case, types, M, N, K, ta, tb, beta, odd, bias, plan)
        assert rc == 0, what + " / " + L.ntsamd_last_error().decode()
        assert "fetch=elementwise" not in plan, what
        if half and types[0] == F16 and odd == 0 and M % 8 == 0 and N % 8 == 0 and K % 8 == 0:
            assert "fetch=lds-direct" in plan, what
        seen[plan.split(" layout")[0]] = seen.get(plan.split(" layout")[0], 0) + 1
    # the draw reaches every family and the walking kernel
    for family in ("gemm_f32_kernel", "gemm_f16_direct_kernel", "gemm_f16_kernel", "gemm_f16_persistent_kernel"):
        assert any(family in k for k in seen), (family, sorted(seen))
    # a bias by row is a pass of its own behind a product on the fast kernels; rows of 2^21 elements are what the
    # element-wise kernel is for
    rc, plan = plan_mm(L, 64, 64, 64, X_NOTRANS, X_NOTRANS, bias=0x400000, bias_mode=nt.BIAS_ROW)
    assert rc == 0 and "fetch=vec16" in plan and "+row_bias_kernel" in plan
    rc, plan = plan_mm(L, 4, 1 << 21, 8, X_NOTRANS, X_NOTRANS)
    assert rc == 0 and "fetch=elementwise" in plan


def test_the_traffic_table_was_read_with_todays_kernels(planning):
    """profiles/hbm_traffic_per_step.md names, per configuration, what the library launched when its counters were
    read; bench.py reports a row as stale when that differs from what it launches. Here, without a GPU: the rows of
    the baseline's single products still name what the dispatcher plans for them."""
    import bench
    L = planning
    for idx, args, kw in ((1, (4096, 2048, 512, X_NOTRANS, X_NOTRANS), {}),
                          (2, (4096, 2048, 512, X_NOTRANS, X_NOTRANS), {"bias": 0x400000}),
                          (4, (8192, 4096, 1024, X_TRANS, X_NOTRANS, (F16, F16, F16)), {}),
                          (5, (4096, 30011, 512, X_NOTRANS, X_TRANS), {"beta": 1.0})):
        rc, plan = plan_mm(L, *args, **kw)
        traffic, taken_with = bench.measured_traffic(idx)
        assert rc == 0 and traffic and taken_with == plan, (idx, plan, taken_with)
