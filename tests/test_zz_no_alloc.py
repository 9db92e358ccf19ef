"""The entry point that allocates nothing (ntsamd_matrix_mul_static: partial products of a k cut into pieces in
a static device array instead of an allocated workspace) against ntsamd_matrix_mul on the same inputs, through the
C ABI: two calls in a row, the second on a smaller product, so that the scratch still holds the first call's
partial products when the second starts. Both entry points run the same kernels on the same plan, so the results
must agree bit for bit; the first is also held against the CPU oracle."""
import numpy as np
import pytest

import niutensor_amd as nt
from niutensor_amd import X_NOTRANS, X_TRANS
from tolerance import assert_fp16, assert_fp32

pytestmark = pytest.mark.gpu


def halfed(oracle, x):
    return oracle.from_f16_bits(oracle.to_f16_bits(x))


@pytest.mark.parametrize("half", (True, False))
def test_static_scratch_matches_the_allocating_entry_point(gpu, oracle, half):
    import torch
    print("\n[gpu-case] static scratch, half=%d" % half, flush=True)
    nt.tuning_set("NTSAMD_TILE_CFG", None)
    for splits in (0, 8):
        # splits = 0: both entry points choose for themselves (these shapes are cut); 8: both are told to
        nt.tuning_set("NTSAMD_SPLIT_K", splits if splits else None)
        for step, (M, N, K) in enumerate(((512, 512, 4096), (200, 136, 2048))):
            a = oracle.normal((K, M), 10 + step, 0, 0.5)
            b = oracle.normal((K, N), 20 + step, 0, 0.5)
            c0 = oracle.uniform((M, N), 30 + step)
            if half:
                a, b, c0 = halfed(oracle, a), halfed(oracle, b), halfed(oracle, c0)
            dt = torch.float16 if half else torch.float32
            da, db = torch.from_numpy(a).to(gpu, dt), torch.from_numpy(b).to(gpu, dt)
            want, got = torch.from_numpy(c0).to(gpu, dt), torch.from_numpy(c0).to(gpu, dt)
            nt.matrix_mul(da, X_TRANS, db, X_NOTRANS, want, 0.5, 1.0)
            nt.matrix_mul_static(da, X_TRANS, db, X_NOTRANS, got, 0.5, 1.0, splits)
            what = "half=%d splits=%d %dx%dx%d" % (half, splits, M, N, K)
            assert torch.equal(got, want), what
            ref = oracle.matmul2d(a, X_TRANS, b, X_NOTRANS, c0.copy(), 0.5, 1.0)
            if half:
                assert_fp16(got.float().cpu().numpy(), ref, what=what)
            else:
                assert_fp32(got.cpu().numpy(), ref, K, what=what)
    nt.tuning_set("NTSAMD_SPLIT_K", None)


def test_static_scratch_refuses_what_does_not_fit(gpu):
    import torch
    a = torch.zeros((4096, 1024), device=gpu)
    b = torch.zeros((4096, 2048), device=gpu)
    c = torch.zeros((1024, 2048), device=gpu)
    with pytest.raises(nt.NtsAmdError, match="exceed the static scratch"):
        nt.matrix_mul_static(a, X_TRANS, b, X_NOTRANS, c, 1.0, 0.0, 4)       # 4 x 8 MiB of partial products
    with pytest.raises(nt.NtsAmdError, match="2, 4, 8 or 16"):
        nt.matrix_mul_static(a, X_TRANS, b, X_NOTRANS, c, 1.0, 0.0, 3)
    with pytest.raises(nt.NtsAmdError, match="too short"):
        nt.matrix_mul_static(a[:64], X_TRANS, b[:64], X_NOTRANS, c, 1.0, 0.0, 2)
    # left to the library, the same product runs (in fewer pieces, or one) and allocates nothing
    a.normal_()
    b.normal_()
    nt.matrix_mul_static(a, X_TRANS, b, X_NOTRANS, c, 1.0, 0.0, 0)
    want = torch.empty_like(c)
    nt.tuning_set("NTSAMD_SPLIT_K", 1)
    nt.matrix_mul(a, X_TRANS, b, X_NOTRANS, want)
    nt.tuning_set("NTSAMD_SPLIT_K", None)
    assert_fp32(c.cpu().numpy(), want.cpu().numpy(), 4096)
