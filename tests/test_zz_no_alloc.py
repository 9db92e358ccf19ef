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


def test_static_entry_point_allocates_nothing_and_can_be_recorded_into_a_graph(gpu, oracle):
    """The defining property, measured: after the library's workspaces are released, a product cut into 8 pieces
    through the static entry point on a stream that never had a workspace leaves the device's free memory where it
    was, and a release that follows finds nothing to free; the allocating entry point on the same stream, for
    contrast, takes its 32 MiB. Then the static call is recorded into a HIP graph (after one eager call of the same
    kind, which loads the kernels' code objects) and every replay gives the eager result."""
    import torch
    print("\n[gpu-case] static scratch: free memory and graph capture", flush=True)
    nt.tuning_set("NTSAMD_TILE_CFG", None)
    nt.tuning_set("NTSAMD_SPLIT_K", None)
    M, N, K = 256, 192, 4096
    for half in (False, True):
        dt = torch.float16 if half else torch.float32
        a = torch.from_numpy(oracle.normal((K, M), 40, 0, 0.5)).to(gpu, dt)
        b = torch.from_numpy(oracle.normal((K, N), 41, 0, 0.5)).to(gpu, dt)
        eager = torch.empty((M, N), device=gpu, dtype=dt)
        got = torch.full((M, N), float("nan"), device=gpu, dtype=dt)
        # one eager call of this kind first: its kernels' code objects are loaded at their first launch
        nt.matrix_mul_static(a, X_TRANS, b, X_NOTRANS, eager, 0.5, 0.0, 8)
        assert "splits=8+split_reduce_kernel" in nt.last_plan()
        side = torch.cuda.Stream(gpu)
        with torch.cuda.stream(side):
            torch.zeros(8, device=gpu).add_(1)              # the stream has run something: whatever it allocates for itself is there
        torch.cuda.synchronize()
        nt.release_workspaces(-1)
        torch.cuda.synchronize()
        free0 = torch.cuda.mem_get_info(gpu)[0]
        with torch.cuda.stream(side):
            nt.matrix_mul_static(a, X_TRANS, b, X_NOTRANS, got, 0.5, 0.0, 8)
        torch.cuda.synchronize()
        assert torch.cuda.mem_get_info(gpu)[0] == free0, "the static entry point changed the device's free memory"
        nt.release_workspaces(-1)
        assert torch.cuda.mem_get_info(gpu)[0] == free0, "there was a workspace to release after a static call"
        assert torch.equal(got, eager)
        # the contrast that shows the measurement sees an allocation: the allocating entry point, same stream, same plan
        nt.tuning_set("NTSAMD_SPLIT_K", 8)
        with torch.cuda.stream(side):
            nt.matrix_mul(a, X_TRANS, b, X_NOTRANS, got, 0.5, 0.0)
        torch.cuda.synchronize()
        nt.tuning_set("NTSAMD_SPLIT_K", None)
        assert free0 - torch.cuda.mem_get_info(gpu)[0] >= 32 << 20, "the allocating entry point took no workspace?"
        nt.release_workspaces(-1)
        assert torch.cuda.mem_get_info(gpu)[0] == free0
        assert torch.equal(got, eager)
        # under capture: nothing may allocate there; replays with eager work and synchronisation between them
        g = torch.cuda.CUDAGraph()
        got.fill_(float("nan"))
        torch.cuda.synchronize()
        with torch.cuda.graph(g):
            nt.matrix_mul_static(a, X_TRANS, b, X_NOTRANS, got, 0.5, 0.0, 8)
        for replay in range(3):
            got.fill_(float("nan"))
            g.replay()
            torch.cuda.synchronize()
            assert torch.equal(got, eager), "replay %d of the recorded static call, half=%d" % (replay, half)
            nt.matrix_mul_static(a, X_TRANS, b, X_NOTRANS, eager, 0.5, 0.0, 8)   # eager work between the replays
            torch.cuda.synchronize()
        del g
        ref = oracle.matmul2d(a.float().cpu().numpy(), X_TRANS, b.float().cpu().numpy(), X_NOTRANS, None, 0.5, 0.0)
        if half:
            assert_fp16(got.float().cpu().numpy(), ref, what="static call replayed from a graph, half")
        else:
            assert_fp32(got.cpu().numpy(), ref, K, what="static call replayed from a graph, float")
