"""The entry points never synchronise, so a caller may record them into a HIP graph on its own stream and
replay it: a linear layer with Rectify, the two attention products, the attention in one kernel, a float
product cut along k (atomics after a scaling pass), a half product cut along k (partial products in the
library's workspace, which the capturing stream does not have yet: the one allocation the library makes,
in the relaxed capture mode) and a conversion are captured once and replayed with new inputs; every
replay must reproduce the eager results bit for bit (the float product cut along k, whose additions are
unordered: within the fp32 limit)."""

import numpy as np
import pytest

import niutensor_amd as nt
from niutensor_amd import X_NOTRANS, X_TRANS
from tolerance import assert_fp32

pytestmark = pytest.mark.gpu


def test_replays_match_eager(gpu, oracle):
    import torch
    print("\n[gpu-case] tests/test_gpu_graph.py::test_replays_match_eager", flush=True)
    dev = gpu
    g = lambda x: torch.from_numpy(np.ascontiguousarray(x)).to(dev)
    x, w, b = g(oracle.uniform((256, 96), 1)), g(oracle.normal((96, 160), 2, 0, 0.1)), g(oracle.normal((160,), 3))
    q, k, v = (g(oracle.normal((4, 70, 64), s)) for s in (4, 5, 6))
    big_a, big_b = g(oracle.uniform((64, 2048), 7)), g(oracle.uniform((2048, 64), 8))
    h = torch.empty((256, 160), device=dev)
    s = torch.empty((4, 70, 70), device=dev)
    o = torch.empty((4, 70, 64), device=dev)
    att = torch.empty((4, 70, 64), device=dev)
    cut = torch.empty((64, 64), device=dev)
    h16 = torch.empty((256, 160), device=dev, dtype=torch.float16)
    big_a16, big_b16 = big_a.half(), big_b.half()
    cut16 = torch.empty((64, 64), device=dev, dtype=torch.float16)

    def step():
        nt.matrix_mul(x, X_NOTRANS, w, X_NOTRANS, h, 1.0, 0.0, bias=b, act=nt.ACT_RECTIFY)
        nt.matrix_mul_batched_strided(q, X_NOTRANS, k, X_TRANS, s, 4, 70 * 64, 70 * 64, 70 * 70, 70, 64, 70, 64, 70, 70, 0.125, 0.0)
        nt.matrix_mul_batched_strided(s, X_NOTRANS, v, X_NOTRANS, o, 4, 70 * 70, 70 * 64, 70 * 64, 70, 70, 70, 64, 70, 64, 1.0, 0.0)
        nt.attention(q, k, v, att, 2, 0.25)
        nt.matrix_mul(big_a, X_NOTRANS, big_b, X_NOTRANS, cut, 1.0, 0.0)
        nt.convert_data_type(h, h16)
        nt.matrix_mul(big_a16, X_NOTRANS, big_b16, X_NOTRANS, cut16, 1.0, 0.0)

    nt.tuning_set("NTSAMD_SPLIT_K", "4")                  # the product with the long k goes out in four pieces
    try:
        side = torch.cuda.Stream()
        side.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(side):
            step()                                      # warm-up outside the capture (loads the code objects)
        torch.cuda.current_stream().wait_stream(side)
        torch.cuda.synchronize()
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph):
            step()
        for rep in range(3):
            # new inputs in place, eager results first
            for t, seed in ((x, 10), (q, 11), (k, 12), (v, 13), (big_a, 14)):
                t.copy_(g(oracle.uniform(tuple(t.shape), seed + 10 * rep)))
            big_a16.copy_(big_a)
            step()
            torch.cuda.synchronize()
            want = [t.clone() for t in (h, s, o, att, cut, h16, cut16)]
            for t in (h, s, o, att, cut, h16, cut16):
                t.fill_(float("nan"))
            graph.replay()
            torch.cuda.synchronize()
            for name, got, ref in zip(("linear layer", "scores", "context", "attention", "cut along k", "conversion",
                                       "half, cut along k"), (h, s, o, att, cut, h16, cut16), want):
                if name == "cut along k":
                    assert_fp32(got.cpu().numpy(), ref.cpu().numpy(), 2048, what="replay %d: %s" % (rep, name))
                else:
                    assert torch.equal(got, ref), "replay %d: %s" % (rep, name)
    finally:
        nt.tuning_set("NTSAMD_SPLIT_K", None)
