#!/usr/bin/env python3
"""Benchmark of the gfx950 matrix-multiplication path.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--config N] [--all] [--no-cpu]

A "step" is one pass of the hot path over one batch of synthetic input that is
already resident in HBM: one launch of the configuration's product through the C
ABI (two launches for the attention pair). The default workload is the
MulAndShift linear layer, fp32 X[32x128x512] x W[512x2048] + b[2048]: the first
configuration the metric's target is quoted on. The headline line (the LAST line
printed) also carries, under "configs", the kernel time, TFLOP/s and fraction of
the matrix peak of every one of the baseline's five configurations, measured in
the same run. `--all` adds one full line per configuration before the headline.

Whatever --warmup says, every configuration first runs until SETTLE_S seconds of
GPU time have passed: the clocks of the part need tens of milliseconds of load to
settle, and a short warm-up would time the ramp.

Each JSON line carries
  value/unit       TFLOP/s = 2 M N K batch / time, over the timed steps
  roofline         the same kernel timed with HIP events on its own stream,
                   against the MI355X dense matrix peak of the data type;
                   kernel_us is with ONE set of buffers used again every step
                   (configurations 1-4 then sit in the 256 MB Infinity Cache),
                   kernel_us_rotated with enough sets in turn to exceed it
  check            the buffers the timed steps wrote, compared after the timed
                   region with a float64 evaluation of sampled rows (and every
                   element tested for being finite); a miss ends the run with
                   a non-zero exit code
  kernels          what the library planned for each launch of a step (kernel
                   family, tile shape, fetch route, pieces of k)
  nts_layer_us     the same operator through the nts:: C++ layer (a child
                   process: tests/cpp/build/nts_tests --bench)
  cpu_baseline     the reference's CPU path (1 thread, as the reference runs it)
                   on a bounded sample of the same product
"""
import argparse
import ctypes as C
import json
import math
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

PEAK_TFLOPS = {"f32": 157.3, "f16": 2516.6}     # MI355X dense matrix peaks (datasheet)
HBM_TBS = 8.0
SETTLE_S = 0.15                                 # GPU time under load before anything is timed
BASELINE_CONFIGS = (1, 2, 3, 4, 5)
ATTENTION_FORMS = (8, 15, 11, 12)               # configuration 3 as the transformer runs it: one kernel (inference, training), or the two halves of training
CACHE_BYTES = 256 << 20                         # Infinity Cache of the part
ROTATE_BYTES = 320 << 20                        # what the sets of buffers cycled by kernel_us_rotated add up to, at least
LAYOUT_OF_4 = "TN"                              # how configuration 4's operands are stored (--layout changes it)


def configs():
    """The five configurations of the baseline, 1-based, two backward steps that follow them
    (the gradient products the reference's autograd issues for configurations 2 and 3), and the
    attention of configuration 3 as one kernel."""
    return {
        1: dict(name="cfg1 fp32 _MatrixMul NN 4096x512 . 512x2048", dtype="f32", M=4096, N=2048, K=512, batch=1),
        2: dict(name="cfg2 fp32 MulAndShift X[32x128x512] . W[512x2048] + b[2048]", dtype="f32", M=4096, N=2048, K=512, batch=1),
        3: dict(name="cfg3 fp32 _MatrixMulBatched Q.K^T/8 then S.V, [256x128x64]", dtype="f32", M=128, N=128, K=64, batch=256),
        4: dict(name="cfg4 fp16 _MatrixMul TN a[1024x8192]^T . b[1024x4096]", dtype="f16", M=8192, N=4096, K=1024, batch=1),
        5: dict(name="cfg5 fp32 _MatrixMul NT H[4096x512] . W[30011x512]^T + C, beta=1", dtype="f32", M=4096, N=30011, K=512, batch=1),
        6: dict(name="cfg6 fp32 GradMulAndShift of cfg2: dX += dY.W^T (NT), dW += X^T.dY (TN) with db += colsum(dY)",
                dtype="f32", M=4096, N=2048, K=512, batch=1),
        7: dict(name="cfg7 fp32 GradMatrixMulBatched of cfg3 step 1: dQ += dS.K/8 (NN), dK += dS^T.Q/8 (TN), [256x128x128]",
                dtype="f32", M=128, N=128, K=64, batch=256),
        8: dict(name="cfg8 fp32 attention in one kernel: softmax(Q.K^T/8).V per head, q,k,v [32x128x512], 8 heads (cfg3 with the "
                     "softmax between its products and the head split/merge folded in)",
                dtype="f32", M=128, N=128, K=64, batch=256),
        10: dict(name="cfg10 fp32 Rectify(MulAndShift(X[32x128x512], W[512x2048], b[2048])) in one kernel (first step of the feed-forward block)",
                 dtype="f32", M=4096, N=2048, K=512, batch=1),
        11: dict(name="cfg11 fp32 attention probabilities in one kernel: softmax(Q.K^T/8) per head as [8x32x128x128] from q,k [32x128x512] "
                      "(cfg3's first product with the scale, the softmax and the head split folded in)",
                 dtype="f32", M=128, N=128, K=64, batch=256),
        12: dict(name="cfg12 fp32 attention context on merged tensors: Merge(BMMul(att[8x32x128x128], Split(v[32x128x512]))) as one "
                      "batched product that reads the heads of v and writes the merged result where they stand",
                 dtype="f32", M=128, N=64, K=128, batch=256),
        13: dict(name="cfg13 fp16 weight gradient of a 512x512 projection over 4096 positions: dW += X^T.dY (TN, beta=1), k cut into "
                      "pieces whose fp32 partial products a second kernel adds up",
                 dtype="f16", M=512, N=512, K=4096, batch=1),
        14: dict(name="cfg14 fp16 attention context whose probabilities are stored as float: BMMul(ConvertDataType(att[256x128x128], "
                      "half), v[256x128x64]) as one batched product that rounds the probabilities where it fetches them; "
                      "the library's conversion pass followed by the all-half product is timed beside it",
                 dtype="f16", M=128, N=64, K=128, batch=256),
        15: dict(name="cfg15 fp32 attention of the training path in one kernel: probabilities [8x32x128x128] written, multiplied "
                      "with a dropout mask and written again, context on merged tensors (cfg11, the caller's Multiply and cfg12 "
                      "in one launch)",
                 dtype="f32", M=128, N=128, K=64, batch=256),
        16: dict(name="cfg16 fp16 attention in one kernel at long sequences: softmax(Q.K^T/sqrt(128)).V per head, q,k,v half "
                      "[2x4096x1024], 8 heads of 128 (the steady state of the half kernel: 64 blocks of 64 keys per workgroup)",
                 dtype="f16", M=4096, N=4096, K=128, batch=16),
        9: dict(name="cfg9 fp16 attention in one kernel: softmax(Q.K^T/8).V per head, q,k,v half [32x128x512], 8 heads, "
                     "fp32 accumulation and softmax",
                dtype="f16", M=128, N=128, K=64, batch=256),
    }


class Workload:
    """Device buffers and the launch closure of one configuration."""

    def __init__(self, idx, dev, oracle):
        import torch
        import niutensor_amd as nt
        self.idx = idx
        self.dev = dev
        self.cfg = configs()[idx]
        T, NT = nt.X_TRANS, nt.X_NOTRANS
        g = lambda x: torch.from_numpy(x).to(dev)
        if idx in (1, 2, 10):
            self.x = g(oracle.uniform((4096, 512), 1))
            self.w = g(oracle.uniform((512, 2048), 2) if idx == 1 else oracle.normal((512, 2048), 2, 0, 0.02))
            self.b = g(oracle.normal((2048,), 3, 0, 0.02))
            self.c = torch.full((4096, 2048), float("nan"), device=dev)
            bias = self.b if idx != 1 else None
            act = nt.ACT_RECTIFY if idx == 10 else nt.ACT_NONE
            self.run = lambda: nt.matrix_mul(self.x, NT, self.w, NT, self.c, 1.0, 0.0, bias=bias, act=act)
            self.flops = 2.0 * 4096 * 2048 * 512
            self.bytes = 4.0 * (4096 * 512 + 512 * 2048 + 4096 * 2048) + (8192 if idx != 1 else 0)
            self.launches = 1
        elif idx == 3:
            self.q = g(oracle.normal((256, 128, 64), 1))
            self.k = g(oracle.normal((256, 128, 64), 2))
            self.v = g(oracle.normal((256, 128, 64), 3))
            self.s = torch.empty((256, 128, 128), device=dev)
            self.o = torch.empty((256, 128, 64), device=dev)

            def run():
                nt.matrix_mul_batched_strided(self.q, NT, self.k, T, self.s, 256, 8192, 8192, 16384,
                                              128, 64, 128, 64, 128, 128, 0.125, 0.0)
                nt.matrix_mul_batched_strided(self.s, NT, self.v, NT, self.o, 256, 16384, 8192, 8192,
                                              128, 128, 128, 64, 128, 64, 1.0, 0.0)
            self.run = run
            self.flops = 2 * 2.0 * 256 * 128 * 128 * 64
            self.bytes = 2 * 4.0 * 256 * (128 * 64 + 128 * 64 + 128 * 128)
            self.launches = 2
        elif idx == 4:
            # LAYOUT_OF_4 (--layout, for profiles of the other three layouts of the same product): the first letter
            # says how a is stored (T: k x m as in the baseline's configuration, N: m x k), the second how b is
            ta, tb = (T if LAYOUT_OF_4[0] == "T" else NT), (T if LAYOUT_OF_4[1] == "T" else NT)
            if LAYOUT_OF_4 != "TN":
                self.cfg = dict(self.cfg, name=self.cfg["name"] + " -- the same product with its operands stored " + LAYOUT_OF_4)
            self.a = g(oracle.normal((1024, 8192), 1, 0, 0.02)).half()
            self.b = g(oracle.normal((1024, 4096), 2, 0, 0.02)).half()
            if ta == NT:
                self.a = self.a.t().contiguous()
            if tb == T:
                self.b = self.b.t().contiguous()
            self.c = torch.empty((8192, 4096), device=dev, dtype=torch.float16)
            self.run = lambda: nt.matrix_mul(self.a, ta, self.b, tb, self.c, 1.0, 0.0)
            self.flops = 2.0 * 8192 * 4096 * 1024
            self.bytes = 2.0 * (1024 * 8192 + 1024 * 4096 + 8192 * 4096)
            self.launches = 1
        elif idx == 13:
            self.x = g(oracle.normal((4096, 512), 1)).half()
            self.dy = g(oracle.normal((4096, 512), 2, 0, 0.02)).half()
            self.dw = torch.zeros((512, 512), device=dev, dtype=torch.float16)
            self.run = lambda: nt.matrix_mul(self.x, T, self.dy, NT, self.dw, 1.0, 1.0)
            self.flops = 2.0 * 512 * 512 * 4096
            # x and dY read once, dW read and written; the partial products (workspace) are no part of the algorithm
            self.bytes = 2.0 * (2 * 4096 * 512 + 2 * 512 * 512)
            self.launches = 2
        elif idx == 5:
            self.h = g(oracle.uniform((4096, 512), 1))
            self.w = g(oracle.normal((30011, 512), 2, 0, 0.02))
            self.c = torch.rand((4096, 30011), device=dev) * 2 - 1
            self.run = lambda: nt.matrix_mul(self.h, NT, self.w, T, self.c, 1.0, 1.0)
            self.flops = 2.0 * 4096 * 30011 * 512
            self.bytes = 4.0 * (4096 * 512 + 30011 * 512 + 2 * 4096 * 30011)
            self.launches = 1
        elif idx == 6:
            self.x = g(oracle.uniform((4096, 512), 1))
            self.w = g(oracle.normal((512, 2048), 2, 0, 0.02))
            self.dy = g(oracle.normal((4096, 2048), 3))
            self.dx = torch.zeros((4096, 512), device=dev)
            self.dw = torch.zeros((512, 2048), device=dev)
            self.db = torch.zeros((2048,), device=dev)

            def run():
                nt.matrix_mul(self.dy, NT, self.w, T, self.dx, 1.0, 1.0)
                nt.matrix_mul_colsum(self.x, T, self.dy, NT, self.dw, self.db, 1.0, 1.0, 1.0)
            self.run = run
            self.flops = 2 * 2.0 * 4096 * 2048 * 512
            # dX: dY, W, dX read and written; dW: X, dY, dW read and written (db is 8 KB)
            self.bytes = 4.0 * ((4096 * 2048 + 512 * 2048 + 2 * 4096 * 512) + (4096 * 512 + 4096 * 2048 + 2 * 512 * 2048))
            self.launches = 2
        elif idx == 7:
            self.q = g(oracle.normal((256, 128, 64), 1))
            self.k = g(oracle.normal((256, 128, 64), 2))
            self.ds = g(oracle.normal((256, 128, 128), 3))
            self.dq = torch.zeros((256, 128, 64), device=dev)
            self.dk = torch.zeros((256, 128, 64), device=dev)

            def run():
                nt.matrix_mul_batched_strided(self.ds, NT, self.k, NT, self.dq, 256, 16384, 8192, 8192,
                                              128, 128, 128, 64, 128, 64, 0.125, 1.0)
                nt.matrix_mul_batched_strided(self.ds, T, self.q, NT, self.dk, 256, 16384, 8192, 8192,
                                              128, 128, 128, 64, 128, 64, 0.125, 1.0)
            self.run = run
            self.flops = 2 * 2.0 * 256 * 128 * 128 * 64
            self.bytes = 2 * 4.0 * 256 * (128 * 128 + 128 * 64 + 2 * 128 * 64)
            self.launches = 2
        elif idx in (8, 9):
            cast = (lambda t: t.half()) if idx == 9 else (lambda t: t)
            self.q = cast(g(oracle.normal((32, 128, 512), 1)))
            self.k = cast(g(oracle.normal((32, 128, 512), 2)))
            self.v = cast(g(oracle.normal((32, 128, 512), 3)))
            self.o = torch.empty((32, 128, 512), device=dev, dtype=self.q.dtype)
            self.run = lambda: nt.attention(self.q, self.k, self.v, self.o, 8, 0.125)
            self.flops = 2 * 2.0 * 256 * 128 * 128 * 64
            # q, k, v read once, the result written once; the scores never reach memory
            self.bytes = 4 * (4.0 if idx == 8 else 2.0) * 32 * 128 * 512
            self.launches = 1
        elif idx == 11:
            self.q = g(oracle.normal((32, 128, 512), 1))
            self.k = g(oracle.normal((32, 128, 512), 2))
            self.p = torch.empty((8, 32, 128, 128), device=dev)
            self.run = lambda: nt.attention_probs(self.q, self.k, self.p, 8, 0.125)
            self.flops = 2.0 * 256 * 128 * 128 * 64
            self.bytes = 4.0 * (2 * 32 * 128 * 512 + 256 * 128 * 128)
            self.launches = 1
        elif idx == 12:
            self.p = torch.softmax(g(oracle.normal((8, 32, 128, 128), 1)), -1)
            self.v = g(oracle.normal((32, 128, 512), 3))
            self.o = torch.empty((32, 128, 512), device=dev)
            self.run = lambda: nt.matrix_mul_batched_grid(self.p, NT, 128, (16384, 32 * 16384), self.v, NT, 512, (65536, 64),
                                                          self.o, 512, (65536, 64), 32, 8, 128, 128, 128, 64, 128, 64)
            self.flops = 2.0 * 256 * 128 * 128 * 64
            self.bytes = 4.0 * (256 * 128 * 128 + 2 * 32 * 128 * 512)
            self.launches = 1
        elif idx == 15:
            self.q = g(oracle.normal((32, 128, 512), 1))
            self.k = g(oracle.normal((32, 128, 512), 2))
            self.v = g(oracle.normal((32, 128, 512), 3))
            self.dm = (torch.rand((8, 32, 128, 128), device=dev) >= 0.1).float() / 0.9
            self.p = torch.empty((8, 32, 128, 128), device=dev)
            self.pd = torch.empty((8, 32, 128, 128), device=dev)
            self.o = torch.empty((32, 128, 512), device=dev)
            self.run = lambda: nt.attention_train(self.q, self.k, self.v, self.p, self.o, 8, 0.125, drop_mask=self.dm, dropped=self.pd)

            def three_steps():
                nt.attention_probs(self.q, self.k, self.p, 8, 0.125)
                torch.mul(self.p, self.dm, out=self.pd)          # stands in for the caller's Multiply
                nt.matrix_mul_batched_grid(self.pd, NT, 128, (16384, 32 * 16384), self.v, NT, 512, (65536, 64),
                                           self.o, 512, (65536, 64), 32, 8, 128, 128, 128, 64, 128, 64)
            self.other = ("ntsamd_attention_probs, an element-wise multiply with the dropout mask (torch.mul), "
                          "ntsamd_matrix_mul_batched_grid", three_steps)
            self.flops = 2 * 2.0 * 256 * 128 * 128 * 64
            # q, k, v read, the context written; the dropout mask read, probabilities and dropped probabilities written
            self.bytes = 4.0 * (4 * 32 * 128 * 512 + 3 * 256 * 128 * 128)
            self.launches = 1
        elif idx == 14:
            self.p = torch.softmax(g(oracle.normal((256, 128, 128), 1)), -1)
            self.ph = torch.empty((256, 128, 128), device=dev, dtype=torch.float16)
            self.v = g(oracle.normal((256, 128, 64), 3)).half()
            self.o = torch.empty((256, 128, 64), device=dev, dtype=torch.float16)
            shape = (256, 16384, 8192, 8192, 128, 128, 128, 64, 128, 64, 1.0, 0.0)
            self.run = lambda: nt.matrix_mul_batched_strided(self.p, NT, self.v, NT, self.o, *shape)

            def two_steps():
                nt.convert_data_type(self.p, self.ph)
                nt.matrix_mul_batched_strided(self.ph, NT, self.v, NT, self.o, *shape)
            self.other = ("ntsamd_convert_data_type of the probabilities, then the all-half batched product", two_steps)
            self.flops = 2.0 * 256 * 128 * 128 * 64
            self.bytes = 4.0 * 256 * 128 * 128 + 2.0 * 2 * 256 * 128 * 64
            self.launches = 1
        elif idx == 16:
            self.q = g(oracle.normal((2, 4096, 1024), 1)).half()
            self.k = g(oracle.normal((2, 4096, 1024), 2)).half()
            self.v = g(oracle.normal((2, 4096, 1024), 3)).half()
            self.o = torch.empty((2, 4096, 1024), device=dev, dtype=torch.float16)
            self.scale = 1.0 / math.sqrt(128.0)
            self.run = lambda: nt.attention(self.q, self.k, self.v, self.o, 8, self.scale)
            self.flops = 2 * 2.0 * 16 * 4096 * 4096 * 128
            self.bytes = 4 * 2.0 * 2 * 4096 * 1024
            self.launches = 1
        else:
            raise SystemExit("no such configuration: %d" % idx)

    def check(self):
        """The buffers the timed steps wrote against a float64 evaluation (torch, on the device: neither this
        library nor the oracle) of sampled rows, at least 64 of them, and every element of every result tested for
        being finite. Steps that accumulate (beta = 1) are checked on one more step from a fresh start of the same
        buffers. Returns max_err (norm-wise: max |got - ref| / max |ref|), the limit (1e-5 sqrt(K) in float, 1e-2 in
        half) and whether both tests passed."""
        import math
        import torch
        idx, dev = self.idx, self.dev
        gen = torch.Generator(device="cpu")
        gen.manual_seed(20251 + idx)
        pick = lambda n, k: torch.randperm(n, generator=gen)[:k].sort().values.to(dev)
        d = lambda t: t.double()
        half = self.cfg["dtype"] == "f16"
        limit = 1e-2 if half else 1e-5 * math.sqrt(self.cfg["K"])
        pairs, whole, rows = [], [], 0

        def heads(t, n=8):          # [b, l, n * dh] -> [n, b, l, dh]
            b, l, hd = t.shape
            return t.reshape(b, l, n, hd // n).permute(2, 0, 1, 3)

        def merged(t):              # [n, b, l, dh] -> [b, l, n * dh]
            n, b, l, dh = t.shape
            return t.permute(1, 2, 0, 3).reshape(b, l, n * dh)

        if idx in (1, 2, 10):
            r = pick(4096, 64)
            ref = d(self.x[r]) @ d(self.w)
            if idx != 1:
                ref = ref + d(self.b)
            if idx == 10:
                ref = ref.clamp(min=0)
            pairs, whole, rows = [(self.c[r], ref)], [self.c], 64
        elif idx == 3:
            r = pick(256, 8)
            sc = d(self.q[r]) @ d(self.k[r]).transpose(1, 2) * 0.125
            pairs, whole, rows = [(self.s[r], sc), (self.o[r], sc @ d(self.v[r]))], [self.s, self.o], 8 * 128
            limit = 1e-5 * math.sqrt(128)
        elif idx == 4:
            r = pick(8192, 64)
            a_rows = self.a[:, r].t() if LAYOUT_OF_4[0] == "T" else self.a[r]
            b_full = self.b.t() if LAYOUT_OF_4[1] == "T" else self.b
            pairs, whole, rows = [(self.c[r], d(a_rows) @ d(b_full))], [self.c], 64
        elif idx == 5:
            r = pick(4096, 64)
            self.c.uniform_(-1, 1)
            c0 = d(self.c[r])
            self.run()
            pairs, whole, rows = [(self.c[r], c0 + d(self.h[r]) @ d(self.w).t())], [self.c], 64
        elif idx == 6:
            r, rk = pick(4096, 64), pick(512, 64)
            for t in (self.dx, self.dw, self.db):
                t.zero_()
            self.run()
            pairs = [(self.dx[r], d(self.dy[r]) @ d(self.w).t()), (self.dw[rk], d(self.x[:, rk]).t() @ d(self.dy)),
                     (self.db, d(self.dy).sum(0))]
            whole, rows, limit = [self.dx, self.dw, self.db], 128, 1e-5 * math.sqrt(4096)
        elif idx == 7:
            r = pick(256, 8)
            self.dq.zero_()
            self.dk.zero_()
            self.run()
            pairs = [(self.dq[r], d(self.ds[r]) @ d(self.k[r]) * 0.125),
                     (self.dk[r], d(self.ds[r]).transpose(1, 2) @ d(self.q[r]) * 0.125)]
            whole, rows, limit = [self.dq, self.dk], 8 * 128, 1e-5 * math.sqrt(128)
        elif idx in (8, 9):
            r = pick(32, 2)
            q, k, v = (heads(d(t[r])) for t in (self.q, self.k, self.v))
            ref = merged(torch.softmax(q @ k.transpose(2, 3) * 0.125, -1) @ v)
            pairs, whole, rows = [(self.o[r], ref)], [self.o], 2 * 128
            limit = 1e-2 if half else 1e-5 * math.sqrt(64 + 128)
        elif idx == 11:
            r = pick(32, 2)
            q, k = heads(d(self.q[r])), heads(d(self.k[r]))
            pairs, whole, rows = [(self.p[:, r], torch.softmax(q @ k.transpose(2, 3) * 0.125, -1))], [self.p], 8 * 2 * 128
            limit = 1e-5 * math.sqrt(64 + 128)
        elif idx == 12:
            r = pick(32, 2)
            pairs, whole, rows = [(self.o[r], merged(d(self.p[:, r]) @ heads(d(self.v[r]))))], [self.o], 2 * 128
        elif idx == 15:
            r = pick(32, 2)
            q, k, v = (heads(d(t[r])) for t in (self.q, self.k, self.v))
            pr = torch.softmax(q @ k.transpose(2, 3) * 0.125, -1)
            dr = pr * d(self.dm[:, r])
            pairs = [(self.p[:, r], pr), (self.pd[:, r], dr), (self.o[r], merged(dr @ v))]
            whole, rows, limit = [self.p, self.pd, self.o], 8 * 2 * 128, 1e-5 * math.sqrt(64 + 128)
        elif idx == 13:
            rk = pick(512, 64)
            self.dw.zero_()
            self.run()
            pairs, whole, rows = [(self.dw[rk], d(self.x[:, rk]).t() @ d(self.dy))], [self.dw], 64
        elif idx == 14:
            r = pick(256, 8)
            pairs, whole, rows = [(self.o[r], d(self.p[r].half()) @ d(self.v[r]))], [self.o], 8 * 128
        elif idx == 16:
            rq = pick(4096, 64)
            q, k, v = (d(t[:1]).reshape(1, -1, 8, 128).transpose(1, 2) for t in (self.q[:, rq], self.k, self.v))
            ref = (torch.softmax(q @ k.transpose(2, 3) * self.scale, -1) @ v).transpose(1, 2).reshape(1, 64, 1024)
            pairs, whole, rows, limit = [(self.o[:1, rq], ref)], [self.o], 64, 1e-2
        err = max(float((d(got) - ref).abs().max() / ref.abs().max()) for got, ref in pairs)
        finite = all(bool(torch.isfinite(t).all()) for t in whole)
        ok = finite and err <= limit
        return {"max_err": float("%.3e" % err), "limit": float("%.3e" % limit), "sampled_rows": rows,
                "all_finite": finite, "ok": ok,
                "against": "float64 evaluation of the sampled rows (torch on the device), norm-wise: max|got - ref| / max|ref|"}

    def tensor_sets(self):
        """For kernel_us_rotated: enough copies of this configuration's device buffers that, used in turn, the sets
        add up to ROTATE_BYTES, more than the part's Infinity Cache holds (one set if one alone exceeds the cache).
        Returns the list of sets (name -> tensor) and the bytes of one set."""
        import torch
        own = {n: t for n, t in vars(self).items() if isinstance(t, torch.Tensor) and t.is_cuda}
        one = sum(t.numel() * t.element_size() for t in own.values())
        if one > CACHE_BYTES:
            return [own], one
        n = -(-ROTATE_BYTES // one)
        return [own] + [{k: t.clone() for k, t in own.items()} for _ in range(n - 1)], one

    def use(self, tensors):
        for name, t in tensors.items():
            setattr(self, name, t)


class HipEvents:
    """hipEvent timing on the stream the kernels are launched on."""

    def __init__(self):
        self.hip = C.CDLL("libamdhip64.so")
        self.hip.hipEventCreate.argtypes = [C.POINTER(C.c_void_p)]
        self.hip.hipEventRecord.argtypes = [C.c_void_p, C.c_void_p]
        self.hip.hipEventSynchronize.argtypes = [C.c_void_p]
        self.hip.hipEventElapsedTime.argtypes = [C.POINTER(C.c_float), C.c_void_p, C.c_void_p]
        self.e0, self.e1 = C.c_void_p(), C.c_void_p()
        assert self.hip.hipEventCreate(C.byref(self.e0)) == 0
        assert self.hip.hipEventCreate(C.byref(self.e1)) == 0

    def time(self, fn, stream, reps):
        assert self.hip.hipEventRecord(self.e0, stream) == 0
        for _ in range(reps):
            fn()
        assert self.hip.hipEventRecord(self.e1, stream) == 0
        assert self.hip.hipEventSynchronize(self.e1) == 0
        ms = C.c_float()
        assert self.hip.hipEventElapsedTime(C.byref(ms), self.e0, self.e1) == 0
        return ms.value * 1e-3 / reps


def cpu_baseline(idx, budget_s=12.0):
    """The CPU restatement of the reference's naive path, one thread (the reference's default:
    no parallel runner means one job), on a row sample of the same product sized for ~budget_s."""
    import numpy as np
    from oracle.binding import Oracle, Reference, X_NOTRANS, X_TRANS
    gen = Oracle(native=True)
    # the forward configurations in float run the REAL reference (its CPU sources compiled by oracle/Makefile into
    # oracle/_ref, which travels with the tree) when that library is there; the others (half: the reference has no
    # CPU half arithmetic; the gradient steps) and a tree without it run the restatement
    use_ref = idx in (1, 2, 3, 5, 8, 10, 11, 12, 15) and Reference.available()
    o = Reference() if use_ref else gen
    if use_ref:
        o.uniform, o.normal = gen.uniform, gen.normal
    kind = "reference" if use_ref else "port"
    if use_ref:
        why = "the reference's own CPU sources, compiled by oracle/Makefile into oracle/_ref (test infrastructure)"
    elif idx in (1, 2, 3, 5, 8, 10, 11, 12, 15):
        why = "oracle/_ref/libnts_ref.so is not in this tree: the C restatement of the reference's CPU path runs instead"
    else:
        why = "the reference has no CPU arithmetic for this step (half operands, or a gradient step): the C restatement on fp32 values"
    flags = "-O3" if use_ref else "-O3 -march=native"
    cfg = configs()[idx]
    M, N, K = cfg["M"], cfg["N"], cfg["K"]
    # measured rates of this path on the GPU box's host: ~0.4 GFLOP/s when an operand is walked by column
    # (NN, TN), ~5 GFLOP/s when both are walked along rows (NT)
    rate = {1: 0.42e9, 2: 0.42e9, 10: 0.42e9, 3: 6e9, 4: 0.43e9, 13: 0.43e9, 5: 2.3e9 if use_ref else 5e9, 6: 0.75e9, 7: 2e9, 8: 4e9, 9: 4e9, 11: 4e9, 12: 2e9, 14: 6e9, 15: 3e9, 16: 4e9}[idx]
    if idx == 3:
        nb = max(1, min(256, int(budget_s * rate / (4.0 * 128 * 128 * 64))))
        q, k, v = o.normal((nb, 128, 64), 1), o.normal((nb, 128, 64), 2), o.normal((nb, 128, 64), 3)
        t0 = time.perf_counter()
        s = o.matmul_batched(q, X_NOTRANS, k, X_TRANS, None, 0.125)
        o.matmul_batched(s, X_NOTRANS, v, X_NOTRANS)
        dt = time.perf_counter() - t0
        fl = nb * 4.0 * 128 * 128 * 64
        sample = "%d of 256 batch items, both products" % nb
    elif idx in (8, 9):
        nb = max(1, min(32, int(budget_s * rate / (8 * 4.0 * 128 * 128 * 64))))
        q, k, v = o.normal((nb, 128, 512), 1), o.normal((nb, 128, 512), 2), o.normal((nb, 128, 512), 3)
        if idx == 9:
            # fp32 arithmetic on the half-rounded values: the reference has no CPU half path
            q, k, v = (o.from_f16_bits(o.to_f16_bits(t)) for t in (q, k, v))
        t0 = time.perf_counter()
        o.attention(q, k, v, 8, 0.125)
        dt = time.perf_counter() - t0
        fl = nb * 8 * 4.0 * 128 * 128 * 64
        sample = "%d of 32 sentences, 8 heads each: split, scale, product, softmax, product, merge" % nb
    elif idx == 11:
        nb = max(1, min(32, int(budget_s * rate / (8 * 2.0 * 128 * 128 * 64))))
        q, k = o.normal((nb, 128, 512), 1), o.normal((nb, 128, 512), 2)
        t0 = time.perf_counter()
        o.attention_probs(q, k, 8, 0.125)
        dt = time.perf_counter() - t0
        fl = nb * 8 * 2.0 * 128 * 128 * 64
        sample = "%d of 32 sentences, 8 heads each: split, scale, product, softmax" % nb
    elif idx == 12:
        nb = max(1, min(32, int(budget_s * rate / (8 * 2.0 * 128 * 128 * 64))))
        p, v = o.uniform((8, nb, 128, 128), 1, 0.0, 1.0), o.normal((nb, 128, 512), 3)
        t0 = time.perf_counter()
        # Split and Merge as numpy copies (the reference's are copies too), the product through the library
        vs = np.ascontiguousarray(v.reshape(nb, 128, 8, 64).transpose(2, 0, 1, 3))
        c = o.matmul_batched(p, X_NOTRANS, vs, X_NOTRANS)
        np.ascontiguousarray(c.transpose(1, 2, 0, 3)).reshape(nb, 128, 512)
        dt = time.perf_counter() - t0
        fl = nb * 8 * 2.0 * 128 * 128 * 64
        sample = "%d of 32 sentences, 8 heads each: split of v, batched product, merge" % nb
    elif idx == 15:
        nb = max(1, min(32, int(budget_s * rate / (8 * 4.0 * 128 * 128 * 64))))
        q, k, v = o.normal((nb, 128, 512), 1), o.normal((nb, 128, 512), 2), o.normal((nb, 128, 512), 3)
        dm = np.where(o.uniform((8, nb, 128, 128), 4, 0.0, 1.0) < 0.1, 0.0, 1.0 / 0.9).astype(np.float32)
        t0 = time.perf_counter()
        # the reference's chain: probabilities, Dropout as its element-wise product with the mask, Split of v, BMMul, Merge
        dr = o.attention_probs(q, k, 8, 0.125) * dm
        vs = np.ascontiguousarray(v.reshape(nb, 128, 8, 64).transpose(2, 0, 1, 3))
        c = o.matmul_batched(dr, X_NOTRANS, vs, X_NOTRANS)
        np.ascontiguousarray(c.transpose(1, 2, 0, 3)).reshape(nb, 128, 512)
        dt = time.perf_counter() - t0
        fl = nb * 8 * 4.0 * 128 * 128 * 64
        sample = "%d of 32 sentences, 8 heads each: split, scale, product, softmax, dropout mask, product, merge" % nb
    elif idx == 16:
        rows = max(16, min(4096, int(budget_s * rate / (8 * 4.0 * 4096 * 128)) // 16 * 16))
        # fp32 arithmetic on the half-rounded values: the reference has no CPU half path
        q, k, v = (o.from_f16_bits(o.to_f16_bits(o.normal((1, n, 1024), seed))) for n, seed in ((rows, 1), (4096, 2), (4096, 3)))
        t0 = time.perf_counter()
        o.attention(q, k, v, 8, 1.0 / math.sqrt(128.0))
        dt = time.perf_counter() - t0
        fl = rows * 8 * 4.0 * 4096 * 128
        sample = "%d of 4096 query rows of one of the 2 sentences against all of its keys, 8 heads: split, scale, product, softmax, product, merge" % rows
    elif idx == 14:
        nb = max(1, min(256, int(budget_s * rate / (2.0 * 128 * 128 * 64))))
        p = o.uniform((nb, 128, 128), 1, 0.0, 1.0)
        v = o.from_f16_bits(o.to_f16_bits(o.normal((nb, 128, 64), 3)))
        t0 = time.perf_counter()
        # fp32 arithmetic on the half-rounded values: the reference has no CPU half product
        o.matmul_batched(o.from_f16_bits(o.convert(p, 3)), X_NOTRANS, v, X_NOTRANS)
        dt = time.perf_counter() - t0
        fl = nb * 2.0 * 128 * 128 * 64
        sample = "%d of 256 batch items: probabilities rounded to half, batched product" % nb
    elif idx == 7:
        nb = max(1, min(256, int(budget_s * rate / (4.0 * 128 * 128 * 64))))
        q, k, ds = o.normal((nb, 128, 64), 1), o.normal((nb, 128, 64), 2), o.normal((nb, 128, 128), 3)
        dq, dk = np.zeros_like(q), np.zeros_like(k)
        t0 = time.perf_counter()
        o.grad_matmul_batched(q, X_NOTRANS, k, X_TRANS, ds, 0.125, dq, dk)
        dt = time.perf_counter() - t0
        fl = nb * 4.0 * 128 * 128 * 64
        sample = "%d of 256 batch items, both gradient products" % nb
    elif idx == 6:
        rows = max(8, min(M, int(budget_s * rate / (4.0 * N * K))))
        x, w, dy = o.uniform((rows, K), 1), o.normal((K, N), 2, 0, 0.02), o.normal((rows, N), 3)
        dx, dw, db = np.zeros_like(x), np.zeros_like(w), np.zeros((N,), np.float32)
        t0 = time.perf_counter()
        o.grad_mulandshift(x, w, dy, 1, 1.0, dx, dw, db)
        dt = time.perf_counter() - t0
        fl = 4.0 * rows * N * K
        sample = "%d of %d rows of x and dE/dc, all of w: both gradient products and the bias sums" % (rows, M)
    else:
        rows = max(8, min(M, int(budget_s * rate / (2.0 * N * K))))
        if idx in (1, 2, 10):
            a, b = o.uniform((rows, K), 1), o.uniform((K, N), 2)
            bias = o.normal((N,), 3, 0, 0.02)
            t0 = time.perf_counter()
            if idx == 1:
                o.matmul2d(a, X_NOTRANS, b, X_NOTRANS)
            elif idx == 2:
                o.mulandshift(a.reshape(1, rows, K), b, bias)
            else:
                o.rectify(o.mulandshift(a.reshape(1, rows, K), b, bias)[0])
            dt = time.perf_counter() - t0
        elif idx in (4, 13):
            # fp32 arithmetic on the half-rounded values: the reference has no CPU half product
            a = o.from_f16_bits(o.to_f16_bits(o.normal((K, rows), 1, 0, 0.02)))
            b = o.from_f16_bits(o.to_f16_bits(o.normal((K, N), 2, 0, 0.02)))
            c = np.zeros((rows, N), np.float32)
            t0 = time.perf_counter()
            o.matmul2d(a, X_TRANS, b, X_NOTRANS, c, 1.0, 1.0 if idx == 13 else 0.0)
            dt = time.perf_counter() - t0
        else:
            a, b = o.uniform((rows, K), 1), o.normal((N, K), 2, 0, 0.02)
            c = o.uniform((rows, N), 3)
            t0 = time.perf_counter()
            o.matmul2d(a, X_NOTRANS, b, X_TRANS, c, 1.0, 1.0)
            dt = time.perf_counter() - t0
        fl = 2.0 * rows * N * K
        sample = "%d of %d result rows, all %d columns, K=%d" % (rows, M, N, K)
    return {"value": round(fl / dt / 1e12, 6), "unit": "TFLOP/s", "cores": 1, "kind": kind, "kind_why": why,
            "sample": sample + " (%.1f s; %.2f GFLOP/s, %s)" % (dt, fl / dt / 1e9, flags)}


def measured_traffic(idx):
    """HBM-side bytes per step from the committed rocprofv3 counter runs and what the library launched when they
    were read: the row of this configuration in profiles/hbm_traffic_per_step.md
    ("| configuration | bytes | algorithmic bytes | plans |"), or (None, None)."""
    import re
    try:
        with open(os.path.join(ROOT, "profiles", "hbm_traffic_per_step.md")) as f:
            for line in f:
                m = re.match(r"\|\s*(\d+)\s*\|\s*(\d+)\s*\|\s*\d+\s*\|\s*(.*?)\s*\|\s*$", line)
                if m and int(m.group(1)) == idx:
                    return int(m.group(2)), m.group(3)
    except OSError:
        pass
    return None, None


def graph_replayed(wl, dev, ev, steps_in_graph=50, replays=20):
    """Seconds per step when 50 steps are captured into one HIP graph and the graph is replayed."""
    import torch
    side = torch.cuda.Stream(dev)
    side.wait_stream(torch.cuda.current_stream(dev))
    with torch.cuda.stream(side):
        wl.run()
    torch.cuda.current_stream(dev).wait_stream(side)
    torch.cuda.synchronize()
    g = torch.cuda.CUDAGraph()
    with torch.cuda.graph(g):
        for _ in range(steps_in_graph):
            wl.run()
    for _ in range(5):
        g.replay()
    torch.cuda.synchronize()
    stream = torch.cuda.current_stream(dev).cuda_stream
    return ev.time(g.replay, stream, replays) / steps_in_graph


def k_scan(dev, ev):
    """Where the time of configuration 3's first product goes: the same 256 x (128 x 128) results with k from 8 to 512,
    a launch that does next to nothing, and a plain copy of the bytes the k = 64 product moves; each replayed from a
    HIP graph (microseconds per launch). The intercept of the scan is what a launch of this grid costs before its
    first MFMA and after its last; the slope is the matrix pipe."""
    import torch
    import niutensor_amd as nt
    T, NT = nt.X_TRANS, nt.X_NOTRANS

    class One:
        launches = 1

    def replayed(fn):
        w = One()
        w.run = fn
        return round(min(graph_replayed(w, dev, ev) for _ in range(3)) * 1e6, 2)

    out = {"scan": "256 x (128 x k) . (128 x k)^T, float, replayed from a HIP graph, us per launch", "k": {}}
    for k in (8, 32, 64, 96, 128, 192, 256, 512):
        q = torch.randn(256, 128, k, device=dev)
        kk = torch.randn(256, 128, k, device=dev)
        s = torch.empty(256, 128, 128, device=dev)
        out["k"][str(k)] = replayed(lambda: nt.matrix_mul_batched_strided(q, NT, kk, T, s, 256, 128 * k, 128 * k, 16384,
                                                                         128, k, 128, k, 128, 128, 0.125, 0.0))
    a = torch.zeros(64, device=dev)
    b = torch.zeros(64, device=dev, dtype=torch.float16)
    out["launch_of_one_workgroup_us"] = replayed(lambda: nt.convert_data_type(a, b))
    x = torch.empty(4 * 1024 * 1024, device=dev)
    y = torch.empty_like(x)
    out["copy_16MiB_read_16MiB_written_us"] = replayed(lambda: y.copy_(x))
    ks = [64, 96, 128, 192, 256, 512]
    ts = [out["k"][str(k)] for k in ks]
    n = len(ks)
    mk, mt = sum(ks) / n, sum(ts) / n
    slope = sum((k - mk) * (t - mt) for k, t in zip(ks, ts)) / sum((k - mk) ** 2 for k in ks)
    out["fit_k64_to_512"] = {"us_per_k": round(slope, 4), "intercept_us": round(mt - slope * mk, 2),
                             "matrix_pipe_alone_us_per_k": round(2.0 * 256 * 128 * 128 / (PEAK_TFLOPS["f32"] * 1e12) * 1e6, 4)}
    return out


def rotated(wl, dev, ev, stream, reps):
    """Seconds per step with the configuration's buffers changed from step to step: enough sets, used in turn, that
    no operand or result is still in the 256 MB Infinity Cache when its turn comes again. Steps of less than 20 us
    are replayed from a HIP graph that holds one step per set, so that changing the buffers costs the host nothing.
    Returns (seconds per step, number of sets, bytes of one set)."""
    import torch
    sets, one = wl.tensor_sets()
    own = sets[0]
    if len(sets) == 1:
        return None, 1, one

    def cycle():
        for t in sets:
            wl.use(t)
            wl.run()
    try:
        for _ in range(3):
            cycle()
        torch.cuda.synchronize()
        rounds = max(2, reps // len(sets))
        per = min(ev.time(cycle, stream, rounds) for _ in range(3)) / len(sets)
        if per / wl.launches < 20e-6:
            g = torch.cuda.CUDAGraph()
            with torch.cuda.graph(g):
                cycle()
            for _ in range(5):
                g.replay()
            torch.cuda.synchronize()
            st = torch.cuda.current_stream(dev).cuda_stream
            per = min(ev.time(g.replay, st, 20) for _ in range(3)) / len(sets)
            del g
    finally:
        wl.use(own)
    return per, len(sets), one


def nts_layer_times():
    """The operators of configurations 2 to 5 through the nts:: C++ layer: tests/cpp/build/nts_tests --bench as a child
    process (run before this process touches the GPU). Returns {config: line} or a reason why not."""
    import subprocess
    exe = os.path.join(ROOT, "tests", "cpp", "build", "nts_tests")
    if not os.path.exists(exe):
        return "tests/cpp/build/nts_tests has not been built"
    try:
        p = subprocess.run([exe, "--bench"], capture_output=True, text=True, timeout=180)
    except subprocess.TimeoutExpired:
        return "nts_tests --bench did not finish in 180 s"
    if p.returncode != 0:
        return "nts_tests --bench ended with code %d: %s" % (p.returncode, (p.stdout + p.stderr)[-300:])
    out = {}
    for line in p.stdout.splitlines():
        if line.startswith("{"):
            rec = json.loads(line)
            out[rec["config"]] = rec
    return out


def settle(wl, ev, stream):
    """Runs the workload until SETTLE_S seconds of GPU time have passed; returns the launches it took."""
    done, spent = 0, 0.0
    reps = 8
    while spent < SETTLE_S:
        spent += ev.time(wl.run, stream, reps) * reps
        done += reps
        reps = min(reps * 2, 512)
    return done


def bench_one(idx, steps, warmup, dev, oracle, with_cpu, cpu_budget_s=12.0, rotate=True):
    import torch
    import niutensor_amd as nt
    wl = Workload(idx, dev, oracle)
    cfg = wl.cfg
    ev = HipEvents()
    stream = torch.cuda.current_stream(dev).cuda_stream
    settled = settle(wl, ev, stream)
    for _ in range(warmup):
        wl.run()
    torch.cuda.synchronize()
    # the timed region: wall clock around it, and HIP events on the stream the launches go to inside it
    t0 = time.perf_counter()
    kt = ev.time(wl.run, stream, steps)
    torch.cuda.synchronize()
    wall = (time.perf_counter() - t0) / steps
    # what those steps left in the result buffers, against float64 on sampled rows
    checked = wl.check()
    torch.cuda.synchronize()
    nt.record_plans(True)
    wl.run()
    kernels = nt.record_plans(False)
    # shortest of five more groups of launches, reported beside the average (clock and power state move it by a few %)
    reps = max(10, min(200, steps))
    kt_best = min(ev.time(wl.run, stream, reps) for _ in range(5))
    kt_graph = graph_replayed(wl, dev, ev) if kt / wl.launches < 20e-6 else None
    kt_rot, rot_sets, set_bytes = rotated(wl, dev, ev, stream, reps) if rotate else (None, 0, 0)
    other = None
    if hasattr(wl, "other"):
        # the same result by the steps this configuration replaces, timed the same way (and replayed from a graph,
        # where the host's issue rate does not count)
        what, fn = wl.other
        for _ in range(warmup):
            fn()
        t_other = min(ev.time(fn, stream, reps) for _ in range(5))
        run, wl.run = wl.run, fn
        g_other = graph_replayed(wl, dev, ev)
        wl.run = run
        other = {"what": what, "us_best": round(t_other * 1e6, 2),
                 "us_graph_replay": None if g_other is None else round(g_other * 1e6, 2)}
    peak = PEAK_TFLOPS[cfg["dtype"]]
    achieved = wl.flops / kt / 1e12
    # Every configuration is held against the dense matrix peak of its data type: that is what the metric and its
    # targets are quoted in. The attention-shaped batches move only 16 flops per byte, so their HBM fraction is given
    # beside it.
    roof = {"bound": "mfma", "achieved": round(achieved, 3), "peak": peak, "unit": "TFLOP/s",
            "frac": round(achieved / peak, 4)}
    traffic, taken_with = measured_traffic(idx)
    source = None
    if traffic is not None:
        if kernels is not None and taken_with != " ; ".join(kernels):
            source = ("stale: the committed table's counters were read when the library launched [%s]; it now launches [%s]"
                      % (taken_with, " ; ".join(kernels)))
            traffic = None
        else:
            source = ("committed rocprofv3 FETCH_SIZE/WRITE_SIZE table (profiles/hbm_traffic_per_step.md), read with the "
                      "kernels this run launched, not measured in this run")
    roof.update({"traffic": traffic,
                 "traffic_source": source,
                 "kernel_us": round(kt / wl.launches * 1e6, 2),
                 "kernel_us_best": round(kt_best / wl.launches * 1e6, 2),
                 "hbm_frac": round(wl.bytes / kt / 1e12 / HBM_TBS, 4),
                 "hbm_floor_us": round(wl.bytes / (HBM_TBS * 1e12) * 1e6, 2)})
    if kt_graph is not None:
        # launches this short are issued by the host about as fast as the GPU runs them: the same launches
        # replayed from a HIP graph, for what the kernel itself takes (not used for value, achieved or frac)
        roof["kernel_us_graph_replay"] = round(kt_graph / wl.launches * 1e6, 2)
    if rotate:
        if kt_rot is None:
            roof["kernel_us_rotated"] = roof["kernel_us"]
            resident = "one set of buffers is %.0f MB, more than the %d MB Infinity Cache holds: every step reads HBM" % (
                set_bytes / 1e6, CACHE_BYTES >> 20)
        else:
            roof["kernel_us_rotated"] = round(kt_rot / wl.launches * 1e6, 2)
            resident = ("one set of buffers (%.0f MB) used again every step: resident in the %d MB Infinity Cache; "
                        "kernel_us_rotated cycles %d sets (%.0f MB)" % (set_bytes / 1e6, CACHE_BYTES >> 20, rot_sets,
                                                                       rot_sets * set_bytes / 1e6))
    else:
        resident = "one set of buffers used again every step (in the Infinity Cache where it fits its 256 MB)"
    out = {
        "metric": "TFLOP/s & % of dense matrix peak for MatrixMul/Batched (fp32, fp16), 1 GPU",
        "value": round(wl.flops / wall / 1e12, 3),
        "unit": "TFLOP/s",
        "n_gpus": 1,
        "steps": steps,
        "warmup": warmup,
        "ms_per_step": round(wall * 1e3, 5),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": cfg["dtype"],
        "data": "synthetic",
        "config": {"workload": cfg["name"], "M": cfg["M"], "N": cfg["N"], "K": cfg["K"], "batch": cfg["batch"],
                   "launches_per_step": wl.launches, "inputs": "device buffers, filled before the timed region; " + resident,
                   "flops_per_step": wl.flops,
                   "algorithmic_bytes_per_step": wl.bytes,
                   "settle": "%d untimed steps (%.2f s of GPU time) before the %d warm-up steps" % (settled, SETTLE_S, warmup)},
        "pct_of_peak": round(100.0 * wl.flops / wall / 1e12 / peak, 2),
        "roofline": roof,
        "check": checked,
        "kernels": kernels,
    }
    if other is not None:
        out["replaces"] = other
    if with_cpu:
        out["cpu_baseline"] = cpu_baseline(idx, cpu_budget_s)
    return out


def brief(line):
    """What the headline line keeps of another configuration's line."""
    keep = {"workload": line["config"]["workload"], "dtype": line["dtype"], "steps": line["steps"],
            "kernel_us": line["roofline"]["kernel_us"], "launches_per_step": line["config"]["launches_per_step"],
            "value": line["value"], "unit": line["unit"], "pct_of_peak": line["pct_of_peak"],
            "roofline": {k: line["roofline"][k] for k in ("bound", "achieved", "peak", "unit", "frac", "hbm_frac",
                                                          "traffic", "traffic_source")},
            "max_err": line["check"]["max_err"], "limit": line["check"]["limit"], "check_ok": line["check"]["ok"],
            "kernels": line["kernels"], "inputs": line["config"]["inputs"]}
    for k in ("kernel_us_best", "kernel_us_graph_replay", "kernel_us_rotated"):
        if k in line["roofline"]:
            keep[k] = line["roofline"][k]
    for k in ("cpu_baseline", "nts_layer_us", "nts_layer"):
        if k in line:
            keep[k] = line[k]
    return keep


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    # the clocks need tens of milliseconds of load to settle: a short warm-up times the ramp
    ap.add_argument("--steps", type=int, default=1000)
    ap.add_argument("--warmup", type=int, default=500)
    ap.add_argument("--config", type=int, default=2, help="configuration 1-16 (default 2, the MulAndShift linear layer; 6 and 7 are backward steps, 8 and 9 the one-kernel attention in float and half, 10 the linear layer with Rectify, 11 the attention probabilities, 12 the product of the probabilities with the merged values, 13 a half weight gradient cut along k, 14 the attention context with float probabilities and half values, 15 the attention of the training path in one kernel, 16 the half attention at 4096 positions and heads of 128)")
    ap.add_argument("--all", action="store_true", help="one line per configuration, then the headline line")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--no-rotate", action="store_true",
                    help="skip kernel_us_rotated (the same steps over enough sets of buffers to exceed the Infinity Cache)")
    ap.add_argument("--no-nts", action="store_true", help="skip the child process that times the nts:: C++ layer")
    ap.add_argument("--only", action="store_true",
                    help="time --config alone, without the other baseline configurations beside it (for a profiler: their "
                         "kernels share names with those of configurations 6, 7, 12 and 14)")
    ap.add_argument("--layout", choices=("TN", "TT", "NN", "NT"), default="TN",
                    help="configuration 4 with its operands stored another way (TN is the baseline's: a as k x m, b as k x n)")
    ap.add_argument("--k-scan", action="store_true",
                    help="run only the scan over k of configuration 3's first product (what a launch costs beside its MFMAs)")
    ap.add_argument("--copy-calibration", action="store_true",
                    help="run only a plain device copy of known size (scale for the FETCH_SIZE / WRITE_SIZE counters)")
    args = ap.parse_args()
    global LAYOUT_OF_4
    LAYOUT_OF_4 = args.layout
    if args.gpus != 1:
        raise SystemExit("bench.py measures one GPU: the path has no multi-GPU part (each product is independent); "
                         "run with --gpus 1")

    # the nts:: layer first, in a process of its own, before this one touches the GPU
    special = args.copy_calibration or args.k_scan
    nts_layer = None if (args.no_nts or args.only or special) else nts_layer_times()

    import torch
    import niutensor_amd as nt
    from oracle.binding import Oracle
    if not torch.cuda.is_available():
        raise SystemExit("bench.py needs a gfx950 GPU")
    nt.load()
    dev = torch.device("cuda:0")
    if args.copy_calibration:
        # 256 MiB read + 256 MiB written per copy: what a profiler's HBM counters should show
        src = torch.empty(64 * 1024 * 1024, dtype=torch.float32, device=dev).normal_()
        dst = torch.empty_like(src)
        for _ in range(args.steps):
            dst.copy_(src)
        torch.cuda.synchronize()
        print(json.dumps({"copy_bytes_read": src.numel() * 4, "copy_bytes_written": src.numel() * 4, "copies": args.steps}))
        return
    if args.k_scan:
        print(json.dumps(k_scan(dev, HipEvents())))
        return
    oracle = Oracle()
    with_cpu = not args.no_cpu
    rotate = not args.no_rotate and not args.only
    lines = {}
    if args.all:
        for idx in (1, 3, 4, 5, 6, 7, 8, 9, 10, 11, 12, 13, 14, 15, 16):
            if idx == args.config:
                continue
            steps = args.steps if idx != 5 else max(5, args.steps // 10)
            lines[idx] = bench_one(idx, steps, args.warmup if idx != 5 else max(3, args.warmup // 10), dev, oracle, with_cpu,
                                   rotate=rotate)
            print(json.dumps(lines[idx]), flush=True)
    head = bench_one(args.config, args.steps, args.warmup, dev, oracle, with_cpu, rotate=rotate)
    lines[args.config] = head
    # the other configurations of the baseline, each settled and timed like the headline (at least 50 steps, so that
    # a short headline run still gives them a steady reading; a tenth for the 1 ms product), CPU leg on a 3 s sample;
    # then configuration 3 in the forms the transformer really runs it in (one kernel; the two halves of training)
    for idx in BASELINE_CONFIGS + ATTENTION_FORMS if not args.only else ():
        if idx not in lines:
            steps = max(50, args.steps) if idx != 5 else max(20, args.steps // 10)
            lines[idx] = bench_one(idx, steps, args.warmup, dev, oracle, with_cpu, cpu_budget_s=3.0, rotate=rotate)
    # the same operators through the nts:: layer (microseconds per launch, a new result tensor per call)
    if isinstance(nts_layer, dict):
        for idx, rec in nts_layer.items():
            if idx in lines:
                lines[idx]["nts_layer_us"] = rec["us_per_call"]
                lines[idx]["nts_layer"] = rec
    elif nts_layer is not None:
        head["nts_layer_note"] = nts_layer
    if not args.only:
        head["configs"] = [brief(lines[idx]) for idx in BASELINE_CONFIGS]
        head["attention_forms"] = [brief(lines[idx]) for idx in ATTENTION_FORMS]
    print(json.dumps(head), flush=True)
    bad = [idx for idx, line in sorted(lines.items()) if not line["check"]["ok"]]
    if bad:
        sys.stderr.write("bench.py: the timed buffers of configuration(s) %s do not agree with float64 (see \"check\")\n" % bad)
        sys.exit(1)


if __name__ == "__main__":
    main()
