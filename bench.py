#!/usr/bin/env python3
"""Benchmark of the quantized-linear hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--only NAME] [--no-cpu] [--no-sweep]

Prints ONE JSON line.  Configs are numbered 1 .. 5: config n is BASELINE.json's configs[n - 1].  The headline workload is the largest single-GPU M = 1 configuration, config 5's
GEMV: e4m3 weights [11008, 4096] with a per-tensor scale under one e4m3 activation row, fp32 accumulate, bf16
out - 45 MB per launch, the size at which a fraction of the HBM roofline means something (config 2's 1.66 MB
layers are launch-bound by construction and stay a row of `results`).  A step is one launch.  Weights, inputs
and outputs are resident in HBM before the timed region; the step rotates through enough distinct copies of
the layer (>= 512 MB) that every call streams from HBM ("cold").  `value` is algorithmic GB/s: every operand
counted once (weights, scale, x, y), no scratch, no padding.

`results` carries every BASELINE config measured with the reference's protocol (warm-up, 7 samples of N calls
between two synchronisations, median sample / N; benchmarks/quant/bench_qlinear_smolvla.mojo:37-38,89-137), each
with its own roofline fraction.  The warm-up is 50 ms of replays (the matrix-core-bound calls need 30 - 40 ms
after an idle spell to reach their steady rate); the large matrix-core-bound rows also carry the figure taken
the reference's way, after ONE warm call (`us_per_call_one_warm_call`), so that a kernel's gain can be told from
the warm-up's.  `roofline` is the headline kernel, with `frac` from the HIP events of this run and
`frac_profiled` from the kernel's average duration in the committed rocprofv3 trace of the same loop (the
profiler brackets every dispatch, so its per-kernel time is the longer one); `roofline_m4096` is the metric's
other half (config 4, the batched-env actor at M = 4096, in TOPS); `roofline_mfma` the large-M fp8 GEMM (config
5) under both protocols, beside what the matrix cores alone sustain on the same GPU (`mfma_only`: back-to-back
MFMAs on register operands, constant and random data, both MFMA shapes).

`--only a16_shapes --a16-class C` re-derives the constants by which the library picks the tile shape of its
kernel for tens to hundreds of activation rows (a grid of calls timed under each shape, nq_diag_forward_a16);
`--only mid_dispatch --a16-class C` times the kernels that compete for those calls side by side and the library's
choice between them.

`cpu_baseline` times the CPU oracle's restatement of the reference's CPU
forward (a fresh dequantize to an fp32 scratch, then the serial triple loop;
noeira/nn/quant/qlinear.mojo:416-426, noeira/nn/core/cpu_gemm.mojo:88-98) on
one host core, on a bounded sample of the same workload.
"""
from __future__ import annotations

import argparse
import json
import os
import statistics
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

HBM_PEAK_GBPS = 8000.0          # MI355X HBM3E
MFMA_PEAK_TOPS = {"fp8": 5000.0, "int8": 5000.0, "bf16": 2500.0}
SAMPLES, COLD_BYTES = 7, 512 << 20
SETTLE_S = 0.05  # warm-up replays before the samples of a row (see median_per_call)
# HBM bytes per launch from rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE (fetched + written), scaled by
# what the same counters read for a plain copy of known size; None until measured
HEADLINE_TRAFFIC = 1804544      # config 2's pair: mean of the two linears' launches (1.66 MB algorithmic)
FP8_GEMV_TRAFFIC = 45199360     # K=4096, N=11008 (45.11 MB algorithmic)
FP8_GEMM_TRAFFIC = 269149440    # M=8192, K=4096, N=4096 (117.4 MB algorithmic; the re-reads hit the Infinity Cache)
# average kernel durations of the committed rocprofv3 kernel traces of the same loops (profiles/), nanoseconds: what
# `frac_profiled` is computed from.  The profiler brackets every dispatch, so these run longer than the un-profiled
# launches timed here; a reader can hold either against the other.
PROFILED_NS = {"fp8_gemv_11008": 8795.1, "fp8_gemm_4096": 100250.0, "actor_fused": 8006.7}


def ensure_built():
    from noeira_amd import _lib

    try:
        _lib.lib()
    except OSError:
        from noeira_amd import build as nq_build

        nq_build.build()
        _lib.lib()


def bf16_t(x):
    import numpy as np
    import torch

    return torch.from_numpy(np.ascontiguousarray(x, np.float32)).to(torch.bfloat16)


class Timer:
    """HIP events on torch's current stream (the stream every launch goes to)."""

    def __init__(self):
        import torch

        self.t = torch
        self.a = torch.cuda.Event(enable_timing=True)
        self.b = torch.cuda.Event(enable_timing=True)

    def run(self, fn, n):
        self.t.cuda.synchronize()
        self.a.record()
        for i in range(n):
            fn(i)
        self.b.record()
        self.t.cuda.synchronize()
        return self.a.elapsed_time(self.b) * 1e-3  # seconds


def capture(fn, n):
    """One HIP graph holding calls fn(0) .. fn(n-1).  The library only enqueues kernels on the
    stream it is given (no allocation, no synchronisation), so a forward is capturable as is; a
    replay then costs the GPU what the kernels cost, without the host's per-call overhead."""
    import torch

    fn(0)
    torch.cuda.synchronize()
    g = torch.cuda.CUDAGraph()
    with torch.cuda.graph(g):
        for i in range(n):
            fn(i)
    return g


def median_both(fn, calls):
    """(one warm call then the samples - the reference's own protocol -, the same after SETTLE_S of replays):
    seconds per call each.  The first is taken right after the workload was built, i.e. after an idle spell."""
    import torch

    tm = Timer()
    g = capture(fn, calls)  # (capture makes the one warm call)
    ref = statistics.median([tm.run(lambda i: g.replay(), 1) / calls for _ in range(SAMPLES)])
    t0 = time.perf_counter()
    while time.perf_counter() - t0 < SETTLE_S:
        g.replay()
        torch.cuda.synchronize()
    settled = statistics.median([tm.run(lambda i: g.replay(), 1) / calls for _ in range(SAMPLES)])
    return ref, settled


def median_per_call(fn, calls, graph=True):
    """The reference's protocol (warm up, SAMPLES samples of `calls` calls between two
    synchronisations, median sample / calls), with the calls of a sample replayed from a graph.
    The warm-up lasts SETTLE_S of replays, not one call: after an idle spell (the host building the next
    workload) the matrix-core-bound calls need 30 - 40 ms to reach their steady rate - config 5's GEMM runs at
    117, then 136, then 104 - 105 us per launch, where it stays - and a sample taken earlier times the power
    management's transient, not the kernel.  The memory-bound calls show no such transient."""
    import torch

    tm = Timer()
    if graph:
        g = capture(fn, calls)
        t0 = time.perf_counter()
        while True:
            g.replay()
            torch.cuda.synchronize()
            if time.perf_counter() - t0 >= SETTLE_S:
                break
        ts = [tm.run(lambda i: g.replay(), 1) / calls for _ in range(SAMPLES)]
    else:
        fn(0)
        ts = [tm.run(fn, calls) / calls for _ in range(SAMPLES)]
    return statistics.median(ts)


# ── workloads ───────────────────────────────────────────────────────────────
def make_act_w8a16(M, copies, seed=2):
    """config 2 (BASELINE.json configs[1]): two W8A16 linears, K=512->N=3200 and K=3200->N=512."""
    import numpy as np
    import torch

    from noeira_amd.qlinear import W8Linear

    rng = np.random.default_rng(seed)
    dims = [(512, 3200), (3200, 512)]
    sets = []
    for _ in range(copies):
        pair = []
        for K, N in dims:
            lin = W8Linear(K, N)
            lin.set_weight(rng.integers(-127, 128, (N, K), dtype=np.int8),
                           rng.uniform(1e-3, 1e-2, N).astype(np.float32))
            pair.append(lin)
        sets.append(pair)
    xs = [bf16_t(rng.standard_normal((M, K))).cuda() for K, _ in dims]
    bs = [bf16_t(rng.standard_normal(N) * 0.02).cuda() for _, N in dims]
    ys = [torch.empty((M, N), dtype=torch.float32, device="cuda") for _, N in dims]
    nbytes = sum(N * K + 4 * N + 2 * N + 2 * K * M + 4 * N * M for K, N in dims)
    ops = sum(2 * M * N * K for K, N in dims)

    def step(i):
        pair = sets[i % copies]
        pair[0].forward(xs[0], bias=bs[0], out=ys[0])
        pair[1].forward(xs[1], bias=bs[1], out=ys[1])

    return dict(step=step, bytes=nbytes, ops=ops, launches=2, keep=(sets, xs, bs, ys))


TILE_COPY = True  # --rows-layout: large layers keep the row-ordered codes only (the kernels before the tile copy)


def make_w8a16_one(K, N, copies, seed=9, M=1):
    """One W8A16 linear (int8 weights, per-channel scales, bf16 activations, fp32 out)."""
    import numpy as np
    import torch

    from noeira_amd.qlinear import W8Linear

    rng = np.random.default_rng(seed)
    w = rng.integers(-127, 128, (N, K), dtype=np.int8)
    s = rng.uniform(1e-3, 1e-2, N).astype(np.float32)
    layers = []
    for _ in range(copies):
        lin = W8Linear(K, N, tile_copy=TILE_COPY)
        lin.set_weight(w, s)
        layers.append(lin)
    x = bf16_t(rng.standard_normal((M, K))).cuda()
    y = torch.empty((M, N), dtype=torch.float32, device="cuda")

    def step(i):
        layers[i % copies].forward(x, out=y)

    return dict(step=step, bytes=N * K + 4 * N + 2 * K * M + 4 * N * M, ops=2 * M * N * K, launches=1,
                keep=(layers, x, y))


def make_q4_0(IN, OUT, M, copies, seed=3, bf16_x=False):
    """The reference's own layer: Q4_0 group 32, fp32 activations (bf16 with `bf16_x`: the activations of the
    reference's int4 tensor-core path, qlinear.mojo:430-463), fp32 out."""
    import numpy as np
    import torch

    from noeira_amd.qlinear import QLinear

    rng = np.random.default_rng(seed)
    nb = OUT * (IN // 32) * 18
    layers = []
    for _ in range(copies):
        blocks = rng.integers(0, 256, nb, dtype=np.uint8)
        sc = rng.uniform(1e-3, 2e-3, OUT * (IN // 32)).astype(np.float16).view(np.uint8).reshape(-1, 2)
        blocks.reshape(-1, 18)[:, 0:2] = sc
        ql = QLinear(IN, OUT, tile_copy=TILE_COPY)
        ql.set_blocks(blocks)
        layers.append(ql)
    x = torch.from_numpy(rng.standard_normal((M, IN)).astype(np.float32)).cuda()
    if bf16_x:
        x = x.to(torch.bfloat16)
    y = torch.empty((M, OUT), dtype=torch.float32, device="cuda")

    def step(i):
        layers[i % copies].forward(x, out=y)

    return dict(step=step, bytes=nb + (2 if bf16_x else 4) * IN * M + 4 * OUT * M, ops=2 * M * IN * OUT, launches=1,
                keep=(layers, x, y))


def make_decoder_layer(M, adapters, copies=1, seed=11):
    """The seven projections of one text layer of the reference's caller (960 wide, 320 k / v, 2560 MLP; Q4_0; fp32
    activations; noeira/deep_agents/smolvla/fused.mojo:287-363) in the caller's order, each on its own input buffer:
    `adapters` = "none": q|k|v fused, o, gate|up + SwiGLU fused, down - four launches;
    "fused": the same groups with a rank-16 adapter on all seven (layer_weights.mojo:713-739): nq_forward_fused_lora for
    q|k|v and for gate|up (SwiGLU applied to the sums; on the nq_fuse_glu layer in one launch at 17 .. 511 rows),
    nq_forward_lora for o and down;
    "per_projection": what the caller does today, seven `proj_fwd` = forward + forward_add, then SwiGLU left out."""
    import numpy as np
    import torch

    from noeira_amd.lora import LoRAAdapter
    from noeira_amd.qlinear import FusedGLU, FusedRows, QLinear

    rng = np.random.default_rng(seed)
    W, KV, FF = 960, 320, 2560

    def q4(IN, OUT):
        blocks = rng.integers(0, 256, OUT * (IN // 32) * 18, dtype=np.uint8)
        sc = rng.uniform(1e-3, 2e-3, OUT * (IN // 32)).astype(np.float16).view(np.uint8).reshape(-1, 2)
        blocks.reshape(-1, 18)[:, 0:2] = sc
        ql = QLinear.make(IN, OUT, "gpu")
        ql.set_blocks(blocks)
        return ql

    def ad(IN, OUT):
        a = LoRAAdapter(IN, OUT, 16, alpha=32.0)
        a.set_params(((rng.random((IN, 16)) * 2 - 1) / np.sqrt(IN)).astype(np.float32),
                     (rng.standard_normal((16, OUT)) * 0.05).astype(np.float32))
        return a

    shapes = [(W, W), (W, KV), (W, KV), (W, W), (W, FF), (W, FF), (FF, W)]  # q k v o gate up down
    lin = [q4(i, o) for (i, o) in shapes]
    ads = [ad(i, o) for (i, o) in shapes]
    qkv, glu, pair = FusedRows(lin[0:3]), FusedGLU(lin[4], lin[5]), FusedRows(lin[4:6])
    x = torch.from_numpy(rng.standard_normal((M, W)).astype(np.float32)).cuda()
    h = torch.from_numpy(rng.standard_normal((M, FF)).astype(np.float32)).cuda()
    yq = [torch.empty((M, n), device="cuda") for n in (W, KV, KV)]
    yo, yd = torch.empty((M, W), device="cuda"), torch.empty((M, W), device="cuda")
    gu = [torch.empty((M, FF), device="cuda") for _ in range(2)]
    yg = torch.empty((M, FF), device="cuda")

    if adapters == "none":
        def step(i):
            qkv.forward(x, outs=yq), lin[3].forward(x, out=yo), glu.forward(x, out=yg), lin[6].forward(h, out=yd)
        launches = 4
    elif adapters == "fused":
        # gate | up: the nq_fuse_glu layer adds both adapters ahead of SwiGLU in its one launch where its kernel takes
        # the rows (17 .. 511); elsewhere the row-fused pair, an adding launch and the activation
        glu_folds = 17 <= M <= 511

        def step(i):
            qkv.forward_lora(x, ads[0:3], outs=yq), ads[3].forward_with(lin[3], x, out=yo)
            if glu_folds:
                glu.forward_lora(x, ads[4], ads[5], out=yg)
            else:
                pair.forward_lora(x, ads[4:6], outs=gu, glu_out=yg)
            ads[6].forward_with(lin[6], h, out=yd)
        launches = 7 if glu_folds else 8
    else:
        outs = [yq[0], yq[1], yq[2], yo, gu[0], gu[1], yd]

        def step(i):
            for l, a_, y in zip(lin, ads, outs):
                xin = x if l.IN == W else h
                l.forward(xin, out=y), a_.forward_add(xin, y)
        launches = 14
    wbytes = sum(o * (i // 32) * 18 for (i, o) in shapes)
    return dict(step=step, bytes=wbytes + 4 * M * (2 * W + FF), ops=2 * M * sum(i * o for (i, o) in shapes), launches=launches,
                keep=(lin, ads, qkv, glu, pair, x, h, yq, yo, yd, gu, yg))


def make_q4_0_fused(IN, OUTS, M, copies, seed=7, bf16_x=False, glu=False, bf16_y=False):
    """The reference caller's q|k|v or gate|up projections as one row-fused launch; with `glu` the SwiGLU between
    gate | up and `down` (fused.mojo:337-353) runs in that launch's epilogue and one [M, H] tensor comes out."""
    import numpy as np
    import torch

    from noeira_amd.qlinear import FusedGLU, FusedRows, QLinear

    rng = np.random.default_rng(seed)
    fused = []
    for _ in range(copies):
        parts = []
        for OUT in OUTS:
            nb = OUT * (IN // 32) * 18
            blocks = rng.integers(0, 256, nb, dtype=np.uint8)
            sc = rng.uniform(1e-3, 2e-3, OUT * (IN // 32)).astype(np.float16).view(np.uint8).reshape(-1, 2)
            blocks.reshape(-1, 18)[:, 0:2] = sc
            ql = QLinear.make(IN, OUT, "gpu")
            ql.set_blocks(blocks)
            parts.append(ql)
        fused.append(FusedGLU(*parts) if glu else FusedRows(parts))  # the parts are copied; they are freed here
    x = torch.from_numpy(rng.standard_normal((M, IN)).astype(np.float32)).cuda()
    if bf16_x:
        x = x.to(torch.bfloat16)
    tot = sum(OUTS)
    ydt = torch.bfloat16 if bf16_y else torch.float32
    if glu:
        yg = torch.empty((M, OUTS[0]), dtype=ydt, device="cuda")
        ybytes = yg.element_size() * OUTS[0] * M

        def step(i):
            fused[i % copies].forward(x, out=yg)

        keep = (fused, x, yg)
    else:
        ys = [torch.empty((M, OUT), dtype=torch.float32, device="cuda") for OUT in OUTS]
        ybytes = 4 * tot * M

        def step(i):
            fused[i % copies].forward(x, outs=ys)

        keep = (fused, x, ys)
    return dict(step=step, bytes=tot * (IN // 32) * 18 + (2 if bf16_x else 4) * IN * M + ybytes, ops=2 * M * IN * tot,
                launches=1, keep=keep)


def make_w4g(K, N, M, copies, seed=4):
    """config 3 (configs[2]): asymmetric uint4, group 128, fp16 scales, bf16 activations."""
    import numpy as np
    import torch

    from noeira_amd import formats as F
    from noeira_amd.qlinear import W4GroupLinear

    rng = np.random.default_rng(seed)
    G = -(-K // 128)
    layers = []
    for _ in range(copies):
        codes = rng.integers(0, 256, (N, K // 2), dtype=np.uint8)
        sc = rng.uniform(1e-3, 1e-2, (N, G)).astype(np.float16)
        zps = F.pack_u4_pairs(rng.integers(0, 16, (N, G), dtype=np.uint8))
        lin = W4GroupLinear(K, N, 128, tile_copy=TILE_COPY)
        lin.set_weight(codes, sc, zps)
        layers.append(lin)
    x = bf16_t(rng.standard_normal((M, K))).cuda()
    y = torch.empty((M, N), dtype=torch.float32, device="cuda")

    def step(i):
        layers[i % copies].forward(x, out=y)

    nbytes = N * K // 2 + 2 * N * G + N * ((G + 1) // 2) + 2 * K * M + 4 * N * M
    return dict(step=step, bytes=nbytes, ops=2 * M * N * K, launches=1, keep=(layers, x, y))


def make_w8a32(seed=1):
    """config 1 (configs[0]): W8A32, M=1, K=N=256."""
    import numpy as np
    import torch

    from noeira_amd.qlinear import W8Linear

    rng = np.random.default_rng(seed)
    lin = W8Linear(256, 256)
    lin.set_weight(rng.integers(-127, 128, (256, 256), dtype=np.int8), rng.uniform(1e-3, 1e-2, 256).astype(np.float32))
    x = torch.from_numpy(rng.standard_normal((1, 256)).astype(np.float32)).cuda()
    b = torch.zeros(256, dtype=torch.float32, device="cuda")
    y = torch.empty((1, 256), dtype=torch.float32, device="cuda")
    return dict(step=lambda i: lin.forward(x, bias=b, out=y), bytes=68608, ops=2 * 256 * 256, launches=1,
                keep=(lin, x, b, y))


def make_actor_w8a8(M=4096, seed=5):
    """config 4 (configs[3]): 64 -> 256 -> 256 -> 8, per-token int8 activations, ReLU."""
    import numpy as np
    import torch

    from noeira_amd.qlinear import W8Linear, quantize_rows_i8

    rng = np.random.default_rng(seed)
    dims = [(64, 256), (256, 256), (256, 8)]
    lins, biases = [], []
    for K, N in dims:
        lin = W8Linear(K, N)
        lin.set_weight(rng.integers(-127, 128, (N, K), dtype=np.int8), rng.uniform(1e-3, 1e-2, N).astype(np.float32))
        lins.append(lin)
        biases.append(torch.from_numpy((rng.standard_normal(N) * 0.02).astype(np.float32)).cuda())
    x = torch.from_numpy(rng.standard_normal((M, 64)).astype(np.float32)).cuda()
    qs = [torch.empty((M, K), dtype=torch.int8, device="cuda") for K, _ in dims]
    ss = [torch.empty((M,), dtype=torch.float32, device="cuda") for _ in dims]
    hs = [torch.empty((M, N), dtype=torch.float32, device="cuda") for _, N in dims]

    def step(i):
        h = x
        for j, lin in enumerate(lins):
            quantize_rows_i8(h, qs[j], ss[j])
            h = lin.forward_a8(qs[j], ss[j], bias=biases[j], epilogue="relu" if j < 2 else "none", out=hs[j])

    ops = sum(2 * M * K * N for K, N in dims)
    nbytes = sum(K * N + 4 * N for K, N in dims) + 4 * M * 64 + 4 * M * 8
    return dict(step=step, bytes=nbytes, ops=ops, launches=6, keep=(lins, biases, x, qs, ss, hs))


def make_actor_fused(M=4096, seed=5):
    """config 4 (configs[3]) as ONE launch: nq_mlp3_w8a8_forward."""
    import numpy as np
    import torch

    from noeira_amd.qlinear import W8Linear, mlp3_w8a8_forward

    rng = np.random.default_rng(seed)
    dims = [(64, 256), (256, 256), (256, 8)]
    lins, biases = [], []
    for K, N in dims:
        lin = W8Linear(K, N)
        lin.set_weight(rng.integers(-127, 128, (N, K), dtype=np.int8), rng.uniform(1e-3, 1e-2, N).astype(np.float32))
        lins.append(lin)
        biases.append(torch.from_numpy((rng.standard_normal(N) * 0.02).astype(np.float32)).cuda())
    x = torch.from_numpy(rng.standard_normal((M, 64)).astype(np.float32)).cuda()
    y = torch.empty((M, 8), dtype=torch.float32, device="cuda")

    def step(i):
        mlp3_w8a8_forward(lins[0], lins[1], lins[2], x, biases[0], biases[1], biases[2], out=y)

    ops = sum(2 * M * K * N for K, N in dims)
    nbytes = sum(K * N + 4 * N + 4 * N for K, N in dims) + 4 * M * 64 + 4 * M * 8
    return dict(step=step, bytes=nbytes, ops=ops, launches=1, keep=(lins, biases, x, y))


def make_fp8(M, N, K=4096, copies=1, seed=6, a16=False):
    """config 5 (configs[4]): e4m3 x e4m3, per-tensor scales, fp32 accumulate, bf16 out.  With `a16` the same
    weight under bf16 activations (the codes decoded to bf16 on their way into the bf16 matrix cores)."""
    import numpy as np
    import torch

    from noeira_amd.qlinear import FP8Linear

    rng = np.random.default_rng(seed)
    g = torch.Generator().manual_seed(seed)
    layers = []
    for _ in range(copies):
        w = torch.randn((N, K), generator=g).clamp_(-448, 448).to(torch.float8_e4m3fn).view(torch.uint8).numpy()
        lin = FP8Linear(K, N)
        lin.set_weight(w, 1.0 / 16)
        layers.append(lin)
    a = torch.randn((M, K), generator=g).clamp_(-448, 448).to(torch.float8_e4m3fn).view(torch.uint8).cuda()
    sa = torch.tensor([1.0 / 16], dtype=torch.float32, device="cuda")
    y = torch.empty((M, N), dtype=torch.bfloat16, device="cuda")
    if a16:
        xb = torch.randn((M, K), generator=g).to(torch.bfloat16).cuda()

        def step16(i):
            layers[i % copies].forward_a16(xb, out=y, out_dtype=torch.bfloat16)

        return dict(step=step16, bytes=N * K + 2 * M * K + 2 * M * N, ops=2 * M * N * K, launches=1,
                    keep=(layers, xb, y))

    def step(i):
        layers[i % copies].forward(a, sa, out=y)

    return dict(step=step, bytes=N * K + M * K + 2 * M * N + 8, ops=2 * M * N * K, launches=1, keep=(layers, a, sa, y))


def make_w8a8_gemm(M, N, K=4096, seed=8):
    """The large-M W8A8 GEMM of the north star: int8 x int8 -> int32 on the matrix cores, per-token and
    per-channel scales and bias in the epilogue, bf16 out."""
    import numpy as np
    import torch

    from noeira_amd.qlinear import W8Linear

    rng = np.random.default_rng(seed)
    lin = W8Linear(K, N)
    lin.set_weight(rng.integers(-127, 128, (N, K), dtype=np.int8), rng.uniform(1e-3, 1e-2, N).astype(np.float32))
    xq = torch.from_numpy(rng.integers(-127, 128, (M, K), dtype=np.int8)).cuda()
    xs = torch.from_numpy(rng.uniform(1e-2, 2e-2, M).astype(np.float32)).cuda()
    bias = torch.from_numpy((rng.standard_normal(N) * 0.02).astype(np.float32)).cuda()
    y = torch.empty((M, N), dtype=torch.bfloat16, device="cuda")

    def step(i):
        lin.forward_a8(xq, xs, bias=bias, out=y, out_dtype=torch.bfloat16)

    return dict(step=step, bytes=N * K + M * K + 2 * M * N + 4 * (M + 2 * N), ops=2 * M * N * K, launches=1,
                keep=(lin, xq, xs, bias, y))


def make_w8a8_m1(K, N, copies, seed=10):
    """int8 x int8 for one row of activations: the W8A8 layer of a single environment."""
    import numpy as np
    import torch

    from noeira_amd.qlinear import W8Linear

    rng = np.random.default_rng(seed)
    w = rng.integers(-127, 128, (N, K), dtype=np.int8)
    s = rng.uniform(1e-3, 1e-2, N).astype(np.float32)
    layers = []
    for _ in range(copies):
        lin = W8Linear(K, N)
        lin.set_weight(w, s)
        layers.append(lin)
    xq = torch.from_numpy(rng.integers(-127, 128, (1, K), dtype=np.int8)).cuda()
    xs = torch.from_numpy(rng.uniform(1e-2, 2e-2, 1).astype(np.float32)).cuda()
    y = torch.empty((1, N), dtype=torch.float32, device="cuda")

    def step(i):
        layers[i % copies].forward_a8(xq, xs, out=y, out_dtype=torch.float32)

    return dict(step=step, bytes=N * K + K + 4 * N + 4 * N + 4, ops=2 * N * K, launches=1, keep=(layers, xq, xs, y))


def mfma_only(iters=4096, reps=5):
    """What the matrix cores alone sustain (nq_diag_mfma_rate: one workgroup per CU, one wavefront per SIMD, MFMAs
    back to back on register operands): constant operands against the e4m3 codes of N(0,1) values (int8: zeros
    against uniform codes).  On data that toggles the multipliers the clock drops (power limit)."""
    import ctypes as C

    import numpy as np
    import torch

    from noeira_amd import _lib as L

    lib = L.lib()
    g = torch.Generator().manual_seed(1)
    n = 1 << 20
    data = {
        ("fp8", "constant 1.0"): torch.full((n,), 0x38, dtype=torch.uint8, device="cuda"),
        ("fp8", "e4m3 of N(0,1)"): torch.randn((n,), generator=g).clamp_(-448, 448).to(torch.float8_e4m3fn).view(torch.uint8).cuda(),
        ("int8", "zeros"): torch.zeros((n,), dtype=torch.uint8, device="cuda"),
        ("int8", "uniform in [-127, 127]"): torch.randint(-127, 128, (n,), generator=g, dtype=torch.int8).view(torch.uint8).cuda(),
    }
    wgs = torch.cuda.get_device_properties(0).multi_processor_count
    stamps = torch.zeros((wgs, 2), dtype=torch.int64, device="cuda")
    stream = C.c_void_p(torch.cuda.current_stream().cuda_stream)
    out = []
    names = {0: "v_mfma_f32_32x32x64_f8f6f4", 1: "v_mfma_i32_32x32x32_i8", 2: "v_mfma_f32_16x16x128_f8f6f4 (the GEMM's)",
             3: "v_mfma_i32_16x16x64_i8 (the GEMM's)"}
    ops_per_iter = {0: 16 * 131072, 1: 16 * 65536, 2: 64 * 65536, 3: 64 * 32768}
    for (kind, what), d in data.items():
        for k in ((0, 2) if kind == "fp8" else (1, 3)):
            its = iters if k < 2 else iters // 2  # (the 16 x 16 kernels issue twice the operations per iteration)

            def go(_i=0):
                L.check(lib.nq_diag_mfma_rate(k, C.c_void_p(d.data_ptr()), d.numel(), its, wgs, C.c_void_p(stamps.data_ptr()), stream))

            t0 = time.perf_counter()
            while time.perf_counter() - t0 < 2 * SETTLE_S:  # (steady clocks: see median_per_call)
                go()
                torch.cuda.synchronize()
            sec = Timer().run(go, reps) / reps
            ops = wgs * 4 * its * ops_per_iter[k]
            st = stamps.cpu().numpy().astype(np.float64)
            out.append({"mfma": names[k], "operands": what, "TOPS": round(ops / sec / 1e12, 1),
                        "shader_clock_GHz": round(st[:, 0].mean() / (st[:, 1].mean() * 10.0), 3), "workgroups": wgs})
    return out


def gemm_timeline(N=4096, K=4096, M=8192, i8=False):
    """Where a config-5 GEMM call's time goes: every workgroup of the 256 x 256 tile kernel stamps the GPU's
    constant 100 MHz clock at entry, when its first K stage has landed, after its K loop and after its stores
    are acknowledged, and the shader clock's cycle counter at the second and third of them
    (nq_diag_gemm8_timeline).  Reported per round of workgroups (the hardware hands out the next tile as a CU
    frees up): medians in microseconds; the K loop also in cycles per stage with the clock that follows."""
    import ctypes as C

    import numpy as np
    import torch

    from noeira_amd import _lib as L

    if i8:
        wl = make_w8a8_gemm(M, N, K=K)
        lin, a, sa, _, y = wl["keep"]
        layers = [lin]
    else:
        wl = make_fp8(M, N, K=K)
        layers, a, sa, y = wl["keep"]
    for i in range(5):
        wl["step"](i)
    torch.cuda.synchronize()
    tiles = (M // 256) * ((N + 255) // 256)
    buf = torch.zeros((tiles, 6), dtype=torch.int64, device="cuda")
    null = C.c_void_p(0)
    t = None
    for _ in range(7):  # single launches differ by a few percent with the clock the chip happens to be at: the fastest
        t0 = time.perf_counter()
        while time.perf_counter() - t0 < 2 * SETTLE_S:  # the stamped launch follows a steady run (see median_per_call)
            for i in range(50):
                wl["step"](i)
            torch.cuda.synchronize()
        for i in range(20):
            wl["step"](i)
        L.check(L.lib().nq_diag_gemm8_timeline(layers[0]._h, C.c_void_p(a.data_ptr()), L.DT_I8 if i8 else L.DT_FP8_E4M3,
                                                C.c_void_p(sa.data_ptr()), C.c_void_p(y.data_ptr()), L.DT_BF16, M,
                                                C.c_void_p(buf.data_ptr()), tiles, null))
        raw = buf.cpu().numpy().astype(np.float64)
        ti = raw[:, :4] * 0.01  # ticks of 10 ns -> us
        ti -= ti[:, 0].min()
        if t is None or ti[:, 3].max() < t[:, 3].max():
            t, cyc = ti, raw[:, 5] - raw[:, 4]
    order = np.argsort(t[:, 0])
    cus = torch.cuda.get_device_properties(0).multi_processor_count
    rounds = []
    for r in range(0, tiles, cus):
        idx = order[r:r + cus]
        rounds.append({"workgroups": int(len(idx)),
                       "entry_us": [round(float(t[idx, 0].min()), 2), round(float(t[idx, 0].max()), 2)],
                       "first_stage_us": round(float(np.median(t[idx, 1] - t[idx, 0])), 2),
                       "k_loop_us": round(float(np.median(t[idx, 2] - t[idx, 1])), 2),
                       "epilogue_us": round(float(np.median(t[idx, 3] - t[idx, 2])), 2),
                       "end_us": [round(float(t[idx, 3].min()), 2), round(float(t[idx, 3].max()), 2)]})
    stages = K // 128
    ghz = cyc / np.maximum(t[:, 2] - t[:, 1], 1e-3) / 1e3
    return {"workload": f"{'int8' if i8 else 'fp8'} GEMM M={M} K={K} N={N}, bf16 out", "tiles": tiles, "kernel_us": round(float(t[:, 3].max()), 2),
            "stage_us": round(float(np.median(t[:, 2] - t[:, 1])) / stages, 4), "stages_per_tile": stages,
            "stage_cycles": round(float(np.median(cyc)) / stages, 1), "mfma_cycles_per_stage": 2048,
            "shader_clock_GHz": [round(float(np.median(ghz)), 3), round(float(ghz.min()), 3), round(float(ghz.max()), 3)],
            "epilogue_bytes_per_round": min(tiles, cus) * 256 * 256 * 2, "rounds": rounds}


def make_read(nbytes, copies):
    """The floor of a weight-streaming call: nq_diag_stream_read over `nbytes` (a kernel that only reads, with
    1 KiB loads), rotating over `copies` distinct regions so that every call streams from HBM."""
    import ctypes as C

    import torch

    from noeira_amd import _lib as L

    stride = (nbytes + 4095) // 4096 * 4096
    buf = torch.full((stride * copies,), 0x5A, dtype=torch.uint8, device="cuda")
    lib = L.lib()

    def step(i):
        L.check(lib.nq_diag_stream_read(C.c_void_p(buf.data_ptr() + (i % copies) * stride), nbytes,
                                        C.c_void_p(torch.cuda.current_stream().cuda_stream)))

    return dict(step=step, bytes=nbytes, ops=0, launches=1, keep=(buf,))


def report(name, wl, seconds, bound, peak_key=None, seconds_ref=None):
    gbps = wl["bytes"] / seconds / 1e9
    tops = wl["ops"] / seconds / 1e12
    r = {"workload": name, "us_per_call": round(seconds * 1e6, 3), "GBps": round(gbps, 2), "TOPS": round(tops, 4),
         "bound": bound}
    if bound == "hbm":
        r["frac_of_roofline"] = round(gbps / HBM_PEAK_GBPS, 4)
    else:
        r["frac_of_roofline"] = round(tops / MFMA_PEAK_TOPS[peak_key], 4)
    if seconds_ref is not None:  # the reference's protocol: samples right after one warm call
        r["us_per_call_one_warm_call"] = round(seconds_ref * 1e6, 3)
        r["frac_of_roofline_one_warm_call"] = round(wl["ops"] / seconds_ref / 1e12 / MFMA_PEAK_TOPS[peak_key], 4)
    return r


def sweep(skip_large=False):
    """Every BASELINE config, the reference's timing protocol."""
    import torch

    out = []

    def run(name, maker, bound, peak_key=None, calls=50, both=False, **kw):
        wl = maker(**kw)
        copies = kw.get("copies", 1)
        # a replay is timed from the host's launch of the graph: with fewer than ~60 calls in it that start-up
        # is a visible share of every call (45 MB GEMV: 8.9 us per call at 13 calls, 8.4 at 52), so a cold rotation
        # goes round its copies several times
        n = max(calls, copies)
        if copies > 1:
            n = copies * max(1, -(-60 // copies))
        if both:
            t_ref, t = median_both(wl["step"], n)
            out.append(report(name, wl, t, bound, peak_key, t_ref))
        else:
            t = median_per_call(wl["step"], n)
            out.append(report(name, wl, t, bound, peak_key))
        del wl
        torch.cuda.empty_cache()

    run("cfg1 W8A32 256->256 M=1 (warm)", make_w8a32, "hbm")
    c2 = -(-COLD_BYTES // (2 * 512 * 3200))
    run("cfg2 W8A16 ACT MLP pair M=1 (cold, two launches per call)", make_act_w8a16, "hbm", M=1, copies=c2, calls=c2)
    run("cfg2 W8A16 ACT MLP pair M=1 (warm: one copy, resident in L2 / Infinity Cache)", make_act_w8a16, "hbm", M=1, copies=1, calls=200)
    run("cfg2 W8A16 ACT MLP M=100 (warm)", make_act_w8a16, "hbm", M=100, copies=1)
    for (K, N) in [(960, 960), (960, 2560), (2560, 960)]:
        c = max(1, COLD_BYTES // (N * K // 2))
        run(f"cfg3 W4A16 g128 {K}->{N} M=1 (cold)", make_w4g, "hbm", K=K, N=N, M=1, copies=c, calls=c)
        run(f"cfg3 W4A16 g128 {K}->{N} M=256 (warm)", make_w4g, "mfma", "bf16", K=K, N=N, M=256, copies=1, calls=20)
    for (IN, OUT) in [(960, 960), (960, 320), (960, 2560), (2560, 960)]:
        c = max(1, COLD_BYTES // (OUT * IN * 9 // 16))
        run(f"ref Q4_0 g32 {IN}->{OUT} M=1 fp32 (cold)", make_q4_0, "hbm", IN=IN, OUT=OUT, M=1, copies=c, calls=c)
        run(f"ref Q4_0 g32 {IN}->{OUT} M=135 fp32 (warm)", make_q4_0, "mfma", "bf16", IN=IN, OUT=OUT, M=135,
            copies=1, calls=20)
        run(f"ref Q4_0 g32 {IN}->{OUT} M=135 bf16 x (warm)", make_q4_0, "mfma", "bf16", IN=IN, OUT=OUT, M=135,
            copies=1, calls=20, bf16_x=True)
    for (name, OUTS) in [("q|k|v 960->960|320|320", [960, 320, 320]), ("gate|up 960->2560|2560", [2560, 2560])]:
        c = max(1, COLD_BYTES // (sum(OUTS) * 960 * 9 // 16))
        run(f"ref Q4_0 {name} row-fused M=1 fp32 (cold)", make_q4_0_fused, "hbm", IN=960, OUTS=OUTS, M=1, copies=c,
            calls=c)
        run(f"ref Q4_0 {name} row-fused M=135 fp32 (warm)", make_q4_0_fused, "mfma", "bf16", IN=960, OUTS=OUTS,
            M=135, copies=1, calls=20)
        run(f"ref Q4_0 {name} row-fused M=135 bf16 x (warm)", make_q4_0_fused, "mfma", "bf16", IN=960, OUTS=OUTS,
            M=135, copies=1, calls=20, bf16_x=True)
    cg = max(1, COLD_BYTES // (5120 * 960 * 9 // 16))
    run("ref Q4_0 gate|up + SwiGLU 960->2560 one launch M=1 fp32 (cold)", make_q4_0_fused, "hbm", IN=960,
        OUTS=[2560, 2560], M=1, copies=cg, calls=cg, glu=True)
    run("ref Q4_0 gate|up + SwiGLU 960->2560 one launch M=135 fp32 (warm)", make_q4_0_fused, "mfma", "bf16", IN=960,
        OUTS=[2560, 2560], M=135, copies=1, calls=20, glu=True)
    run("ref Q4_0 gate|up + SwiGLU 960->2560 one launch M=135 bf16 in / bf16 out (warm)", make_q4_0_fused, "mfma",
        "bf16", IN=960, OUTS=[2560, 2560], M=135, copies=1, calls=20, glu=True, bf16_x=True, bf16_y=True)
    for M in (135, 1):
        run(f"ref text layer, 7 Q4_0 projections M={M}: q|k|v, o, gate|up+SwiGLU, down (4 launches, no adapters)",
            make_decoder_layer, "mfma", "bf16", M=M, adapters="none", calls=20)
        run(f"ref text layer M={M} + rank-16 adapters on all seven, fused calls ({7 if 17 <= M <= 511 else 8} launches)", make_decoder_layer, "mfma",
            "bf16", M=M, adapters="fused", calls=20)
        run(f"ref text layer M={M} + rank-16 adapters, per projection as the caller does (14 launches, SwiGLU not counted)",
            make_decoder_layer, "mfma", "bf16", M=M, adapters="per_projection", calls=20)
    run("cfg4 W8A8 actor 64->256->256->8 M=4096 (fused, 1 launch)", make_actor_fused, "mfma", "int8", calls=20)
    run("cfg4 W8A8 actor 64->256->256->8 M=4096 (unfused, 6 launches)", make_actor_w8a8, "mfma", "int8", calls=20)
    for N in (4096, 11008):
        c = max(1, COLD_BYTES // (N * 4096))
        run(f"cfg5 fp8 GEMV K=4096 N={N} M=1 (cold)", make_fp8, "hbm", M=1, N=N, copies=c, calls=max(c, 20))
        if not skip_large:
            run(f"cfg5 fp8 GEMM M=8192 K=4096 N={N}", make_fp8, "mfma", "fp8", M=8192, N=N, copies=1, calls=10, both=True)
    if not skip_large:
        run("W8A8 int8 GEMM M=8192 K=4096 N=4096 (scales + bias epilogue, bf16 out)", make_w8a8_gemm, "mfma", "int8",
            M=8192, N=4096, calls=10, both=True)
        # thousands of rows with 16-bit activations (prefill over a 4-bit or 8-bit weight)
        run("W4A16 g128 M=4096 K=4096 N=4096 (warm)", make_w4g, "mfma", "bf16", K=4096, N=4096, M=4096, copies=1, calls=10, both=True)
        run("ref Q4_0 g32 960->2560 M=4096 fp32 (warm)", make_q4_0, "mfma", "bf16", IN=960, OUT=2560, M=4096, copies=1,
            calls=10)
        c8 = max(1, COLD_BYTES // (4096 * 11008))
        run("W8A8 int8 GEMV K=4096 N=11008 M=1 (cold)", make_w8a8_m1, "hbm", K=4096, N=11008, copies=c8, calls=c8)
        # a few rows to several hundred: the 16-row tile kernel's range
        # (1024: the 128 x 128 tile GEMM's range; 2048: back on the 256 x 256 tiles)
        for M in (16, 64, 256, 512, 1024, 2048):
            run(f"W8A8 int8 M={M} K=4096 N=4096 (warm)", make_w8a8_gemm, "mfma", "int8", M=M, N=4096, calls=20)
            run(f"fp8 x fp8 M={M} K=4096 N=4096 (warm)", make_fp8, "mfma", "fp8", M=M, N=4096, copies=1, calls=20)
        # e4m3 weights under bf16 activations: the bf16 matrix-core kernels
        for M in (16, 256, 4096):
            run(f"fp8 W x bf16 A M={M} K=4096 N=4096 (warm)", make_fp8, "mfma", "bf16", M=M, N=4096, copies=1, calls=20,
                a16=True)
        # the dequant-GEMVs at a size where the HBM fraction means something (22 - 45 MB of codes)
        c = max(1, COLD_BYTES // (4096 * 11008 // 2))
        run("W4A16 g128 4096->11008 M=1 (cold)", make_w4g, "hbm", K=4096, N=11008, M=1, copies=c, calls=c)
        run("ref Q4_0 g32 4096->11008 M=1 fp32 (cold)", make_q4_0, "hbm", IN=4096, OUT=11008, M=1, copies=c, calls=c)
        run("W8A16 4096->11008 M=1 (cold)", make_w8a16_one, "hbm", K=4096, N=11008, copies=max(1, c // 2),
            calls=max(1, c // 2))
        # what a kernel that only reads those weights takes (launch + stream): the floor of the rows above
        run("floor: a launch alone (plain read of 1 KiB as a graph node)", make_read, "hbm", nbytes=1024, copies=1, calls=200)
        for mb, nb in (("1.66 MB", 512 * 3200 + 4 * 3200), ("16.8 MB", 4096 * 4096),
                       ("23.2 MB", 4096 * 11008 // 2 + 2 * 32 * 11008 + 16 * 11008), ("45.1 MB", 4096 * 11008),
                       ("235 MB", 8192 * 28672)):
            cr = max(1, COLD_BYTES // nb)
            run(f"floor: plain read of {mb}, no arithmetic (cold)", make_read, "hbm", nbytes=nb, copies=cr, calls=cr)
        # the same kernels where the stream is long enough for the fixed part of a call (launch, first trip to
        # memory, the last wavefronts) to vanish: 8192 -> 28672, 235 MB of 8-bit codes / 117 - 132 MB of 4-bit ones
        KB, NB = 8192, 28672
        run(f"fp8 x fp8 GEMV {KB}->{NB} M=1 (cold, 235 MB)", make_fp8, "hbm", M=1, N=NB, K=KB, copies=3)
        run(f"W8A8 int8 GEMV {KB}->{NB} M=1 (cold, 235 MB)", make_w8a8_m1, "hbm", K=KB, N=NB, copies=3)
        run(f"W8A16 {KB}->{NB} M=1 (cold, 235 MB)", make_w8a16_one, "hbm", K=KB, N=NB, copies=3)
        run(f"W4A16 g128 {KB}->{NB} M=1 (cold, 122 MB)", make_w4g, "hbm", K=KB, N=NB, M=1, copies=5)
        run(f"ref Q4_0 g32 {KB}->{NB} M=1 fp32 (cold, 132 MB)", make_q4_0, "hbm", IN=KB, OUT=NB, M=1, copies=4)
        run("W4A16 g128 4096->11008 M=16 (cold)", make_w4g, "hbm", K=4096, N=11008, M=16, copies=c, calls=c)
        run("ref Q4_0 g32 4096->11008 M=16 fp32 (cold)", make_q4_0, "hbm", IN=4096, OUT=11008, M=16, copies=c, calls=c)
        run("W8A16 4096->11008 M=16 (cold)", make_w8a16_one, "hbm", K=4096, N=11008, M=16, copies=max(1, c // 2),
            calls=max(1, c // 2))
    return out


def vendor_gemm():
    """A yardstick, not a product path: the vendor library's fp8 GEMM (torch._scaled_mm -> hipBLASLt) on config 5's
    shapes, timed the way the GEMM rows are (50 ms of the same launches first, then medians of 20 launches)."""
    import torch

    out = []
    g = torch.Generator().manual_seed(6)
    for (M, N, K) in ((8192, 4096, 4096), (8192, 11008, 4096), (8192, 8192, 8192)):
        a = torch.randn((M, K), generator=g).clamp_(-448, 448).to(torch.float8_e4m3fn).cuda()
        w = torch.randn((N, K), generator=g).clamp_(-448, 448).to(torch.float8_e4m3fn).cuda()
        sa, sb = torch.tensor(1.0 / 16, device="cuda"), torch.tensor(1.0 / 16, device="cuda")

        def f(i):
            torch._scaled_mm(a, w.t(), scale_a=sa, scale_b=sb, out_dtype=torch.bfloat16)

        try:
            f(0)
            torch.cuda.synchronize()
        except Exception as e:  # (a torch build without the call: say so, measure nothing)
            out.append({"M": M, "N": N, "K": K, "error": repr(e)[:200]})
            continue
        tm = Timer()
        t0 = time.perf_counter()
        while time.perf_counter() - t0 < SETTLE_S:
            tm.run(f, 20)
        t = statistics.median([tm.run(f, 20) / 20 for _ in range(SAMPLES)])
        out.append({"M": M, "N": N, "K": K, "us_per_call": round(t * 1e6, 2),
                    "frac_of_fp8_peak": round(2.0 * M * N * K / t / 1e12 / MFMA_PEAK_TOPS["fp8"], 4)})
        del a, w
        torch.cuda.empty_cache()
    return out


def only_loop(which, steps, warmup):
    """One kernel, launched call by call `steps` times after `warmup` untimed calls: the loop a
    rocprofv3 run (kernel trace or one counter pass) is wrapped around."""
    import torch

    tm = Timer()
    if which == "copy":
        n = 256 << 20
        src = torch.full((n,), 7, dtype=torch.uint8, device="cuda")
        dst = torch.empty_like(src)
        wl = dict(step=lambda i: dst.copy_(src), bytes=2 * n, ops=0, keep=(src, dst))
        name = "plain device copy, 256 MiB read + 256 MiB written"
    elif which == "act":
        c = -(-COLD_BYTES // (2 * 512 * 3200))
        wl = make_act_w8a16(1, c)
        name = f"cfg2 W8A16 ACT MLP pair M=1, cold rotation over {c} copies of the two layers"
    elif which == "fp8gemv":
        N = 11008
        c = max(1, COLD_BYTES // (N * 4096))
        wl = make_fp8(1, N, copies=c)
        name = f"cfg5 fp8 GEMV K=4096 N={N} M=1, cold rotation over {c} weight copies"
    elif which == "mid":
        wls = [make_act_w8a16(100, 1)]
        wls += [make_w4g(K, N, 256, 1) for (K, N) in [(960, 960), (960, 2560), (2560, 960)]]
        wls += [make_q4_0(K, N, 135, 1) for (K, N) in [(960, 960), (960, 320), (960, 2560), (2560, 960)]]

        def step_all(i):
            for w in wls:
                w["step"](i)

        wl = dict(step=step_all, bytes=sum(w["bytes"] for w in wls), ops=sum(w["ops"] for w in wls), keep=wls)
        name = "configs 1 (M=100), 2 (M=256) and the reference's Q4_0 shapes at T=135, one call each per step"
    elif which == "biggemv":
        K, N = 4096, 11008
        c = max(1, COLD_BYTES // (N * K // 2))
        wls = [make_w4g(K=K, N=N, M=1, copies=c), make_q4_0(IN=K, OUT=N, M=1, copies=c),
               make_w8a16_one(K=K, N=N, copies=max(1, c // 2))]

        def step_big(i):
            for w in wls:
                w["step"](i)

        wl = dict(step=step_big, bytes=sum(w["bytes"] for w in wls), ops=sum(w["ops"] for w in wls), keep=wls)
        name = "W4A16 g128, Q4_0 (fp32 x) and W8A16 at 4096->11008, M=1, cold rotation, one call each per step"
    elif which == "hugegemv":
        K, N = 8192, 28672
        wls = [make_w4g(K=K, N=N, M=1, copies=5), make_q4_0(IN=K, OUT=N, M=1, copies=4)]

        def step_huge(i):
            for w in wls:
                w["step"](i)

        wl = dict(step=step_huge, bytes=sum(w["bytes"] for w in wls), ops=sum(w["ops"] for w in wls), keep=wls)
        name = "W4A16 g128 and Q4_0 (fp32 x) at 8192->28672 (122 / 132 MB), M=1, cold rotation, one call each per step"
    elif which == "smallm":
        K, N, M = 4096, 11008, 16
        c = max(1, COLD_BYTES // (N * K // 2))
        wls = [make_w4g(K=K, N=N, M=M, copies=c), make_q4_0(IN=K, OUT=N, M=M, copies=c),
               make_w8a16_one(K=K, N=N, M=M, copies=max(1, c // 2))]

        def step_small(i):
            for w in wls:
                w["step"](i)

        wl = dict(step=step_small, bytes=sum(w["bytes"] for w in wls), ops=sum(w["ops"] for w in wls), keep=wls)
        name = "W4A16 g128, Q4_0 (fp32 x) and W8A16 at 4096->11008, M=16, cold rotation, one call each per step"
    elif which == "manyrows":
        wls = [make_w4g(K=4096, N=4096, M=4096, copies=1), make_w8a16_one(K=4096, N=4096, M=4096, copies=1),
               make_q4_0(IN=960, OUT=2560, M=4096, copies=1), make_q4_0(IN=960, OUT=2560, M=1120, copies=1)]

        def step_mr(i):
            for w in wls:
                w["step"](i)

        wl = dict(step=step_mr, bytes=sum(w["bytes"] for w in wls), ops=sum(w["ops"] for w in wls), keep=wls)
        name = ("W4A16 g128 and W8A16 at 4096 x 4096, M = 4096; Q4_0 (fp32 x) 960->2560 at M = 4096 and 1120; "
                "one call each per step")
    elif which == "tile8":
        wls = [make_w8a8_gemm(M, 4096) for M in (16, 64, 128, 256, 512)] + [make_fp8(M, 4096) for M in (16, 64, 128, 256, 512)]

        def step_t8(i):
            for w in wls:
                w["step"](i)

        wl = dict(step=step_t8, bytes=sum(w["bytes"] for w in wls), ops=sum(w["ops"] for w in wls), keep=wls)
        name = "W8A8 and fp8 x fp8 at 4096 x 4096, M = 16, 64, 128, 256, 512, one call each per step"
    elif which == "gemm_mid":
        wls = [make_fp8(M, 4096) for M in (512, 1024)] + [make_w8a8_gemm(M, 4096) for M in (512, 1024)]

        def step_gm(i):
            for w in wls:
                w["step"](i)

        wl = dict(step=step_gm, bytes=sum(w["bytes"] for w in wls), ops=sum(w["ops"] for w in wls), keep=wls)
        name = "fp8 x fp8 and W8A8 at 4096 x 4096, M = 512 and 1024 (the 128 x 128 tile GEMM), one call each per step"
    elif which == "i8gemm":
        wl = make_w8a8_gemm(8192, 4096)
        name = "W8A8 int8 GEMM M=8192 K=4096 N=4096, scales + bias, bf16 out (the 256 x 256 tile on eight wavefronts)"
    elif which == "fp8gemm_n11008":
        wl = make_fp8(8192, 11008)
        name = "cfg5 fp8 GEMM M=8192 K=4096 N=11008 (five rounds of 256 x 256 tiles, then the 96 left over as 192 tiles of 128 x 256)"
    elif which == "gemm_half":
        wls = [make_fp8(2048, 4096), make_w8a8_gemm(2048, 4096)]

        def step_gh(i):
            for w in wls:
                w["step"](i)

        wl = dict(step=step_gh, bytes=sum(w["bytes"] for w in wls), ops=sum(w["ops"] for w in wls), keep=wls)
        name = "fp8 x fp8 and W8A8 at M=2048 over 4096 x 4096 (128 x 256 tiles), one call each per step"
    elif which == "adapters":
        wl = make_decoder_layer(135, "fused")
        name = "the reference text layer's seven Q4_0 projections at T = 135 with rank-16 adapters, fused calls"
    elif which == "gemm_timeline":
        return {"only": which, "timelines": [gemm_timeline(4096, 4096), gemm_timeline(4096, 8192), gemm_timeline(11008, 4096),
                                            gemm_timeline(4096, 4096, 2048), gemm_timeline(4096, 4096, i8=True)]}
    elif which == "mfma_peak":
        return {"only": which, "mfma_only": mfma_only()}
    elif which == "vendor_gemm":
        return {"only": which, "vendor_fp8_gemm": vendor_gemm()}
    elif which == "actor":
        wl = make_actor_fused()
        name = "cfg4 W8A8 actor 64->256->256->8 M=4096, fused"
    else:
        N = 4096
        wl = make_fp8(8192, N)
        name = f"cfg5 fp8 GEMM M=8192 K=4096 N={N}"
    for i in range(warmup):
        wl["step"](i)
    sec = tm.run(wl["step"], steps) / steps
    return {"only": which, "workload": name, "steps": steps, "us_per_call_eager": round(sec * 1e6, 3),
            "algorithmic_bytes_per_call": wl["bytes"], "ops_per_call": wl["ops"]}


def cpu_baseline(budget_s=12.0):
    """The oracle's restatement of the reference's CPU forward, one core, on the headline workload (config 5's GEMV:
    e4m3 weights [11008, 4096] under one e4m3 row) for about `budget_s` seconds: a fresh dequantize of the weight to
    an fp32 [OUT, IN] scratch, then the serial triple loop."""
    import numpy as np
    import torch

    from oracle import oracle as O

    rng = np.random.default_rng(2)
    K, N = 4096, 11008
    g = torch.Generator().manual_seed(6)
    w = torch.randn((N, K), generator=g).clamp_(-448, 448).to(torch.float8_e4m3fn).view(torch.uint8).numpy()
    x = torch.randn((1, K), generator=g).clamp_(-448, 448).to(torch.float8_e4m3fn).view(torch.uint8).numpy()
    nbytes = N * K + K + 2 * N + 8
    O.fp8_qlinear_forward_cpu(w, 1.0 / 16, x, 1.0 / 16)
    n, t0 = 0, time.perf_counter()
    while True:
        O.fp8_qlinear_forward_cpu(w, 1.0 / 16, x, 1.0 / 16)
        n += 1
        dt = time.perf_counter() - t0
        if dt >= budget_s and n >= 3:
            break
    # the reference's own layer on its own shapes (Q4_0, fp32 x), same CPU path, a few calls each
    q4 = []
    for (IN, OUT) in [(960, 960), (960, 320), (960, 2560), (2560, 960)]:
        blocks = rng.integers(0, 256, OUT * (IN // 32) * 18, dtype=np.uint8)
        sc = rng.uniform(1e-3, 2e-3, OUT * (IN // 32)).astype(np.float16).view(np.uint8).reshape(-1, 2)
        blocks.reshape(-1, 18)[:, 0:2] = sc
        for M, calls in ((1, 5), (135, 1)):
            x = rng.standard_normal((M, IN)).astype(np.float32)
            O.qlinear_forward_cpu(blocks, IN, OUT, x)
            t1 = time.perf_counter()
            for _ in range(calls):
                O.qlinear_forward_cpu(blocks, IN, OUT, x)
            q4.append({"layer": f"Q4_0 {IN}->{OUT}", "M": M, "ms_per_call": round((time.perf_counter() - t1) / calls * 1e3, 3)})
    return {"value": round(nbytes * n / dt / 1e9, 4), "unit": "GB/s", "cores": 1, "kind": "port",
            "ms_per_step": round(dt / n * 1e3, 3), "q4_0_reference_shapes": q4,
            "sample": f"{n} steps of the headline workload (e4m3 [11008, 4096] under one e4m3 row): a fresh dequantize to "
                      f"an fp32 [OUT, IN] scratch then the serial triple loop, single thread, {dt:.1f} s"}


def a16_shapes(cls="w4g"):
    """Times a grid of medium-M calls of one weight format / activation type under each of the 16-row tile kernel's
    five tile shapes (`nq_diag_forward_a16`) and under the library's own choice, and re-derives the constants of
    the estimate the library chooses by: t = F + ceil(workgroups / 256) * (p0 + p1 * k-steps) microseconds per
    shape, by least squares on relative errors.  Reports the constants, the fit's mean error, what always taking
    the shape of least estimate costs against always taking the fastest, and the same for the library's choice."""
    import ctypes as C

    import numpy as np
    import torch

    from noeira_amd import _lib as L
    from noeira_amd import formats as F
    from noeira_amd.qlinear import QLinear, W4GroupLinear, W8Linear

    xf32, kind = cls.endswith("f"), cls.rstrip("f")
    kstep = 64 if kind == "w8" else 128
    rng = np.random.default_rng(1)
    shapes = [(2, 4), (2, 2), (1, 4), (1, 2), (1, 1)]
    rows = []
    for K in ((512, 2048, 4096) if kind == "w8" else (960, 2048, 4096)):
        for N in (512, 2048, 4096):
            if kind == "q4":
                lin = QLinear(K, N, tile_copy=False)
                blocks = rng.integers(0, 256, (N, K // 32, 18), dtype=np.uint8)
                sc = rng.uniform(1e-3, 1e-2, (N, K // 32)).astype(np.float16).view(np.uint16)
                blocks[:, :, 0], blocks[:, :, 1] = sc & 0xFF, sc >> 8
                lin.set_blocks(blocks.reshape(-1))
            elif kind == "w4g":
                G = -(-K // 128)
                codes, zps = F.pack_w4g(rng.integers(0, 16, (N, K), dtype=np.uint8), rng.integers(0, 16, (N, G), dtype=np.uint8))
                lin = W4GroupLinear(K, N, 128, tile_copy=False)
                lin.set_weight(codes, rng.uniform(1e-3, 1e-2, (N, G)).astype(np.float16), zps)
            else:
                lin = W8Linear(K, N, tile_copy=False)
                lin.set_weight(rng.integers(-127, 128, (N, K), dtype=np.int8), rng.uniform(1e-3, 1e-2, N).astype(np.float32))
            for M in (17, 64, 100, 135, 256, 384, 500):
                x = torch.from_numpy(rng.standard_normal((M, K)).astype(np.float32)).cuda()
                x = x if xf32 else x.to(torch.bfloat16)
                y = torch.empty((M, N), dtype=torch.float32, device="cuda")
                step = lambda i: lin.forward(x, out=y)
                median_per_call(step, 20)  # (clocks up before the first timed shape)
                xc = L.DT_F32 if xf32 else L.DT_BF16
                ts = []
                for mw, nw in shapes + [(0, 0)]:
                    def shaped(i, mw=mw, nw=nw):
                        L.check(L.lib().nq_diag_forward_a16(lin._h, C.c_void_p(x.data_ptr()), xc, C.c_void_p(y.data_ptr()), L.DT_F32, M,
                                                             mw, nw, C.c_void_p(torch.cuda.current_stream().cuda_stream)))
                    fn = step if (mw, nw) == (0, 0) else shaped
                    ts.append(float("nan") if (xf32 and mw * nw == 8) else median_per_call(fn, 20) * 1e6)
                rows.append((K, N, M, ts))

    def feats(K, N, M, mw, nw):
        mt = (M + 15) // 16
        wgs = ((mt + mw - 1) // mw) * ((N + 16 * nw - 1) // (16 * nw))
        return -(-wgs // 256), (K + kstep - 1) // kstep

    consts, errs = {}, {}
    for si, (mw, nw) in enumerate(shapes):
        A, t = [], []
        for K, N, M, ts in rows:
            if ts[si] == ts[si]:
                R, ns = feats(K, N, M, mw, nw)
                A.append([1.0, R, R * ns])
                t.append(ts[si])
        if not A:
            continue
        A, t = np.array(A), np.array(t)
        c = np.linalg.lstsq(A / t[:, None], np.ones(len(t)), rcond=None)[0]
        consts[(mw, nw)] = c
        errs[(mw, nw)] = float(np.mean(np.abs(A @ c - t) / t))
    by_estimate = fastest = library = 0.0
    for K, N, M, ts in rows:
        est = {}
        for si, sh in enumerate(shapes):
            if sh in consts and not (sh[0] == 2 and M <= 16):
                R, ns = feats(K, N, M, *sh)
                est[si] = consts[sh][0] + R * (consts[sh][1] + consts[sh][2] * ns)
        by_estimate += ts[min(est, key=est.get)]
        fastest += min(v for v in ts[:5] if v == v)
        library += ts[5]
    return {"only": "a16_shapes", "class": cls, "calls": len(rows),
            "constants_F_p0_p1": {f"{mw}x{nw}": [round(float(v), 4) for v in c] for (mw, nw), c in consts.items()},
            "fit_mean_rel_err": {f"{mw}x{nw}": round(e, 4) for (mw, nw), e in errs.items()},
            "least_estimate_vs_fastest": round(by_estimate / fastest, 4),
            "library_choice_vs_fastest": round(library / fastest, 4)}



def mid_dispatch(cls="w4g"):
    """Which kernel takes a call of tens to hundreds of rows over a 4-bit layer, checked from outside: a grid of
    calls timed on a layer made with NQ_FLAG_PREFER_TILE (the M-tile kernel wherever the shape allows it), on one
    made without the tile-ordered copy (the 16-row tile kernel, or the many-rows kernel from 256 rows) and on a
    plain one (the library's choice between them).  Reports the library's total against always taking the faster
    of the two, and the calls where it is more than a tenth slower."""
    import numpy as np
    import torch

    from noeira_amd import formats as F
    from noeira_amd.qlinear import QLinear, W4GroupLinear

    xf32, kind = cls.endswith("f"), cls.rstrip("f")
    rng = np.random.default_rng(1)

    def layer(K, N, **kw):
        if kind == "q4":
            lin = QLinear(K, N, **kw)
            blocks = rng.integers(0, 256, (N, K // 32, 18), dtype=np.uint8)
            sc = rng.uniform(1e-3, 1e-2, (N, K // 32)).astype(np.float16).view(np.uint16)
            blocks[:, :, 0], blocks[:, :, 1] = sc & 0xFF, sc >> 8
            lin.set_blocks(blocks.reshape(-1))
            return lin
        G = -(-K // 128)
        codes, zps = F.pack_w4g(rng.integers(0, 16, (N, K), dtype=np.uint8), rng.integers(0, 16, (N, G), dtype=np.uint8))
        lin = W4GroupLinear(K, N, 128, **kw)
        lin.set_weight(codes, rng.uniform(1e-3, 1e-2, (N, G)).astype(np.float16), zps)
        return lin

    rows, slow = [], []
    for K in ((960, 2048) if xf32 else (960, 2048, 4096)):
        for N in (2560, 5120, 11008):
            ls = [layer(K, N, prefer_tile=True), layer(K, N, tile_copy=False), layer(K, N)]
            for M in (33, 100, 135, 256, 384, 511):
                x = torch.from_numpy(rng.standard_normal((M, K)).astype(np.float32)).cuda()
                x = x if xf32 else x.to(torch.bfloat16)
                y = torch.empty((M, N), dtype=torch.float32, device="cuda")
                ts = [median_per_call((lambda l: (lambda i: l.forward(x, out=y)))(l), 20) * 1e6 for l in ls]
                rows.append(ts)
                if ts[2] > 1.1 * min(ts[:2]):
                    slow.append({"K": K, "N": N, "M": M, "m_tile_us": round(ts[0], 2), "other_us": round(ts[1], 2),
                                 "library_us": round(ts[2], 2)})
            del ls
    lib, best = sum(t[2] for t in rows), sum(min(t[:2]) for t in rows)
    return {"only": "mid_dispatch", "class": cls, "calls": len(rows), "library_vs_faster_kernel": round(lib / best, 4),
            "always_m_tile_vs_faster": round(sum(t[0] for t in rows) / best, 4),
            "never_m_tile_vs_faster": round(sum(t[1] for t in rows) / best, 4), "more_than_a_tenth_slower": slow}



def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=2000)
    ap.add_argument("--warmup", type=int, default=200)
    ap.add_argument("--only", default="", choices=["", "headline", "act", "fp8gemv", "fp8gemm", "mid", "actor", "copy", "biggemv", "smallm", "tile8", "gemm_mid", "i8gemm", "fp8gemm_n11008", "gemm_half", "adapters", "manyrows", "hugegemv", "mfma_peak", "vendor_gemm", "gemm_timeline", "a16_shapes", "mid_dispatch"],
                    help="run one loop only and print a short JSON line (for rocprofv3 runs): headline = the "
                         "headline line alone (graph replays), act = config 2's pair of linears at M=1, fp8gemv / fp8gemm = "
                         "config 5 at N=11008 (the headline's kernel, launched call by call) / N=4096, mid = the M=100..256 "
                         "calls of configs 1, 2 and the reference's T=135 shapes, actor = config 3 fused, "
                         "copy = a plain 256 MiB device copy (the counter calibration kernel), biggemv / smallm = the "
                         "three 4096->11008 layers with 16-bit or fp32 activations at M=1 / M=16, hugegemv = the two 4-bit layers at 8192->28672, M=1, tile8 = int8 and fp8 "
                         "activations at M = 16 .. 512 over 4096 x 4096, manyrows = bf16 / fp32 activations at M = 1120 "
                         "and 4096, mfma_peak = the matrix cores alone (nq_diag_mfma_rate) on constant and random operands, gemm_timeline = the "
                         "config-5 GEMM's workgroups stamping entry / first stage / K loop / stores (nq_diag_gemm8_timeline), i8gemm / fp8gemm_n11008 / "
                         "gemm_half = the int8 GEMM 8192 x 4096 x 4096, config 5's GEMM at N = 11008, the two at M = 2048 over 4096 x 4096")
    ap.add_argument("--eager", action="store_true", help="with --only: launch call by call, no HIP graph")
    ap.add_argument("--rows-layout", action="store_true",
                    help="large layers keep only their row-ordered codes (NQ_FLAG_NO_TILE_COPY): the single-row kernels "
                         "that read them, for a before / after comparison with the tile-ordered copy")
    ap.add_argument("--a16-class", default="w4g", choices=["w8", "w8f", "q4", "q4f", "w4g", "w4gf"],
                    help="with --only a16_shapes: int8 codes, Q4_0 or groups of 128 with zero points; f: fp32 activations")
    ap.add_argument("--no-cpu", action="store_true")
    ap.add_argument("--no-sweep", action="store_true")
    a = ap.parse_args()
    if a.gpus != 1:
        print(f"bench.py: this build runs on one GPU; --gpus {a.gpus} is not supported "
              "(one layer's forward needs no second device).", file=sys.stderr)
        sys.exit(2)
    import torch

    ensure_built()
    assert torch.cuda.is_available(), "bench.py needs a GPU"
    torch.cuda.set_device(0)
    if a.rows_layout:
        global TILE_COPY
        TILE_COPY = False
    if a.only == "a16_shapes":
        print(json.dumps(a16_shapes(a.a16_class)))
        return
    if a.only == "mid_dispatch":
        if a.a16_class.startswith("w8"):
            sys.exit("bench.py: --only mid_dispatch is about the 4-bit formats (--a16-class q4, q4f, w4g or w4gf)")
        print(json.dumps(mid_dispatch(a.a16_class)))
        return
    if a.only in ("act", "fp8gemv", "fp8gemm", "mid", "actor", "copy", "biggemv", "smallm", "tile8", "gemm_mid", "i8gemm", "fp8gemm_n11008", "gemm_half", "adapters", "manyrows", "hugegemv", "mfma_peak", "vendor_gemm", "gemm_timeline"):
        print(json.dumps(only_loop(a.only, a.steps, a.warmup)))
        return

    # ---- headline: config 5's GEMV, e4m3 x e4m3, K = 4096, N = 11008, M = 1, every call from HBM
    K_H, N_H = 4096, 11008
    copies = max(1, -(-COLD_BYTES // (N_H * K_H)))
    wl = make_fp8(1, N_H, K=K_H, copies=copies)
    tm = Timer()
    for i in range(a.warmup):
        wl["step"](i)
    # The timed region is EXACTLY a.steps steps.  They are replayed from a HIP graph holding g consecutive steps
    # of the rotation (g = the largest divisor of steps that is <= 200: a replay is timed from the host's launch of
    # the graph, and in a graph of a dozen calls that start-up is a visible share of every call), a.steps / g
    # replays back to back, bracketed by synchronisations.  The events sit on the stream the kernels run on.
    g_steps = max(d for d in range(1, min(a.steps, 200) + 1) if a.steps % d == 0)
    if a.only and a.eager:
        sec = tm.run(wl["step"], a.steps)
    else:
        graph = capture(wl["step"], g_steps)
        graph.replay()
        sec = tm.run(lambda i: graph.replay(), a.steps // g_steps)
    ms_per_step = sec / a.steps * 1e3
    launch_s = sec / a.steps
    value = wl["bytes"] / launch_s / 1e9
    eager_sec = tm.run(wl["step"], a.steps)
    prof = PROFILED_NS["fp8_gemv_11008"]

    line = {
        "metric": "qlinear GB/s at M=1 and TOPS at M=4096, as % of MI355X roofline",
        "value": round(value, 2), "unit": "GB/s", "n_gpus": 1, "steps": a.steps, "warmup": a.warmup,
        "ms_per_step": round(ms_per_step, 6), "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "f32", "data": "synthetic",
        "config": {"workload": "BASELINE config 5 (configs[4]) at M=1, the largest single-GPU M=1 configuration: fp8 e4m3 "
                               f"weights [{N_H}, {K_H}] with a per-tensor fp32 scale under one e4m3 activation row, fp32 "
                               f"accumulate, bf16 out; cold: rotating over {copies} distinct weight copies "
                               f"({copies * N_H * K_H >> 20} MiB); launched as HIP-graph replays of {g_steps} steps",
                   "arithmetic": "e4m3 x e4m3 products on the fp8 matrix cores, fp32 sums",
                   "algorithmic_bytes_per_step": wl["bytes"], "launches_per_step": 1},
        "pct_of_hbm_roofline": round(100 * value / HBM_PEAK_GBPS, 3),
        "eager": {"GBps": round(wl["bytes"] * a.steps / eager_sec / 1e9, 2),
                  "us_per_step": round(eager_sec / a.steps * 1e6, 3),
                  "note": "the same steps launched one by one from Python through ctypes (host-bound)"},
        "roofline": {"bound": "hbm", "achieved": round(value, 2), "peak": HBM_PEAK_GBPS, "unit": "GB/s",
                     "frac": round(value / HBM_PEAK_GBPS, 5), "traffic": FP8_GEMV_TRAFFIC,
                     "kernel": "nq::gemv8_row_kernel<fp8>", "avg_launch_us": round(launch_s * 1e6, 3),
                     "frac_profiled": round(wl["bytes"] / (prof * 1e-9) / 1e9 / HBM_PEAK_GBPS, 5) if prof else None,
                     "profiled_avg_kernel_ns": prof,
                     "note": "frac: algorithmic bytes / this run's launch time (HIP events around graph replays); "
                             "frac_profiled: the same bytes / the kernel's average duration in the committed rocprofv3 "
                             "kernel trace of `bench.py --only fp8gemv` (launched call by call under the profiler, which "
                             "brackets every dispatch)"},
    }
    del wl
    torch.cuda.empty_cache()
    if a.only:
        print(json.dumps(line))
        return
    # the metric's other half: config 4 at M = 4096 (one fused launch), in TOPS against the int8 peak.  It is a
    # 0.69 GOP call: 0.14 us of matrix-core time at peak, so what bounds it is the launch and the chain of three layers.
    actor = make_actor_fused()
    actor_s = median_per_call(actor["step"], 20)
    actor_tops = actor["ops"] / actor_s / 1e12
    line["roofline_m4096"] = {"workload": "BASELINE config 4 (configs[3]): W8A8 actor 64->256->256->8, M=4096, one fused launch",
                              "kernel": "nq::mlp3_w8a8_kernel", "us_per_call": round(actor_s * 1e6, 3),
                              "bound": "mfma", "achieved": round(actor_tops, 3), "peak": MFMA_PEAK_TOPS["int8"],
                              "unit": "TOP/s", "frac": round(actor_tops / MFMA_PEAK_TOPS["int8"], 5),
                              "frac_profiled": round(actor["ops"] / (PROFILED_NS["actor_fused"] * 1e-9) / 1e12 / MFMA_PEAK_TOPS["int8"], 5),
                              "profiled_avg_kernel_ns": PROFILED_NS["actor_fused"],
                              "note": "launch- and latency-bound by construction (see results for the MFMA-bound GEMMs)"}
    del actor
    if not a.no_sweep:
        line["results"] = sweep()
        mf = [r for r in line["results"] if "fp8 GEMM" in r["workload"]]
        if mf:
            best = next((r for r in mf if "N=4096" in r["workload"]), mf[0])  # the shape the traffic figure is for
            pg = PROFILED_NS["fp8_gemm_4096"]
            line["roofline_mfma"] = {"bound": "mfma", "achieved": best["TOPS"], "peak": MFMA_PEAK_TOPS["fp8"],
                                     "unit": "TFLOP/s", "frac": round(best["TOPS"] / MFMA_PEAK_TOPS["fp8"], 5),
                                     "frac_one_warm_call": best.get("frac_of_roofline_one_warm_call"),
                                     "frac_profiled": round(2 * 8192 * 4096 * 4096 / (pg * 1e-9) / 1e12 / MFMA_PEAK_TOPS["fp8"], 5) if pg else None,
                                     "profiled_avg_kernel_ns": pg,
                                     "traffic": FP8_GEMM_TRAFFIC, "kernel": "nq::gemm8_kernel<fp8>",
                                     "workload": best["workload"], "avg_launch_us": best["us_per_call"],
                                     "avg_launch_us_one_warm_call": best.get("us_per_call_one_warm_call"),
                                     "note": "frac: after 50 ms of the same launches (steady clocks); frac_one_warm_call: the "
                                             "reference's protocol, samples right after one warm call (the power "
                                             "management's transient after an idle spell); frac_profiled: from the committed "
                                             "rocprofv3 trace of a long run of `bench.py --only fp8gemm`",
                                     "mfma_only": mfma_only()}
    if not a.no_cpu:
        line["cpu_baseline"] = cpu_baseline()
    print(json.dumps(line))


if __name__ == "__main__":
    main()
