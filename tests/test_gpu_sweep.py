"""Randomised shapes for every format and activation type, through the C ABI.

Each case draws a format, M (1 .. 1000, dense around the kernel-selection
thresholds), IN, OUT (ragged on purpose: OUT = 1 .. 3000, IN any legal
multiple), activation and output dtypes, bias kind and epilogue, and checks
the result against an fp64 product with the weights the CPU oracle dequantises
from the codes the case drew (tests/refw.py; the library is never asked what
its weights are); the int8 x int8 accumulators are compared exactly.
Bars as everywhere: 1e-3 * RMS (fp8: 1e-2), plus half a bf16 step when the
output is bf16.
"""
import numpy as np
import pytest
import torch

from noeira_amd import formats as F
from noeira_amd.qlinear import FP8Linear, QLinear, W4GroupLinear, W8Linear, quantize_rows_i8
import refw

pytestmark = pytest.mark.gpu

MS = [1, 1, 1, 2, 3, 4, 5, 7, 8, 15, 16, 17, 31, 32, 33, 63, 64, 65, 100, 127, 128, 135, 255, 256, 257, 300, 513, 1000]


def _pick_k(rng, mult, hi=4096):
    c = rng.integers(0, 4)
    if c == 0:
        return int(mult * rng.integers(1, 9))
    if c == 1:
        return int(rng.choice([256, 512, 960, 1024, 2560, 3200, 4096]) // mult * mult)
    return int(mult * rng.integers(1, hi // mult + 1))


def _pick_n(rng):
    c = rng.integers(0, 4)
    if c == 0:
        return int(rng.integers(1, 40))
    if c == 1:
        return int(rng.choice([8, 256, 320, 512, 960, 2560, 3200, 4096]))
    return int(rng.integers(1, 3000))


def _check(tag, y, exact, out_bf16, tol=1e-3):
    y = y.double()
    rms = max(float(exact.pow(2).mean().sqrt()), 1e-30)
    err = (y - exact).abs()
    allow = tol * rms + (2.0 ** -8) * exact.abs() * (1 if out_bf16 else 0)
    assert not bool(torch.isnan(y).any()), tag
    assert not bool((err > allow).any()), (tag, float(err.max()) / rms)


@pytest.mark.parametrize("seed,prefer", [(11, False), (12, False), (21, True), (22, True)])
def test_random_shapes(seed, prefer):
    """prefer: the layers ask for the kernels over their tile-ordered copy wherever those can run
    (NQ_FLAG_PREFER_TILE), so the same ragged shapes reach them below the sizes they take by default."""
    rng = np.random.default_rng(seed)
    for case in range(150):
        fmt = ["q4_0", "w8", "w4g", "fp8", "w8a8"][case % 5]
        M = int(rng.choice(MS))
        N = _pick_n(rng)
        xdt = torch.float32 if rng.integers(0, 2) else torch.bfloat16
        odt = torch.float32 if rng.integers(0, 3) else torch.bfloat16
        use_bias = int(rng.integers(0, 3))  # 0 none, 1 fp32, 2 bf16
        epi = "relu" if rng.integers(0, 3) == 0 else "none"
        w = None
        hi = 8192 if (prefer and rng.integers(0, 3) == 0) else 4096  # (the tile kernels' own K ranges end at 4096 .. 8192)
        if fmt == "q4_0":
            K = _pick_k(rng, 32, hi)
            lin = QLinear(K, N, prefer_tile=prefer)
            blocks = rng.integers(0, 256, (N, K // 32, 18), dtype=np.uint8)
            sc = rng.uniform(1e-3, 1e-2, (N, K // 32)).astype(np.float16).view(np.uint16)
            blocks[:, :, 0] = sc & 0xFF
            blocks[:, :, 1] = sc >> 8
            lin.set_blocks(blocks.reshape(-1))
            deq = refw.q4_0(blocks, N, K)
        elif fmt in ("w8", "w8a8"):
            K = _pick_k(rng, 128 if (fmt == "w8a8" and rng.integers(0, 2)) else 16, hi)
            lin = W8Linear(K, N, prefer_tile=prefer)
            w = rng.integers(-127, 128, (N, K), dtype=np.int8)
            sw_host = rng.uniform(1e-3, 1e-2, N).astype(np.float32)
            lin.set_weight(w, sw_host)
            deq = refw.w8(w, sw_host)
        elif fmt == "w4g":
            group = int(rng.choice([128, 128, 64, 32]))
            K = _pick_k(rng, 32, hi)
            G = -(-K // group)
            q = rng.integers(0, 16, (N, K), dtype=np.uint8)
            z = rng.integers(0, 16, (N, G), dtype=np.uint8)
            codes, zps = F.pack_w4g(q, z)
            lin = W4GroupLinear(K, N, group, prefer_tile=prefer)
            sg = rng.uniform(1e-3, 1e-2, (N, G)).astype(np.float16)
            lin.set_weight(codes, sg, zps)
            deq = refw.w4g(codes, sg, zps, N, K, group)
        else:
            K = _pick_k(rng, 16)
            lin = FP8Linear(K, N)
            wt = torch.from_numpy(rng.standard_normal((N, K)).astype(np.float32)).to(torch.float8_e4m3fn)
            lin.set_weight(wt.view(torch.uint8).numpy(), 1.0 / 16)
            deq = refw.fp8(wt.view(torch.uint8).numpy(), 1.0 / 16)
        tag = "%s M=%d K=%d N=%d x=%s y=%s bias=%d %s" % (fmt, M, K, N, str(xdt)[6:], str(odt)[6:], use_bias, epi)
        bias = None
        if use_bias:
            bias = torch.from_numpy((rng.standard_normal(N) * 0.02).astype(np.float32)).cuda()
            if use_bias == 2:
                bias = bias.to(torch.bfloat16)
        x = torch.from_numpy(rng.standard_normal((M, K)).astype(np.float32)).cuda().to(xdt)

        def fin(e):
            if bias is not None:
                e = e + bias.double()
            return e.clamp_min(0) if epi == "relu" else e

        if fmt in ("q4_0", "w8", "w4g"):
            y = lin.forward(x, bias=bias, epilogue=epi, out_dtype=odt)
            _check(tag, y, fin(x.double() @ deq.T), odt == torch.bfloat16)
        elif fmt == "fp8":
            xc = x.float().to(torch.float8_e4m3fn)
            sa = torch.tensor([0.125], dtype=torch.float32, device="cuda")
            y = lin.forward(xc.view(torch.uint8), sa, bias=bias, epilogue=epi, out_dtype=odt)
            _check(tag, y, fin(0.125 * (xc.double() @ deq.T)), odt == torch.bfloat16, 1e-2)
        else:
            xq, sx = quantize_rows_i8(x.float().contiguous())
            wd = torch.from_numpy(w).cuda().double()
            acc_exact = xq.double() @ wd.T  # exact: |acc| < 2^53
            acc = lin.forward_a8(xq, sx, out_dtype=torch.int32)
            assert bool((acc.double() == acc_exact).all()), tag + ": int32 accumulators differ"
            sw = torch.from_numpy(sw_host).cuda().double()
            y = lin.forward_a8(xq, sx, bias=bias, epilogue=epi, out_dtype=odt)
            _check(tag, y, fin(acc_exact * sx.double()[:, None] * sw[None, :]), odt == torch.bfloat16)
        del lin


@pytest.mark.parametrize("fmt", ["q4_0", "w8", "w4g", "w4g64"])
@pytest.mark.parametrize("xdt", [torch.bfloat16, torch.float32])
def test_many_rows(fmt, xdt):
    """Many rows (512 and more, where its workgroups fill the chip): bf16 / fp32 activations take the kernel that stages a [64 or 128] x 128 tile per
    workgroup: ragged M, N and K (K not a multiple of its k-step, N not a multiple of 128, M not a multiple
    of the tile), bias, ReLU and bf16 output, against the fp64 product with the oracle's dequantised weights."""
    rng = np.random.default_rng(sum(map(ord, fmt + str(xdt))))
    for (M, K, N) in ((2048, 960, 1600), (2100, 992, 1200), (5000, 4096, 650), (4096, 160, 1000), (513, 960, 3000)):
        if fmt.startswith("w4g"):
            group = 128 if fmt == "w4g" else 64
            G = -(-K // group)
            q = rng.integers(0, 16, (N, K), dtype=np.uint8)
            z = rng.integers(0, 16, (N, G), dtype=np.uint8)
            codes, zps = F.pack_w4g(q, z)
            lin = W4GroupLinear(K, N, group)
            sg = rng.uniform(1e-3, 1e-2, (N, G)).astype(np.float16)
            lin.set_weight(codes, sg, zps)
            deq = refw.w4g(codes, sg, zps, N, K, group)
        elif fmt == "w8":
            lin = W8Linear(K, N)
            w, sw_host = rng.integers(-127, 128, (N, K), dtype=np.int8), rng.uniform(1e-3, 1e-2, N).astype(np.float32)
            lin.set_weight(w, sw_host)
            deq = refw.w8(w, sw_host)
        else:
            lin = QLinear(K, N)
            blocks = rng.integers(0, 256, (N, K // 32, 18), dtype=np.uint8)
            sc = rng.uniform(1e-3, 1e-2, (N, K // 32)).astype(np.float16).view(np.uint16)
            blocks[:, :, 0] = sc & 0xFF
            blocks[:, :, 1] = sc >> 8
            lin.set_blocks(blocks.reshape(-1))
            deq = refw.q4_0(blocks, N, K)
        x = torch.from_numpy(rng.standard_normal((M, K)).astype(np.float32)).cuda().to(xdt)
        tag = "%s M=%d K=%d N=%d %s" % (fmt, M, K, N, str(xdt)[6:])
        bias = torch.from_numpy((rng.standard_normal(N) * 0.02).astype(np.float32)).cuda()
        y = lin.forward(x, bias=bias, epilogue="relu", out_dtype=torch.bfloat16)
        _check(tag, y, (x.double() @ deq.T + bias.double()).clamp_min(0), True)
        _check(tag, lin.forward(x), x.double() @ deq.T, False)
        del lin


def test_many_rows_fused_parts_match_their_own_layers():
    """From 512 rows on the kernel, and with it the order of a row's sum, may follow the total row count:
    a part of a row-fused layer then matches its own layer to the last bits' worth, not bit for bit."""
    from noeira_amd.qlinear import FusedRows

    rng = np.random.default_rng(77)
    K, outs, M = 960, [2560, 320, 130], 2100
    layers = []
    for n in outs:
        ql = QLinear(K, n)
        blocks = rng.integers(0, 256, (n, K // 32, 18), dtype=np.uint8)
        sc = rng.uniform(1e-3, 1e-2, (n, K // 32)).astype(np.float16).view(np.uint16)
        blocks[:, :, 0] = sc & 0xFF
        blocks[:, :, 1] = sc >> 8
        ql.set_blocks(blocks.reshape(-1))
        layers.append(ql)
    fused = FusedRows(layers)
    x = torch.from_numpy(rng.standard_normal((M, K)).astype(np.float32)).cuda()
    for l, y in zip(layers, fused.forward(x)):
        own = l.forward(x)
        assert (y - own).abs().max().item() <= 2e-6 * own.abs().max().item()


@pytest.mark.parametrize("fmt", ["q4_0", "w4g", "w4g64"])
def test_single_row_fp32_x_through_lds(fmt):
    """One row of fp32 activations over a 4-bit weight with a thousand wavefronts and more: the workgroup
    stages x in LDS and every lane takes its chunks from there.  A row of 30, 31 (odd) and 191 chunks (the
    most the kernel holds; the last lane group's chunks run past the row), and a short launch that loads x
    directly, for comparison."""
    rng = np.random.default_rng(sum(map(ord, fmt)) + 5)
    for (K, N) in ((960, 2560), (992, 3000), (6112, 1100), (960, 5120), (960, 700)):
        if fmt.startswith("w4g"):
            group = 128 if fmt == "w4g" else 64
            G = -(-K // group)
            q = rng.integers(0, 16, (N, K), dtype=np.uint8)
            z = rng.integers(0, 16, (N, G), dtype=np.uint8)
            codes, zps = F.pack_w4g(q, z)
            lin = W4GroupLinear(K, N, group)
            sg = rng.uniform(1e-3, 1e-2, (N, G)).astype(np.float16)
            lin.set_weight(codes, sg, zps)
            deq = refw.w4g(codes, sg, zps, N, K, group)
        else:
            lin = QLinear(K, N)
            blocks = rng.integers(0, 256, (N, K // 32, 18), dtype=np.uint8)
            sc = rng.uniform(1e-3, 1e-2, (N, K // 32)).astype(np.float16).view(np.uint16)
            blocks[:, :, 0] = sc & 0xFF
            blocks[:, :, 1] = sc >> 8
            lin.set_blocks(blocks.reshape(-1))
            deq = refw.q4_0(blocks, N, K)
        x = torch.from_numpy(rng.standard_normal((1, K)).astype(np.float32)).cuda()
        tag = "%s M=1 K=%d N=%d fp32" % (fmt, K, N)
        exact = x.double() @ deq.T
        y = lin.forward(x)
        _check(tag, y, exact, False)
        # the reference's band for its fp32 path: 1e-5 of the largest value
        assert float((y.double() - exact).abs().max()) <= 1e-5 * float(exact.abs().max()), tag
        assert torch.equal(y, lin.forward(x)), tag + ": a repeated call differs"
        del lin


def test_random_large_layers():
    """Layers of 4 M to 100 M weights with ragged OUT, at row counts from 1 to 512 (every kernel's range of rows and
    the counts either side of each hand-over): the kernels over the
    tile-ordered copy and the row-ordered ones (tile copy and preference drawn per case), bias + ReLU, fp32 or bf16
    out, against the fp64 product with the oracle's dequantised weights; a repeated call returns the same bits."""
    rng = np.random.default_rng(2026)
    for case in range(90):
        fmt = ["q4_0", "w4g", "w8"][case % 3]
        K = int(rng.choice([1536, 2048, 2176, 2560, 3072, 4096, 4224, 5120, 6144, 8192]))
        N = int(rng.integers(2100, 12500))
        M = int(rng.choice([1, 2, 3, 5, 6, 8, 11, 16, 17, 24, 33, 48, 64, 95, 96, 100, 135, 200, 256, 257, 300, 384, 500, 511, 512]))
        prefer, tc = bool(rng.integers(0, 2)), bool(rng.integers(0, 4))
        xdt = torch.bfloat16 if rng.integers(0, 3) else torch.float32
        odt = torch.float32 if rng.integers(0, 2) else torch.bfloat16
        if fmt == "q4_0":
            lin = QLinear(K, N, tile_copy=tc, prefer_tile=prefer)
            blocks = rng.integers(0, 256, (N, K // 32, 18), dtype=np.uint8)
            sc = rng.uniform(1e-3, 1e-2, (N, K // 32)).astype(np.float16).view(np.uint16)
            blocks[:, :, 0] = sc & 0xFF
            blocks[:, :, 1] = sc >> 8
            lin.set_blocks(blocks.reshape(-1))
            deq = refw.q4_0(blocks, N, K)
        elif fmt == "w4g":
            G = -(-K // 128)
            codes, zps = F.pack_w4g(rng.integers(0, 16, (N, K), dtype=np.uint8), rng.integers(0, 16, (N, G), dtype=np.uint8))
            lin = W4GroupLinear(K, N, 128, tile_copy=tc, prefer_tile=prefer)
            sg = rng.uniform(1e-3, 1e-2, (N, G)).astype(np.float16)
            lin.set_weight(codes, sg, zps)
            deq = refw.w4g(codes, sg, zps, N, K, 128)
        else:
            lin = W8Linear(K, N, tile_copy=tc, prefer_tile=prefer)
            w, sw_host = rng.integers(-127, 128, (N, K), dtype=np.int8), rng.uniform(1e-3, 1e-2, N).astype(np.float32)
            lin.set_weight(w, sw_host)
            deq = refw.w8(w, sw_host)
        tag = "%s M=%d K=%d N=%d x=%s y=%s prefer=%d tile_copy=%d" % (fmt, M, K, N, str(xdt)[6:], str(odt)[6:], prefer, tc)
        bias = torch.from_numpy((rng.standard_normal(N) * 0.02).astype(np.float32)).cuda()
        x = torch.from_numpy(rng.standard_normal((M, K)).astype(np.float32)).cuda().to(xdt)
        y = lin.forward(x, bias=bias, epilogue="relu", out_dtype=odt)
        _check(tag, y, (x.double() @ deq.T + bias.double()).clamp_min(0), odt == torch.bfloat16)
        assert torch.equal(lin.forward(x, bias=bias, epilogue="relu", out_dtype=odt), y), tag + ": a repeated call differs"
        del lin, deq
