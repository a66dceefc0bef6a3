"""The single-row GEMV over large 4-bit and int8 weights (megabytes of codes), through the C ABI, on both
device layouts: the tile-ordered copy large layers keep by default (nq_gemv_tile.hip) and the row-ordered
codes alone (tile_copy=False: nq_gemv_row4 / row8 / split8),
against fp64 products with the weights the CPU oracle dequantises from the codes each test drew
(tests/refw.py; the library is not asked what its weights are) and, at a size the oracle
finishes in seconds, against the oracle's own forward.

Bars: the reference's fp32 band for Q4_0 with fp32 activations (1e-5 of the largest reference
value, tests/nn/quant/qlinear_common.mojo:39-45), 1e-3 of the output RMS otherwise; repeated
calls return the same bits (test_qlinear_gpu.mojo:96,128).
"""
import numpy as np
import pytest
import torch

from noeira_amd import formats as F
from noeira_amd.qlinear import FusedRows, QLinear, W4GroupLinear
from oracle import oracle as O
import refw

pytestmark = pytest.mark.gpu


TILE = pytest.mark.parametrize("tile_copy", [True, False], ids=["tile", "rows"])


def q4_layer(rng, K, N, scale_kind="uniform", tile_copy=True):
    lin = QLinear(K, N, tile_copy=tile_copy)
    blocks = rng.integers(0, 256, (N, K // 32, 18), dtype=np.uint8)
    sc = rng.uniform(1e-3, 1e-2, (N, K // 32)).astype(np.float16)
    if scale_kind == "signed":
        sc *= rng.choice([-1.0, 1.0], sc.shape).astype(np.float16)
    bits = sc.view(np.uint16)
    blocks[:, :, 0] = bits & 0xFF
    blocks[:, :, 1] = bits >> 8
    lin.set_blocks(blocks.reshape(-1))
    lin.host_blocks = blocks
    lin.ref_deq = lambda: refw.q4_0(blocks, N, K)
    return lin


# rows of 1 .. 8 KiB of codes; 11008 = 5.375 loads of a wavefront (a ragged last one); N off every tile size
@pytest.mark.parametrize("K,N", [(2048, 2051), (2176, 1999), (4096, 1100), (4096, 4096), (5504, 800), (11008, 777),
                                 (16384, 300), (8192, 1031)])
@pytest.mark.parametrize("xdt", [torch.float32, torch.bfloat16])
@TILE
def test_q4_0_large_single_row(K, N, xdt, tile_copy):
    rng = np.random.default_rng(K + N)
    lin = q4_layer(rng, K, N, "signed", tile_copy)
    deq = lin.ref_deq()
    x = torch.from_numpy(rng.standard_normal((1, K)).astype(np.float32)).to(xdt).cuda()
    y = lin.forward(x)
    exact = x.double() @ deq.T
    rel = float((y.double() - exact).abs().max() / exact.abs().max())
    assert rel < 1e-5, rel
    assert torch.equal(lin.forward(x), y)


def test_q4_0_large_against_oracle_forward():
    rng = np.random.default_rng(7)
    K, N = 4096, 1024
    lin = q4_layer(rng, K, N)
    x = rng.standard_normal((1, K)).astype(np.float32)
    y = lin.forward(torch.from_numpy(x).cuda()).cpu().numpy()
    want = O.qlinear_forward_cpu(lin.host_blocks.reshape(-1), K, N, x)
    assert O.rel_max(y, want) < 1e-5
    exact = O.dense_forward_f64(O.dequantize_q4_0(lin.host_blocks.reshape(N, -1), N, K), x)
    assert O.rel_max(y, exact.astype(np.float32)) < 1e-5


@pytest.mark.parametrize("K,N,group", [(4096, 1500, 128), (2048, 2100, 64), (11008, 600, 128), (4096, 1030, 32),
                                         (8192, 520, 256), (2176, 2003, 128), (16384, 270, 128)])
@pytest.mark.parametrize("xdt", [torch.float32, torch.bfloat16])
@TILE
def test_w4_group_large_single_row(K, N, group, xdt, tile_copy):
    rng = np.random.default_rng(K + N + group)
    G = -(-K // group)
    q = rng.integers(0, 16, (N, K), dtype=np.uint8)
    z = rng.integers(0, 16, (N, G), dtype=np.uint8)
    codes, zps = F.pack_w4g(q, z)
    lin = W4GroupLinear(K, N, group, tile_copy=tile_copy)
    sg = rng.uniform(1e-3, 1e-2, (N, G)).astype(np.float16)
    lin.set_weight(codes, sg, zps)
    deq = refw.w4g(codes, sg, zps, N, K, group)
    x = torch.from_numpy(rng.standard_normal((1, K)).astype(np.float32)).to(xdt).cuda()
    bias = torch.from_numpy((rng.standard_normal(N) * 0.02).astype(np.float32)).cuda()
    exact = x.double() @ deq.T + bias.double()
    rms = float(exact.pow(2).mean().sqrt())
    y = lin.forward(x, bias=bias)
    assert float((y.double() - exact).abs().max()) < 1e-5 * rms  # (the north star's bar is 1e-3)
    assert torch.equal(lin.forward(x, bias=bias), y)
    yr = lin.forward(x, bias=bias.to(torch.bfloat16), epilogue="relu", out_dtype=torch.bfloat16)
    want = (x.double() @ deq.T + bias.to(torch.bfloat16).double()).clamp_min(0)
    assert float((yr.double() - want).abs().max()) <= 1e-3 * rms + 2.0 ** -8 * float(want.abs().max())


@TILE
def test_large_fused_rows_single_row(tile_copy):
    """q | k | v of a 4096-wide model as one row-fused layer: every part equals its own forward."""
    rng = np.random.default_rng(11)
    K = 4096
    parts = [q4_layer(rng, K, n, tile_copy=tile_copy) for n in (1024, 256, 260)]
    fused = FusedRows(parts)
    x = torch.from_numpy(rng.standard_normal((1, K)).astype(np.float32)).cuda()
    outs = fused.forward(x)
    for lin, y in zip(parts, outs):
        want = lin.forward(x)
        assert float((y - want).abs().max()) <= 2e-6 * float(want.abs().max())


@TILE
def test_nan_and_zero_scales_stay_local(tile_copy):
    """A zero scale silences its group whatever the codes (qlinear.mojo:32-34); a NaN scale poisons its own
    row only."""
    rng = np.random.default_rng(13)
    K, N = 4096, 1024
    lin = QLinear(K, N, tile_copy=tile_copy)
    blocks = rng.integers(0, 256, (N, K // 32, 18), dtype=np.uint8)
    bits = rng.uniform(1e-3, 1e-2, (N, K // 32)).astype(np.float16).view(np.uint16)
    bits[5, :] = 0          # row 5: all groups silent
    bits[9, 17] = 0x7E01    # row 9: one NaN scale
    blocks[:, :, 0] = bits & 0xFF
    blocks[:, :, 1] = bits >> 8
    lin.set_blocks(blocks.reshape(-1))
    x = torch.from_numpy(rng.standard_normal((1, K)).astype(np.float32)).cuda()
    y = lin.forward(x).cpu().numpy()[0]
    assert y[5] == 0.0
    assert np.isnan(y[9]) and np.isnan(y).sum() == 1


# ── 8-bit weights (int8 per-channel; fp8 is reached through the C ABI with bf16 / fp32 x only) ──
@pytest.mark.parametrize("K,N", [(4096, 4096), (4112, 1030), (8192, 600), (11008, 400), (16384, 260), (5120, 1500),
                                 (1024, 4100), (1088, 3900)])
@pytest.mark.parametrize("xdt", [torch.float32, torch.bfloat16])
@TILE
def test_w8_large_single_row(K, N, xdt, tile_copy):
    from noeira_amd.qlinear import W8Linear
    rng = np.random.default_rng(K * 7 + N)
    w = rng.integers(-127, 128, (N, K), dtype=np.int8)
    w[3, :] = -128  # the one code the symmetric range leaves out
    s = rng.uniform(1e-3, 1e-2, N).astype(np.float32)
    lin = W8Linear(K, N, tile_copy=tile_copy)
    lin.set_weight(w, s)
    x = torch.from_numpy(rng.standard_normal((1, K)).astype(np.float32)).to(xdt).cuda()
    bias = torch.from_numpy((rng.standard_normal(N) * 0.02).astype(np.float32)).cuda()
    y = lin.forward(x, bias=bias)
    exact = O.w8_forward_f64(w, s, x.float().cpu().numpy(), bias.cpu().numpy())
    rms = np.sqrt((exact ** 2).mean())
    assert np.abs(y.cpu().numpy() - exact).max() < 1e-5 * rms  # (the north star's bar is 1e-3)
    assert torch.equal(lin.forward(x, bias=bias), y)
    yr = lin.forward(x, bias=bias.to(torch.bfloat16), epilogue="relu", out_dtype=torch.bfloat16).float().cpu().numpy()
    want = np.maximum(O.w8_forward_f64(w, s, x.float().cpu().numpy(), bias.to(torch.bfloat16).float().cpu().numpy()), 0)
    assert np.abs(yr - want).max() <= 1e-3 * rms + 2.0 ** -8 * np.abs(want).max()


# the int8-matrix-core kernel that splits x into three int8 terms: rows of 4096 .. 8192 codes, 16 MB and more
# (one, two and four rows per wavefront; N off every tile size)
@pytest.mark.parametrize("K,N", [(4096, 6403), (4096, 8201), (5120, 8197), (8192, 3101), (4112, 8195)])
@pytest.mark.parametrize("xdt", [torch.float32, torch.bfloat16])
@TILE
def test_w8_split_single_row(K, N, xdt, tile_copy):
    from noeira_amd.qlinear import W8Linear
    rng = np.random.default_rng(K * 3 + N)
    w = rng.integers(-127, 128, (N, K), dtype=np.int8)
    w[3, :] = -128
    s = rng.uniform(1e-3, 1e-2, N).astype(np.float32)
    lin = W8Linear(K, N, tile_copy=tile_copy)
    lin.set_weight(w, s)
    x = rng.standard_normal((1, K)).astype(np.float32)
    x[0, 5] = 300.0  # an outlier sets the scale of the split: the small elements still count
    x = torch.from_numpy(x).to(xdt).cuda()
    bias = torch.from_numpy((rng.standard_normal(N) * 0.02).astype(np.float32)).cuda()
    wd = torch.from_numpy(w).cuda().double()
    sd = torch.from_numpy(s).cuda().double()
    exact = (x.double() @ wd.T) * sd + bias.double()
    rms = float(exact.pow(2).mean().sqrt())
    y = lin.forward(x, bias=bias)
    # the split leaves up to 6e-8 of |x|max per element: under an outlier of 60 sigma that is 1e-5 of the output RMS,
    # a hundredth of the band of 1e-3
    assert float((y.double() - exact).abs().max()) < 1e-4 * rms
    assert torch.equal(lin.forward(x, bias=bias), y)
    yr = lin.forward(x, bias=bias.to(torch.bfloat16), epilogue="relu", out_dtype=torch.bfloat16)
    want = ((x.double() @ wd.T) * sd + bias.to(torch.bfloat16).double()).clamp_min(0)
    assert float((yr.double() - want).abs().max()) <= 1e-3 * rms + 2.0 ** -8 * float(want.abs().max())


@TILE
def test_w8_split_special_rows(tile_copy):
    from noeira_amd.qlinear import W8Linear
    rng = np.random.default_rng(77)
    K, N = 4096, 6400
    w = rng.integers(-127, 128, (N, K), dtype=np.int8)
    s = rng.uniform(1e-3, 1e-2, N).astype(np.float32)
    lin = W8Linear(K, N, tile_copy=tile_copy)
    lin.set_weight(w, s)
    bias = torch.from_numpy((rng.standard_normal(N) * 0.02).astype(np.float32)).cuda()
    zero = torch.zeros((1, K), dtype=torch.float32, device="cuda")
    assert torch.equal(lin.forward(zero, bias=bias)[0], bias)  # a zero row: the bias, bit for bit
    tiny = torch.full((1, K), 1e-38, dtype=torch.float32, device="cuda")
    assert float((lin.forward(tiny, bias=bias)[0] - bias).abs().max()) < 1e-30
    for bad in (float("nan"), float("inf"), -float("inf")):  # a NaN or an infinity in x: every output is NaN
        xb = torch.from_numpy(rng.standard_normal((1, K)).astype(np.float32)).cuda()
        xb[0, 1234] = bad
        assert bool(torch.isnan(lin.forward(xb, bias=bias)).all())


@TILE
def test_w8_split_fused_rows(tile_copy):
    from noeira_amd.qlinear import W8Linear
    rng = np.random.default_rng(22)
    K = 4096
    parts = []
    for n in (6000, 2200, 260):
        lin = W8Linear(K, n, tile_copy=tile_copy)
        lin.set_weight(rng.integers(-127, 128, (n, K), dtype=np.int8), rng.uniform(1e-3, 1e-2, n).astype(np.float32))
        parts.append(lin)
    fused = FusedRows(parts)
    x = torch.from_numpy(rng.standard_normal((1, K)).astype(np.float32)).to(torch.bfloat16).cuda()
    for lin, y in zip(parts, fused.forward(x)):
        want = lin.forward(x)  # (the parts alone take other kernels: same products, another order of sums)
        assert float((y - want).abs().max()) <= 2e-6 * float(want.abs().max())


@TILE
def test_w8_large_fused_rows_single_row(tile_copy):
    from noeira_amd.qlinear import W8Linear
    rng = np.random.default_rng(21)
    K = 8192
    parts = []
    for n in (1024, 300, 260):
        lin = W8Linear(K, n, tile_copy=tile_copy)
        lin.set_weight(rng.integers(-127, 128, (n, K), dtype=np.int8), rng.uniform(1e-3, 1e-2, n).astype(np.float32))
        parts.append(lin)
    fused = FusedRows(parts)
    x = torch.from_numpy(rng.standard_normal((1, K)).astype(np.float32)).to(torch.bfloat16).cuda()
    for lin, y in zip(parts, fused.forward(x)):
        want = lin.forward(x)  # (the small parts alone take another kernel: same products, another order of sums)
        assert float((y - want).abs().max()) <= 2e-6 * float(want.abs().max())


@pytest.mark.parametrize("K,N", [(4096, 2048), (5504, 1000)])
def test_tile_copy_agrees_with_row_kernels(K, N):
    """The two device layouts hold the same weights: same products, another order of sums."""
    from noeira_amd.qlinear import W8Linear
    rng = np.random.default_rng(K + 3 * N)
    x = torch.from_numpy(rng.standard_normal((1, K)).astype(np.float32)).cuda()
    a, b = q4_layer(np.random.default_rng(5), K, N, tile_copy=True), q4_layer(np.random.default_rng(5), K, N, tile_copy=False)
    assert np.array_equal(a.blocks(), b.blocks())
    ya, yb = a.forward(x), b.forward(x)
    assert float((ya - yb).abs().max()) <= 2e-6 * float(yb.abs().max())
    assert torch.equal(a.dequantized_dev().double(), a.ref_deq())  # (fp32 values of the oracle, exactly)
    assert torch.equal(a.dequantized_dev(), b.dequantized_dev())
    w = rng.integers(-127, 128, (N, K), dtype=np.int8)
    s = rng.uniform(1e-3, 1e-2, N).astype(np.float32)
    la, lb = W8Linear(K, N), W8Linear(K, N, tile_copy=False)
    la.set_weight(w, s), lb.set_weight(w, s)
    for xdt in (torch.float32, torch.bfloat16):
        ya, yb = la.forward(x.to(xdt)), lb.forward(x.to(xdt))
        assert float((ya - yb).abs().max()) <= 2e-6 * float(yb.abs().max())


def test_tile_relu_rule_and_nonfinite_x():
    """z > 0 ? z : 0 (ops/relu_op.mojo:29-31): a NaN pre-activation becomes 0, -0.0 becomes +0.0."""
    from noeira_amd.qlinear import W8Linear
    rng = np.random.default_rng(31)
    K, N = 4096, 1040
    lin = q4_layer(rng, K, N)
    x = torch.from_numpy(rng.standard_normal((1, K)).astype(np.float32)).cuda()
    bias = torch.zeros(N, device="cuda")
    xz = torch.zeros((1, K), device="cuda")
    y = lin.forward(xz, bias=-bias, epilogue="relu")  # bias -0.0, products 0: z = -0.0 or +0.0
    assert torch.equal(y.view(torch.int32), torch.zeros_like(y, dtype=torch.int32))  # +0.0 bit for bit
    x[0, 77] = float("nan")
    assert bool(torch.isnan(lin.forward(x)).all())
    assert torch.equal(lin.forward(x, epilogue="relu"), torch.zeros((1, N), device="cuda"))
    w8 = W8Linear(K, N)
    w8.set_weight(rng.integers(-127, 128, (N, K), dtype=np.int8), rng.uniform(1e-3, 1e-2, N).astype(np.float32))
    assert bool(torch.isnan(w8.forward(x)).all())
    assert torch.equal(w8.forward(x, epilogue="relu"), torch.zeros((1, N), device="cuda"))


# ---- 4-bit codes on the int8 matrix cores (the persistent route large layers take at one row) --------------
def _w4g_layer(rng, K, N, **kw):
    G = K // 128
    codes, zps = F.pack_w4g(rng.integers(0, 16, (N, K), dtype=np.uint8), rng.integers(0, 16, (N, G), dtype=np.uint8))
    lin = W4GroupLinear(K, N, 128, **kw)
    sg = rng.uniform(1e-3, 1e-2, (N, G)).astype(np.float16)
    lin.set_weight(codes, sg, zps)
    lin.ref_deq = lambda: refw.w4g(codes, sg, zps, N, K, 128)
    return lin


def _q4_signed(rng, K, N, **kw):
    lin = QLinear(K, N, **kw)
    blocks = rng.integers(0, 256, (N, K // 32, 18), dtype=np.uint8)
    bits = (rng.uniform(1e-3, 1e-2, (N, K // 32)) * rng.choice([-1.0, 1.0], (N, K // 32))).astype(np.float16).view(np.uint16)
    blocks[:, :, 0], blocks[:, :, 1] = bits & 0xFF, bits >> 8
    lin.set_blocks(blocks.reshape(-1))
    lin.ref_deq = lambda: refw.q4_0(blocks, N, K)
    return lin


# default dispatch: layers with three row tiles and more per resident workgroup (N >= 24576 up to K = 4096, >= 12288
# beyond); with NQ_FLAG_PREFER_TILE: every K split of the kernel on small layers (2 .. 4 steps per wavefront, 8 and 16
# wavefronts, K not a multiple of the wavefronts' share), one tile per workgroup
@pytest.mark.parametrize("K,N,prefer", [(2048, 24600, False), (4224, 12400, False), (8192, 12300, False), (2048, 2051, True),
                                        (2176, 1999, True), (4096, 1100, True), (5504, 800, True), (8192, 1031, True),
                                        (3072, 1400, True)])
@pytest.mark.parametrize("fmt", ["q4_0", "w4g"])
@pytest.mark.parametrize("xdt", [torch.float32, torch.bfloat16])
def test_four_bit_single_row_on_the_int8_matrix_cores(K, N, prefer, fmt, xdt):
    """x enters as three int8 terms under one scale per wavefront slice (error <= 6e-8 of the slice's largest
    |x| per element), the codes as int8, sums exact in int32: the fp32 band of the reference (1e-5 of the largest
    reference value) holds for fp32 and bf16 activations alike."""
    rng = np.random.default_rng(K + N + len(fmt))
    lin = (_q4_signed if fmt == "q4_0" else _w4g_layer)(rng, K, N, prefer_tile=prefer)
    deq = lin.ref_deq()
    x = torch.from_numpy(rng.standard_normal((1, K)).astype(np.float32)).to(xdt).cuda()
    bias = torch.from_numpy((rng.standard_normal(N) * 0.02).astype(np.float32)).cuda()
    y = lin.forward(x, bias=bias)
    exact = x.double() @ deq.T + bias.double()
    assert float((y.double() - exact).abs().max()) <= 1e-5 * float(exact.abs().max())
    assert torch.equal(lin.forward(x, bias=bias), y)
    yr = lin.forward(x, bias=bias.to(torch.bfloat16), epilogue="relu", out_dtype=torch.bfloat16)
    want = (x.double() @ deq.T + bias.to(torch.bfloat16).double()).clamp_min(0)
    assert float((yr.double() - want).abs().max()) <= 2.0 ** -8 * float(want.abs().max()) + 1e-5 * float(exact.abs().max())
    del exact, want
    # an outlier sixty times the rest: the terms keep 24 bits under the slice's scale
    xo = x.clone()
    xo[0, K // 3] = 60.0
    yo = lin.forward(xo)
    eo = xo.double() @ deq.T
    assert float((yo.double() - eo).abs().max()) <= 1e-5 * float(eo.abs().max())
    # a NaN or an infinity in x: every output NaN (the exact result would be NaN or +-inf per row)
    xn = x.clone()
    xn[0, 5] = float("inf")
    assert bool(torch.isnan(lin.forward(xn)).all())


@pytest.mark.parametrize("fmt", ["q4_0", "w4g", "w8_tile", "w8_rows"])
@pytest.mark.parametrize("mag", [1e-35, 3e-25, 1e20])
def test_single_row_of_tiny_or_huge_activations_keeps_its_direction(fmt, mag):
    """The kernels that split x into int8 terms under the slice's largest magnitude: an x whose every value is
    around 1e-35 (or 1e20) is still a vector with a direction, and y = deq(W) x scales with it - against the fp64
    product over the oracle's weights, to the fp32 band of the reference (1e-5 of the largest value).  (A slice below
    2^-60 is lifted by 2^64 before the split; it used to count as zero, which left the zero-point term of a 4-bit
    layer standing alone.)"""
    from noeira_amd.qlinear import W8Linear
    rng = np.random.default_rng(int(abs(np.log10(mag))) + len(fmt))
    K, N = 4096, 6403
    if fmt == "q4_0":
        lin = _q4_signed(rng, K, N, prefer_tile=True)
        deq = lin.ref_deq()
    elif fmt == "w4g":
        lin = _w4g_layer(rng, K, N, prefer_tile=True)
        deq = lin.ref_deq()
    else:
        w = rng.integers(-127, 128, (N, K), dtype=np.int8)
        s = rng.uniform(1e-3, 1e-2, N).astype(np.float32)
        lin = W8Linear(K, N, tile_copy=fmt == "w8_tile")
        lin.set_weight(w, s)
        deq = refw.w8(w, s)
    for xdt in (torch.float32, torch.bfloat16):
        x = torch.from_numpy((rng.standard_normal((1, K)) * mag).astype(np.float32)).to(xdt).cuda()
        y = lin.forward(x)
        exact = x.double() @ deq.T
        assert float((y.double() - exact).abs().max()) <= 1e-5 * float(exact.abs().max()), (fmt, mag, xdt)
        yr = lin.forward(x, epilogue="relu")
        assert float((yr.double() - exact.clamp_min(0)).abs().max()) <= 1e-5 * float(exact.abs().max())
