"""A few activation rows (2 .. 16) over a large 4-bit weight: the persistent tile kernel of nq_gemv_tile.hip
(bf16 rows as the matrix core's A rows, fp32 rows as three A rows each), through the C ABI, against fp64 products with
the weights the CPU oracle dequantises from the codes each test drew (tests/refw.py) and against the oracle's own
forward at a size it finishes in seconds.  Bars: 1e-5 of the largest reference value (the reference's fp32 band,
tests/nn/quant/qlinear_common.mojo:39-45); repeated calls return the same bits."""
import numpy as np
import pytest
import torch

from noeira_amd import formats as F
from noeira_amd.qlinear import FusedRows, QLinear, W4GroupLinear
from oracle import oracle as O
import refw

pytestmark = pytest.mark.gpu


def q4_layer(rng, K, N, tile_copy=True):
    lin = QLinear(K, N, tile_copy=tile_copy)
    blocks = rng.integers(0, 256, (N, K // 32, 18), dtype=np.uint8)
    sc = (rng.uniform(1e-3, 1e-2, (N, K // 32)) * rng.choice([-1.0, 1.0], (N, K // 32))).astype(np.float16).view(np.uint16)
    blocks[:, :, 0], blocks[:, :, 1] = sc & 0xFF, sc >> 8
    lin.set_blocks(blocks.reshape(-1))
    lin.ref_deq = lambda: refw.q4_0(blocks, N, K)
    return lin


def w4g_layer(rng, K, N, tile_copy=True):
    G = K // 128
    codes, zps = F.pack_w4g(rng.integers(0, 16, (N, K), dtype=np.uint8), rng.integers(0, 16, (N, G), dtype=np.uint8))
    lin = W4GroupLinear(K, N, 128, tile_copy=tile_copy)
    sg = rng.uniform(1e-3, 1e-2, (N, G)).astype(np.float16)
    lin.set_weight(codes, sg, zps)
    lin.ref_deq = lambda: refw.w4g(codes, sg, zps, N, K, 128)
    return lin


# K = 2048 (one step per wavefront), 2176 (17 steps: a ragged second step), 4096 (two), 5504 (43 steps: three, ragged),
# 6144 (the most the kernel holds); N off the tile size; fewer tiles than CUs and several tiles per workgroup
SHAPES = [(2048, 2051), (2176, 1999), (4096, 1100), (4096, 11008), (5504, 800), (6144, 700)]


@pytest.mark.parametrize("K,N", SHAPES)
@pytest.mark.parametrize("fmt", ["q4_0", "w4g"])
@pytest.mark.parametrize("xdt,M", [(torch.bfloat16, 2), (torch.bfloat16, 7), (torch.bfloat16, 16), (torch.float32, 2),
                                   (torch.float32, 5)])
def test_few_rows_over_tile_copy(K, N, fmt, xdt, M):
    rng = np.random.default_rng(K + N + M + len(fmt))
    lin = q4_layer(rng, K, N) if fmt == "q4_0" else w4g_layer(rng, K, N)
    deq = lin.ref_deq()
    x = torch.from_numpy(rng.standard_normal((M, K)).astype(np.float32)).to(xdt).cuda()
    bias = torch.from_numpy((rng.standard_normal(N) * 0.02).astype(np.float32)).cuda()
    y = lin.forward(x, bias=bias)
    exact = x.double() @ deq.T + bias.double()
    assert y.shape == (M, N)
    assert float((y.double() - exact).abs().max()) <= 1e-5 * float(exact.abs().max())
    assert torch.equal(lin.forward(x, bias=bias), y)
    yr = lin.forward(x, bias=bias.to(torch.bfloat16), epilogue="relu", out_dtype=torch.bfloat16)
    want = (x.double() @ deq.T + bias.to(torch.bfloat16).double()).clamp_min(0)
    rms = float(exact.pow(2).mean().sqrt())
    assert float((yr.double() - want).abs().max()) <= 1e-3 * rms + 2.0 ** -8 * float(want.abs().max())


def test_few_rows_against_oracle_forward():
    rng = np.random.default_rng(17)
    K, N, M = 4096, 1024, 5
    lin = q4_layer(rng, K, N)
    x = rng.standard_normal((M, K)).astype(np.float32)
    y = lin.forward(torch.from_numpy(x).cuda()).cpu().numpy()
    assert O.rel_max(y, O.qlinear_forward_cpu(lin.blocks(), K, N, x)) < 1e-5


def test_few_rows_agree_with_the_row_ordered_kernels_and_with_one_row():
    rng = np.random.default_rng(19)
    K, N, M = 4096, 2048, 4
    a, b = q4_layer(np.random.default_rng(3), K, N), q4_layer(np.random.default_rng(3), K, N, tile_copy=False)
    x = torch.from_numpy(rng.standard_normal((M, K)).astype(np.float32)).to(torch.bfloat16).cuda()
    ya, yb = a.forward(x), b.forward(x)
    assert float((ya - yb).abs().max()) <= 2e-6 * float(yb.abs().max())
    for m in range(M):  # a row of the batch against the same row alone (another kernel: same products, another order)
        y1 = a.forward(x[m:m + 1].contiguous())
        assert float((ya[m] - y1[0]).abs().max()) <= 2e-6 * float(y1.abs().max())


def test_few_rows_fused_parts():
    rng = np.random.default_rng(23)
    K = 4096
    parts = [q4_layer(rng, K, n) for n in (1024, 256, 260)]
    fused = FusedRows(parts)
    x = torch.from_numpy(rng.standard_normal((3, K)).astype(np.float32)).cuda()
    for lin, y in zip(parts, fused.forward(x)):
        want = lin.forward(x)
        assert y.shape == want.shape
        assert float((y - want).abs().max()) <= 2e-6 * float(want.abs().max())


def test_few_rows_nonfinite_stay_in_their_row():
    rng = np.random.default_rng(29)
    K, N, M = 4096, 1040, 6
    lin = w4g_layer(rng, K, N)
    x = torch.from_numpy(rng.standard_normal((M, K)).astype(np.float32)).to(torch.bfloat16).cuda()
    x[2, 100] = float("nan")
    x[4, 7] = float("inf")
    y = lin.forward(x)
    assert bool(torch.isnan(y[2]).all()) and not bool(torch.isnan(y[[0, 1, 3, 5]]).any())
    assert not bool(torch.isfinite(y[4]).any())


# ---- int8 codes: the activation rows as the matrix core's A rows, three int8 terms each under the row's own scale
def w8_layer(rng, K, N, tile_copy=True, prefer_tile=True):
    # (prefer_tile: the kernel wherever it applies, not only on the long-row layers it is dispatched to by default)
    from noeira_amd.qlinear import W8Linear
    w = rng.integers(-127, 128, (N, K), dtype=np.int8)
    w[3, :] = -128  # the one code the symmetric range leaves out
    s = rng.uniform(1e-3, 1e-2, N).astype(np.float32)
    lin = W8Linear(K, N, tile_copy=tile_copy, prefer_tile=prefer_tile and tile_copy)
    lin.set_weight(w, s)
    return lin, w, s


# K = 1024 (one step per wavefront), 1088 (17 steps: a ragged second step), 2048 (two), 3136 (49: four, ragged),
# 4096 (the most the kernel holds); N off the tile size; fewer tiles than CUs and several tiles per workgroup
W8_SHAPES = [(1024, 4100), (1088, 3900), (2048, 2051), (3136, 1400), (4096, 1100), (4096, 11008)]


@pytest.mark.parametrize("K,N", W8_SHAPES)
@pytest.mark.parametrize("xdt,M", [(torch.bfloat16, 2), (torch.bfloat16, 7), (torch.bfloat16, 16), (torch.float32, 2),
                                   (torch.float32, 5), (torch.float32, 16)])
@pytest.mark.parametrize("prefer", [True, False])
def test_few_rows_over_int8_tile_copy(K, N, xdt, M, prefer):
    if not prefer and K < 4096:
        pytest.skip("the default dispatch differs from the preferred one on rows of 3072 codes and more only")
    rng = np.random.default_rng(K + N + M)
    lin, w, s = w8_layer(rng, K, N, prefer_tile=prefer)
    xh = rng.standard_normal((M, K)).astype(np.float32)
    xh[M - 1] *= 1e-3  # a quiet row beside loud ones: every row is split under its own scale
    xh[0, 5] = 40.0    # an outlier 40 sigma out
    x = torch.from_numpy(xh).to(xdt).cuda()
    bias = torch.from_numpy((rng.standard_normal(N) * 0.02).astype(np.float32)).cuda()
    y = lin.forward(x, bias=bias)
    xe = x.float().cpu().numpy()
    exact = O.w8_forward_f64(w, s, xe, np.zeros(N, np.float32))
    assert y.shape == (M, N)
    got = y.cpu().numpy().astype(np.float64) - bias.cpu().numpy().astype(np.float64)
    for m in range(M):  # each row to 1e-5 of its own RMS (the north star's bar is 1e-3)
        assert np.abs(got[m] - exact[m]).max() < 1e-5 * np.sqrt((exact[m] ** 2).mean()) + 1e-7 * np.abs(bias.cpu().numpy()).max()
    assert torch.equal(lin.forward(x, bias=bias), y)
    yr = lin.forward(x, bias=bias.to(torch.bfloat16), epilogue="relu", out_dtype=torch.bfloat16).float().cpu().numpy()
    want = np.maximum(O.w8_forward_f64(w, s, xe, bias.to(torch.bfloat16).float().cpu().numpy()), 0)
    rms = np.sqrt((exact ** 2).mean())
    assert np.abs(yr - want).max() <= 1e-3 * rms + 2.0 ** -8 * np.abs(want).max()


def test_few_rows_int8_agree_with_the_row_ordered_kernels_and_with_one_row():
    rng = np.random.default_rng(31)
    K, N, M = 4096, 2048, 4
    a, _, _ = w8_layer(np.random.default_rng(3), K, N)
    b, _, _ = w8_layer(np.random.default_rng(3), K, N, tile_copy=False)
    x = torch.from_numpy(rng.standard_normal((M, K)).astype(np.float32)).to(torch.bfloat16).cuda()
    ya, yb = a.forward(x), b.forward(x)
    assert float((ya - yb).abs().max()) <= 1e-5 * float(yb.abs().max())
    for m in range(M):
        y1 = a.forward(x[m:m + 1].contiguous())
        assert float((ya[m] - y1[0]).abs().max()) <= 1e-5 * float(y1.abs().max())


def test_few_rows_int8_fused_parts():
    rng = np.random.default_rng(37)
    K = 4096
    parts = [w8_layer(rng, K, n)[0] for n in (1024, 256, 260)]
    fused = FusedRows(parts)
    x = torch.from_numpy(rng.standard_normal((3, K)).astype(np.float32)).cuda()
    for lin, y in zip(parts, fused.forward(x)):
        want = lin.forward(x)
        assert y.shape == want.shape
        assert float((y - want).abs().max()) <= 1e-5 * float(want.abs().max())


def test_few_rows_int8_nonfinite_stay_in_their_row():
    rng = np.random.default_rng(41)
    K, N, M = 4096, 1040, 6
    lin, _, _ = w8_layer(rng, K, N)
    x = torch.from_numpy(rng.standard_normal((M, K)).astype(np.float32)).to(torch.bfloat16).cuda()
    x[2, 100] = float("nan")
    x[4, 7] = float("inf")
    y = lin.forward(x)
    assert bool(torch.isnan(y[2]).all()) and not bool(torch.isnan(y[[0, 1, 3, 5]]).any())
    assert not bool(torch.isfinite(y[4]).any())
