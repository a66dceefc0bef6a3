"""Tens to hundreds of activation rows over 4-bit codes: the M-tile kernel of nq_gemv_tile.hip (a workgroup keeps
the A operands of 16 activation rows in registers and walks the 16-row weight tiles of the tile-ordered copy),
through the C ABI.  The reference's caller runs exactly this regime: T = 135 tokens over 960 -> 960 / 320 / 2560 and
2560 -> 960 (noeira/deep_agents/smolvla/fused.mojo:255-384), its gate tests/nn/quant/test_qlinear_gpu.mojo.  Against
the oracle's forward (1e-5 of the largest reference value, tests/nn/quant/qlinear_common.mojo:39-45), against fp64
over the oracle's dequantised weights (tests/refw.py, from the codes each test drew) for every K split the kernel has, row-fused parts and the SwiGLU epilogue included;
repeated calls return the same bits; a row-fused layer returns the bits of its parts' own forwards."""
import numpy as np
import pytest
import torch

from noeira_amd import formats as F
from noeira_amd.qlinear import FusedGLU, FusedRows, QLinear, W4GroupLinear
from oracle import oracle as O
import refw

pytestmark = pytest.mark.gpu


def q4_layer(rng, K, N, tile_copy=True):
    # (prefer_tile: the M-tile kernel wherever it applies, not only on the wide layers it is dispatched to by default)
    lin = QLinear(K, N, tile_copy=tile_copy, prefer_tile=True)
    blocks = rng.integers(0, 256, (N, K // 32, 18), dtype=np.uint8)
    sc = (rng.uniform(1e-3, 1e-2, (N, K // 32)) * rng.choice([-1.0, 1.0], (N, K // 32))).astype(np.float16).view(np.uint16)
    blocks[:, :, 0], blocks[:, :, 1] = sc & 0xFF, sc >> 8
    lin.set_blocks(blocks.reshape(-1))
    lin.ref_deq = lambda: refw.q4_0(blocks, N, K)
    return lin


def w4g_layer(rng, K, N, tile_copy=True):
    G = -(-K // 128)
    codes, zps = F.pack_w4g(rng.integers(0, 16, (N, K), dtype=np.uint8), rng.integers(0, 16, (N, G), dtype=np.uint8))
    lin = W4GroupLinear(K, N, 128, tile_copy=tile_copy, prefer_tile=True)
    sg = rng.uniform(1e-3, 1e-2, (N, G)).astype(np.float16)
    lin.set_weight(codes, sg, zps)
    lin.ref_deq = lambda: refw.w4g(codes, sg, zps, N, K, 128)
    return lin


@pytest.mark.parametrize("IN,OUT", [(960, 960), (960, 320), (960, 2560), (2560, 960)])
@pytest.mark.parametrize("M", [135, 17])
def test_reference_shapes_against_the_oracle(IN, OUT, M):
    rng = np.random.default_rng(IN + OUT + M)
    lin = QLinear(IN, OUT, prefer_tile=True)
    lin.set_weight((rng.standard_normal((OUT, IN)) * 0.05).astype(np.float32))
    x = rng.standard_normal((M, IN)).astype(np.float32)
    want = O.qlinear_forward_cpu(lin.blocks(), IN, OUT, x)
    if IN <= 2048:   # fp32 activations: three exact bf16 terms (IN <= 2048: beyond, the 16-row tile kernel of medium M)
        y = lin.forward(torch.from_numpy(x).cuda())
        assert O.rel_max(y.cpu().numpy(), want) < 1e-5
        assert torch.equal(lin.forward(torch.from_numpy(x).cuda()), y)
    xb = torch.from_numpy(x).to(torch.bfloat16)
    want_b = O.qlinear_forward_cpu(lin.blocks(), IN, OUT, xb.float().numpy())
    yb = lin.forward(xb.cuda())
    assert O.rel_max(yb.cpu().numpy(), want_b) < 1e-5     # bf16 activations are exact operands: the fp32 band holds


# every K split: NJ = 4 (KW 4, 4 groups), 5, 8 (KW 8, 2 groups; 960 = 7.5 steps: a half step of padding), 16, 17
# (JPW 2), 20 (JPW 3, KW 7), 32, 33, 43, 48 (the most the registers hold); N off the tile size, fewer weight tiles
# than workgroups, several per workgroup; M off the tile size
SHAPES = [(512, 777), (640, 100), (960, 1000), (992, 48), (2048, 531), (2176, 300), (2560, 960), (4096, 1100),
          (4224, 200), (5504, 160), (6144, 90)]


@pytest.mark.parametrize("K,N", SHAPES)
@pytest.mark.parametrize("fmt", ["q4_0", "w4g"])
@pytest.mark.parametrize("xdt,M", [(torch.bfloat16, 17), (torch.bfloat16, 100), (torch.bfloat16, 256), (torch.float32, 40),
                                   (torch.float32, 135)])
def test_m_tiles_over_tile_copy(K, N, fmt, xdt, M):
    rng = np.random.default_rng(K + N + M + len(fmt))
    lin = q4_layer(rng, K, N) if fmt == "q4_0" else w4g_layer(rng, K, N)
    deq = lin.ref_deq()
    x = torch.from_numpy(rng.standard_normal((M, K)).astype(np.float32)).to(xdt).cuda()
    bias = torch.from_numpy((rng.standard_normal(N) * 0.02).astype(np.float32)).cuda()
    y = torch.full((M, N), float("nan"), device="cuda")
    lin.forward(x, bias=bias, out=y)
    exact = x.double() @ deq.T + bias.double()
    assert float((y.double() - exact).abs().max()) <= 1e-5 * float(exact.abs().max())
    assert torch.equal(lin.forward(x, bias=bias), y)
    yr = lin.forward(x, bias=bias.to(torch.bfloat16), epilogue="relu", out_dtype=torch.bfloat16)
    want = (x.double() @ deq.T + bias.to(torch.bfloat16).double()).clamp_min(0)
    rms = float(exact.pow(2).mean().sqrt())
    assert float((yr.double() - want).abs().max()) <= 1e-3 * rms + 2.0 ** -8 * float(want.abs().max())
    # the kernel that reads the row-ordered codes: the same products, another order
    other = (q4_layer if fmt == "q4_0" else w4g_layer)(np.random.default_rng(K + N + M + len(fmt)), K, N, tile_copy=False)
    yo = other.forward(x, bias=bias)
    assert float((y - yo).abs().max()) <= 4e-6 * float(yo.abs().max())


@pytest.mark.parametrize("xdt", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("M", [24, 135])
def test_row_fused_parts_and_glu(M, xdt):
    """q | k | v through the part table and gate | up with the SwiGLU epilogue, on the M-tile kernel: every part
    the bits of its own forward, the GLU output within the band of fp64 over the dequantised weights."""
    rng = np.random.default_rng(M)
    IN = 960
    q, k, v = q4_layer(rng, IN, 960), q4_layer(rng, IN, 320), q4_layer(rng, IN, 320)
    x = torch.from_numpy(rng.standard_normal((M, IN)).astype(np.float32)).to(xdt).cuda()
    outs = FusedRows([q, k, v]).forward(x)
    for part, y in zip((q, k, v), outs):
        assert torch.equal(y, part.forward(x))
    gate, up = q4_layer(rng, IN, 2560), q4_layer(rng, IN, 2560)
    g = x.double() @ gate.ref_deq().T
    u = x.double() @ up.ref_deq().T
    want = u * (g * torch.sigmoid(g))
    glu = FusedGLU(gate, up)
    y = glu.forward(x)
    assert float((y.double() - want).abs().max()) <= 1e-5 * float(want.abs().max())
    assert torch.equal(glu.forward(x), y)
    yb = glu.forward(x, out_dtype=torch.bfloat16)
    assert float((yb.double() - want).abs().max()) <= (2.0 ** -8 + 1e-5) * float(want.abs().max())


def test_default_dispatch_keeps_fused_parts_bitwise():
    """By default the M-tile kernel takes layers 2048 wide and more where its estimated time is the lower one, and a
    row-fused layer part by part: gate | up (2560 | 2560) and each of the two alone run on it at T = 135, q | k | v
    (960 | 320 | 320) and its parts do not; either way every part of the fused launch carries the bits of its own
    forward."""
    rng = np.random.default_rng(77)
    M, IN = 135, 960
    mk = lambda n: QLinear.from_linear((rng.standard_normal((IN, n)) * 0.05).astype(np.float32))
    for xdt in (torch.float32, torch.bfloat16):
        x = torch.from_numpy(rng.standard_normal((M, IN)).astype(np.float32)).to(xdt).cuda()
        for widths in ([2560, 2560], [960, 320, 320], [2560, 320]):
            parts = [mk(n) for n in widths]
            for part, y in zip(parts, FusedRows(parts).forward(x)):
                assert torch.equal(y, part.forward(x))


def test_default_dispatch_below_a_hundred_rows_over_large_layers():
    """Below a hundred rows the M-tile kernel takes a call by default over the widest layers (2048 -> 11008 here;
    2048 -> 2048 stays on the 16-row tile kernel): against fp64 over the dequantised weights, and a row-fused layer of
    a large and a small part returns the bits of each part's own forward."""
    rng = np.random.default_rng(83)
    K, M = 2048, 33
    x = torch.from_numpy(rng.standard_normal((M, K)).astype(np.float32)).to(torch.bfloat16).cuda()
    big, small = QLinear(K, 11008), QLinear(K, 2048)
    for lin in (big, small):
        blocks = rng.integers(0, 256, (lin.OUT, K // 32, 18), dtype=np.uint8)
        sc = rng.uniform(1e-3, 1e-2, (lin.OUT, K // 32)).astype(np.float16).view(np.uint16)
        blocks[:, :, 0], blocks[:, :, 1] = sc & 0xFF, sc >> 8
        lin.set_blocks(blocks.reshape(-1))
        y = lin.forward(x)
        exact = x.double() @ refw.q4_0(blocks, lin.OUT, K).T
        assert float((y.double() - exact).abs().max()) <= 1e-5 * float(exact.abs().max())
        assert torch.equal(lin.forward(x), y)
    for part, y in zip((big, small), FusedRows([big, small]).forward(x)):
        assert torch.equal(y, part.forward(x))


@pytest.mark.parametrize("M", [100, 135, 200])
def test_default_dispatch_at_a_hundred_rows_follows_each_parts_own_rule(M):
    """The choice between the M-tile kernel and the medium-M one follows each part's own width and the row count
    (the two kernels' estimated times): a row-fused layer whose parts may fall on different sides - IN = 2048 with
    parts 2560 and 8192 wide, and IN = 2560 (three steps of K per wavefront) with 2560 and 5120 - returns the bits of
    each part's own forward, and those are within the band of the fp64 product."""
    rng = np.random.default_rng(91 + M)
    for K, outs in ((2048, (2560, 8192)), (2560, (2560, 5120))):
        x = torch.from_numpy(rng.standard_normal((M, K)).astype(np.float32)).to(torch.bfloat16).cuda()
        parts = [QLinear(K, n) for n in outs]
        for lin in parts:
            blocks = rng.integers(0, 256, (lin.OUT, K // 32, 18), dtype=np.uint8)
            sc = rng.uniform(1e-3, 1e-2, (lin.OUT, K // 32)).astype(np.float16).view(np.uint16)
            blocks[:, :, 0], blocks[:, :, 1] = sc & 0xFF, sc >> 8
            lin.set_blocks(blocks.reshape(-1))
            y = lin.forward(x)
            exact = x.double() @ refw.q4_0(blocks, lin.OUT, K).T
            assert float((y.double() - exact).abs().max()) <= 1e-5 * float(exact.abs().max())
            assert torch.equal(lin.forward(x), y)
        for part, y in zip(parts, FusedRows(parts).forward(x)):
            assert torch.equal(y, part.forward(x))


@pytest.mark.parametrize("fmt,K,N,M,xdt", [
    ("q4_0", 2048, 11008, 33, torch.float32),    # fp32 activations below a hundred rows over the widest layers
    ("w4g", 1280, 8192, 48, torch.float32),
    ("q4_0", 960, 8192, 384, torch.bfloat16),    # bf16 activations beyond 256 rows
    ("w4g", 2048, 11008, 500, torch.bfloat16),
    ("w4g", 2560, 4096, 96, torch.bfloat16),     # three steps of K per wavefront at a hundred rows
    ("q4_0", 3072, 5120, 160, torch.bfloat16),
    ("q4_0", 960, 2560, 511, torch.float32),     # the last row count before the many-rows kernel
])
def test_default_dispatch_by_estimate(fmt, K, N, M, xdt):
    """Calls whose kernel changed when the dispatch went from row-count and width thresholds to the two kernels'
    estimated times: whichever takes them, the result is within the fp32 band of the fp64 product over the
    dequantised weights, repeats bit for bit, and a row-fused layer of two such parts returns each part's own bits."""
    rng = np.random.default_rng(K + N + M)
    def layer(n):
        if fmt == "q4_0":
            lin = QLinear(K, n)
            blocks = rng.integers(0, 256, (n, K // 32, 18), dtype=np.uint8)
            sc = rng.uniform(1e-3, 1e-2, (n, K // 32)).astype(np.float16).view(np.uint16)
            blocks[:, :, 0], blocks[:, :, 1] = sc & 0xFF, sc >> 8
            lin.set_blocks(blocks.reshape(-1))
            lin.ref_deq = lambda: refw.q4_0(blocks, n, K)
            return lin
        G = -(-K // 128)
        codes, zps = F.pack_w4g(rng.integers(0, 16, (n, K), dtype=np.uint8), rng.integers(0, 16, (n, G), dtype=np.uint8))
        lin = W4GroupLinear(K, n, 128)
        sg = rng.uniform(1e-3, 1e-2, (n, G)).astype(np.float16)
        lin.set_weight(codes, sg, zps)
        lin.ref_deq = lambda: refw.w4g(codes, sg, zps, n, K, 128)
        return lin
    x = torch.from_numpy(rng.standard_normal((M, K)).astype(np.float32)).to(xdt).cuda()
    big, small = layer(N), layer(960)
    for lin in (big, small):
        y = lin.forward(x)
        exact = x.double() @ lin.ref_deq().T
        assert float((y.double() - exact).abs().max()) <= 1e-5 * float(exact.abs().max())
        assert torch.equal(lin.forward(x), y)
    for part, y in zip((big, small), FusedRows([big, small]).forward(x)):
        assert torch.equal(y, part.forward(x))
