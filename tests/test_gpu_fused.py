"""Row-fused layers (q|k|v, gate|up): `nq_fuse_rows` + `nq_forward_fused` against each part's own
forward and against the oracle.  The caller these serve is the reference's
`DecoderLayerWeights.proj_fwd` (noeira/deep_agents/smolvla/layer_weights.mojo:455-508)."""
import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu

from noeira_amd import _lib as L  # noqa: E402
from noeira_amd import formats as F  # noqa: E402
from noeira_amd.qlinear import FP8Linear, FusedRows, QLinear, W4GroupLinear, W8Linear  # noqa: E402
from oracle import oracle as O  # noqa: E402
import refw  # noqa: E402


def q4_layer(rng, IN, OUT):
    nb = OUT * (IN // 32)
    blocks = rng.integers(0, 256, nb * 18, dtype=np.uint8)
    sc = rng.uniform(1e-3, 2e-3, nb).astype(np.float16).view(np.uint8).reshape(-1, 2)
    blocks.reshape(-1, 18)[:, 0:2] = sc
    ql = QLinear.make(IN, OUT, "gpu")
    ql.set_blocks(blocks)
    return ql, blocks


@pytest.mark.parametrize("M", [1, 3, 135])
@pytest.mark.parametrize("xdt", [torch.float32, torch.bfloat16])
def test_q4_0_qkv_fused_equals_parts(M, xdt):
    rng = np.random.default_rng(700 + M)
    IN, outs = 960, [960, 320, 320]
    layers, blocks = zip(*[q4_layer(rng, IN, n) for n in outs])
    fused = FusedRows(layers)
    assert fused.parts() == 3
    x = torch.from_numpy(rng.standard_normal((M, IN)).astype(np.float32)).cuda().to(xdt)
    ys = fused.forward(x)
    for l, y, b, n in zip(layers, ys, blocks, outs):
        own = l.forward(x)
        assert y.shape == (M, n)
        if M >= 2:
            assert torch.equal(y, own)
        else:
            scale = own.abs().max().item()
            assert (y - own).abs().max().item() <= 2e-6 * scale
        # and the oracle (the reference's band: 1e-5 of max|ref| for fp32 x, 1e-2 for bf16 x)
        xf = x.float().cpu().numpy()
        ref = O.dense_forward_f64(O.dequantize_q4_0(b, n, IN), xf)
        assert np.abs(y.cpu().numpy() - ref).max() <= 1e-5 * np.abs(ref).max()


def test_q4_0_gate_up_fused_and_single_output():
    rng = np.random.default_rng(71)
    IN, M = 960, 135
    (g, gb), (u, ub) = q4_layer(rng, IN, 2560), q4_layer(rng, IN, 2560)
    fused = FusedRows([g, u])
    x = torch.from_numpy(rng.standard_normal((M, IN)).astype(np.float32)).cuda()
    yg, yu = fused.forward(x)
    assert torch.equal(yg, g.forward(x)) and torch.equal(yu, u.forward(x))
    # the fused handle is an ordinary layer too: nq_forward writes one [M, 5120] output
    y = torch.empty((M, 5120), dtype=torch.float32, device="cuda")
    L.check(L.lib().nq_forward(fused._h, x.data_ptr(), L.DT_F32, None, y.data_ptr(), L.DT_F32, M, None, L.DT_F32,
                               L.EPI_NONE, None))
    torch.cuda.synchronize()
    assert torch.equal(y, torch.cat([yg, yu], dim=1))
    # its logical blocks are the parts' blocks, row after row
    out = np.empty(gb.size + ub.size, np.uint8)
    L.check(L.lib().nq_get_blocks(fused._h, out.ctypes.data, out.size))
    assert np.array_equal(out, np.concatenate([gb, ub]))


@pytest.mark.parametrize("M", [1, 100])
def test_w8_fused_with_bias_and_relu(M):
    rng = np.random.default_rng(72 + M)
    IN, outs = 512, [3200, 512, 40]
    layers = []
    for n in outs:
        lin = W8Linear(IN, n)
        lin.set_weight(rng.integers(-127, 128, (n, IN), dtype=np.int8), rng.uniform(1e-3, 1e-2, n).astype(np.float32))
        layers.append(lin)
    fused = FusedRows(layers)
    x = torch.from_numpy(rng.standard_normal((M, IN)).astype(np.float32)).cuda().to(torch.bfloat16)
    bias = torch.from_numpy(rng.standard_normal(sum(outs)).astype(np.float32) * 0.1).cuda()
    ys = fused.forward(x, bias=bias, epilogue="relu")
    r0 = 0
    for l, y, n in zip(layers, ys, outs):
        own = l.forward(x, bias=bias[r0:r0 + n].contiguous(), epilogue="relu")
        if M >= 2:
            assert torch.equal(y, own)
        else:
            assert (y - own).abs().max().item() <= 2e-6 * max(own.abs().max().item(), 1e-30)
        r0 += n


@pytest.mark.parametrize("M", [1, 256])
def test_w4g_fused(M):
    rng = np.random.default_rng(73 + M)
    K, outs = 960, [960, 2560]
    G = -(-K // 128)
    layers = []
    for n in outs:
        lin = W4GroupLinear(K, n, 128)
        lin.set_weight(rng.integers(0, 256, (n, K // 2), dtype=np.uint8),
                       rng.uniform(1e-3, 1e-2, (n, G)).astype(np.float16),
                       F.pack_u4_pairs(rng.integers(0, 16, (n, G), dtype=np.uint8)))
        layers.append(lin)
    fused = FusedRows(layers)
    x = torch.from_numpy(rng.standard_normal((M, K)).astype(np.float32)).cuda().to(torch.bfloat16)
    for l, y in zip(layers, fused.forward(x)):
        own = l.forward(x)
        if M >= 2:
            assert torch.equal(y, own)
        else:
            assert (y - own).abs().max().item() <= 2e-6 * own.abs().max().item()


@pytest.mark.parametrize("M", [1, 9, 64])
def test_fp8_fused_runs_part_by_part(M):
    """fp8 x fp8 has no part-placing kernel: the fused call launches once per part on a view of
    its rows, so every output is bit for bit the part's own."""
    rng = np.random.default_rng(74 + M)
    K, outs = 1024, [256, 48]
    layers = []
    for n in outs:
        lin = FP8Linear(K, n)
        lin.set_weight(F.encode_e4m3(rng.standard_normal((n, K)).astype(np.float32)), 0.25)
        layers.append(lin)
    fused = FusedRows(layers)
    x = torch.from_numpy(F.encode_e4m3(rng.standard_normal((M, K)).astype(np.float32))).cuda()
    xs = torch.tensor([0.5], dtype=torch.float32, device="cuda")
    ys = fused.forward(x, x_scale=xs, out_dtype=torch.bfloat16)
    for l, y in zip(layers, ys):
        assert torch.equal(y, l.forward(x, xs))


def test_fuse_rows_errors():
    rng = np.random.default_rng(75)
    a, _ = q4_layer(rng, 64, 8)
    b, _ = q4_layer(rng, 96, 8)
    with pytest.raises(L.NQError, match="share format, IN"):
        FusedRows([a, b])
    empty = QLinear.make(64, 8, "gpu")
    with pytest.raises(L.NQError, match="no weights"):
        FusedRows([a, empty])
    c, _ = q4_layer(rng, 64, 16)
    f = FusedRows([a, c])
    with pytest.raises(L.NQError, match="cannot be fused again"):
        FusedRows([f, a])
    x = torch.zeros((2, 64), dtype=torch.float32, device="cuda")
    with pytest.raises(L.NQError, match="1 outputs for a layer of 2 fused parts"):
        f.forward(x, outs=[torch.empty((2, 24), dtype=torch.float32, device="cuda")])
    with pytest.raises(L.NQError, match="between 1 and 4"):
        FusedRows([a, a, a, a, a])


@pytest.mark.parametrize("M", [256, 300, 400, 511])
def test_parts_keep_their_bits_between_the_medium_and_the_many_rows_kernel(M):
    """From 256 rows on the many-rows kernel takes a layer where its estimated time is the lower one: wide layers
    first.  Below 512 rows a row-fused layer follows its parts: a wide and a narrow part run part by part, two wide
    ones in one launch, and every part returns the bits of its own layer's forward (and those agree with the fp64
    product of the dequantised weights)."""
    rng = np.random.default_rng(M)
    K = 1024
    x = torch.from_numpy(rng.standard_normal((M, K)).astype(np.float32)).to(torch.bfloat16).cuda()

    def w8(n):
        lin = W8Linear(K, n)
        wq, ws = rng.integers(-127, 128, (n, K), dtype=np.int8), rng.uniform(1e-3, 1e-2, n).astype(np.float32)
        lin.set_weight(wq, ws)
        lin.ref_deq = lambda: refw.w8(wq, ws)
        return lin

    def q4(n):
        lin = QLinear(K, n, tile_copy=False)
        blocks = rng.integers(0, 256, (n, K // 32, 18), dtype=np.uint8)
        sc = rng.uniform(1e-3, 1e-2, (n, K // 32)).astype(np.float16).view(np.uint16)
        blocks[:, :, 0], blocks[:, :, 1] = sc & 0xFF, sc >> 8
        lin.set_blocks(blocks.reshape(-1))
        lin.ref_deq = lambda: refw.q4_0(blocks, n, K)
        return lin

    for make in (w8, q4):
        for widths in ((8192, 512), (8192, 6144), (512, 640)):
            parts = [make(n) for n in widths]
            fused = FusedRows(parts)
            outs = fused.forward(x)
            for part, y in zip(parts, outs):
                own = part.forward(x)
                assert torch.equal(y, own), (make.__name__, widths, part.OUT)
                exact = x.double() @ part.ref_deq().T
                assert float((own.double() - exact).abs().max()) <= 1e-5 * float(exact.abs().max())
            if make is w8:  # bias and ReLU travel with each part when the call runs part by part
                bias = torch.from_numpy(rng.standard_normal(sum(widths)).astype(np.float32)).cuda()
                r0 = 0
                for part, y in zip(parts, fused.forward(x, bias=bias, epilogue="relu")):
                    assert torch.equal(y, part.forward(x, bias=bias[r0:r0 + part.OUT].contiguous(), epilogue="relu"))
                    r0 += part.OUT
