"""The int8 / uint4-group / fp8 layers BASELINE's configs name, on the GPU
through the C ABI, against the CPU oracle on identical seeded inputs.

The reference implements none of these formats, so the oracle's closed forms
(pinned in tests/test_oracle_ext.py) are the checker.  Bars: int32 accumulators
bit-exact; fp32/bf16 outputs max-abs-err <= 1e-3 * RMS(exact output);
fp8 <= 1e-2 * RMS.  At sizes the oracle cannot finish in seconds, parity is
shown through size-independent properties (linearity in the activations, a
row/column sample checked exactly, agreement between the GEMV and GEMM paths).
"""
import numpy as np
import pytest
import torch

from noeira_amd import formats as F
from noeira_amd.qlinear import FP8Linear, W4GroupLinear, W8Linear, quantize_rows_i8
from oracle import oracle as O

pytestmark = pytest.mark.gpu

TOL_RMS = 1e-3
TOL_RMS_FP8 = 1e-2


def rel_rms(a, b):
    b = np.asarray(b, np.float64)
    return np.abs(np.asarray(a, np.float64) - b).max() / max(np.sqrt((b ** 2).mean()), 1e-300)


def bf16(x):
    return torch.from_numpy(np.ascontiguousarray(x, np.float32)).to(torch.bfloat16)


def w8_layer(rng, K, N):
    w = rng.integers(-127, 128, (N, K), dtype=np.int8)
    s = rng.uniform(1e-3, 1e-2, N).astype(np.float32)
    lin = W8Linear(K, N)
    lin.set_weight(w, s)
    return lin, w, s


# ── config 1: W8A32, M=1, K=256, N=256 (SAC actor hidden layer), zero bias ─────
def test_config1_w8a32_sac_hidden():
    rng = np.random.default_rng(1)
    lin, w, s = w8_layer(rng, 256, 256)
    x = rng.standard_normal((1, 256)).astype(np.float32)
    bias = np.zeros(256, np.float32)
    y = lin.forward(torch.from_numpy(x).cuda(), bias=torch.from_numpy(bias).cuda()).cpu().numpy()
    exact = O.w8_forward_f64(w, s, x, bias)
    assert rel_rms(y, exact) < TOL_RMS
    assert rel_rms(y, O.w8_forward_f32(w, s, x, bias)) < TOL_RMS
    # the integer-activation reading: per-token int8 x, int32 accumulate (bit-exact), then scale
    xq, sx = quantize_rows_i8(torch.from_numpy(x).cuda())
    xq_o, sx_o = O.quantize_rows_i8(x)
    assert np.array_equal(xq.cpu().numpy(), xq_o) and np.array_equal(sx.cpu().numpy(), sx_o)
    acc = lin.forward_a8(xq, sx, out_dtype=torch.int32).cpu().numpy()
    assert np.array_equal(acc, O.w8a8_acc_i32(xq_o, w))
    y8 = lin.forward_a8(xq, sx).cpu().numpy()
    assert rel_rms(y8, O.w8a8_epilogue(O.w8a8_acc_i32(xq_o, w), sx_o, s)) < 1e-6


# ── config 2: ACT policy MLP, W8A16, M in {1, 100}, bf16 bias, fp32 out ────────
@pytest.mark.parametrize("M", [1, 100])
@pytest.mark.parametrize("K,N", [(512, 3200), (3200, 512)])
def test_config2_w8a16_act_mlp(K, N, M):
    rng = np.random.default_rng(K + N + M)
    lin, w, s = w8_layer(rng, K, N)
    xb = bf16(rng.standard_normal((M, K)))
    bb = bf16(rng.standard_normal(N) * 0.02)
    y = lin.forward(xb.cuda(), bias=bb.cuda()).cpu().numpy()
    assert y.dtype == np.float32 and y.shape == (M, N)
    exact = O.w8_forward_f64(w, s, xb.float().numpy(), bb.float().numpy())
    assert rel_rms(y, exact) < TOL_RMS, rel_rms(y, exact)
    # ReLU epilogue and bf16 output
    yr = lin.forward(xb.cuda(), bias=bb.cuda(), epilogue="relu", out_dtype=torch.bfloat16).float().cpu().numpy()
    want = bf16(np.maximum(exact, 0).astype(np.float32)).float().numpy()
    assert np.abs(yr - want).max() <= np.abs(want).max() * 2.0 ** -7  # one bf16 ulp of the largest value


# ── config 3: VLM block, W4A16 group 128 asymmetric, M in {1, 256} ────────────
W4_SHAPES = [(960, 960), (960, 2560), (2560, 960)]


@pytest.mark.parametrize("M", [1, 256])
@pytest.mark.parametrize("K,N", W4_SHAPES)
def test_config3_w4a16_group128(K, N, M):
    rng = np.random.default_rng(K * 3 + N + M)
    group = 128
    G = -(-K // group)
    assert (K, G) != (960, 8) or K % group == 64      # the ragged 8th group (64 wide)
    q = rng.integers(0, 16, (N, K), dtype=np.uint8)
    z = rng.integers(0, 16, (N, G), dtype=np.uint8)
    sc = rng.uniform(1e-3, 1e-2, (N, G)).astype(np.float16)
    codes, zps = F.pack_w4g(q, z)
    lin = W4GroupLinear(K, N, group)
    lin.set_weight(codes, sc, zps)
    deq = O.w4g_dequantize(codes, sc.view(np.uint16), zps, N, K, group)
    assert np.array_equal(lin.dequantized_dev().cpu().numpy().view(np.uint32), deq.view(np.uint32))
    xb = bf16(rng.standard_normal((M, K)))
    y = lin.forward(xb.cuda()).cpu().numpy()
    exact = O.dense_forward_f64(deq, xb.float().numpy())
    assert rel_rms(y, exact) < TOL_RMS, rel_rms(y, exact)


def test_config3_quantized_from_gaussian_weights():
    """The same path on weights produced by the host quantiser (not random codes)."""
    rng = np.random.default_rng(33)
    K, N = 960, 320
    w = (rng.standard_normal((N, K)) * 0.05).astype(np.float32)
    q, sc, z = F.quantize_w4g_asym(w, 128)
    codes, zps = F.pack_w4g(q, z)
    lin = W4GroupLinear(K, N, 128)
    lin.set_weight(codes, sc, zps)
    deq = O.w4g_dequantize(codes, sc.view(np.uint16), zps, N, K, 128)
    assert np.abs(deq - w).max() <= 0.51 * sc.astype(np.float32).max()
    xb = bf16(rng.standard_normal((3, K)))
    assert rel_rms(lin.forward(xb.cuda()).cpu().numpy(), O.dense_forward_f64(deq, xb.float().numpy())) < TOL_RMS


# ── config 4: batched-env actor, W8A8, M=4096, 64 -> 256 -> 256 -> 8, ReLU ─────
def actor_layers(rng):
    dims = [(64, 256), (256, 256), (256, 8)]
    layers = []
    for K, N in dims:
        lin, w, s = w8_layer(rng, K, N)
        b = (rng.standard_normal(N) * 0.02).astype(np.float32)
        layers.append((lin, w, s, b))
    return layers


def oracle_actor(layers, x):
    """Layer by layer: per-token int8, exact int32 accumulate, relu(sx*sw*acc + b)."""
    h = x
    accs = []
    for i, (_, w, s, b) in enumerate(layers):
        hq, sx = O.quantize_rows_i8(h)
        acc = O.w8a8_acc_i32(hq, w)
        accs.append((hq, sx, acc))
        h = O.w8a8_epilogue(acc, sx, s, b, relu=(i < 2))
    return h, accs


def test_config4_w8a8_actor_layer_by_layer():
    rng = np.random.default_rng(4)
    layers = actor_layers(rng)
    M = 4096
    x = rng.standard_normal((M, 64)).astype(np.float32)
    want, accs = oracle_actor(layers, x)
    h = torch.from_numpy(x).cuda()
    for i, (lin, w, s, b) in enumerate(layers):
        hq, sx = quantize_rows_i8(h)
        hq_o, sx_o, acc_o = accs[i]
        if i == 0:  # identical inputs: the quantiser and the accumulators are bit-exact
            assert np.array_equal(hq.cpu().numpy(), hq_o) and np.array_equal(sx.cpu().numpy(), sx_o)
            acc = lin.forward_a8(hq, sx, out_dtype=torch.int32).cpu().numpy()
            assert np.array_equal(acc, acc_o)
        else:       # fed the oracle's codes, the accumulators are bit-exact at every layer
            acc = lin.forward_a8(torch.from_numpy(hq_o).cuda(), torch.from_numpy(sx_o).cuda(),
                                 out_dtype=torch.int32).cpu().numpy()
            assert np.array_equal(acc, acc_o)
        h = lin.forward_a8(hq, sx, bias=torch.from_numpy(b).cuda(), epilogue="relu" if i < 2 else "none")
    assert rel_rms(h.cpu().numpy(), want) < TOL_RMS


def test_quantize_rows_i8_edges():
    rng = np.random.default_rng(44)
    x = rng.standard_normal((37, 256)).astype(np.float32)
    x[3] = 0.0
    x[4] = 0.5 * np.arange(256, dtype=np.float32) - 64
    x[4, 0] = -127.0     # scale exactly 1: the halves are exact ties
    q, s = quantize_rows_i8(torch.from_numpy(x).cuda())
    q_o, s_o = O.quantize_rows_i8(x)
    assert np.array_equal(q.cpu().numpy(), q_o) and np.array_equal(s.cpu().numpy().view(np.uint32), s_o.view(np.uint32))
    qb, sb = quantize_rows_i8(bf16(x).cuda())
    q_o, s_o = O.quantize_rows_i8(bf16(x).float().numpy())
    assert np.array_equal(qb.cpu().numpy(), q_o) and np.array_equal(sb.cpu().numpy(), s_o)


# ── config 5: fp8 e4m3 x fp8 e4m3, per-tensor scales, fp32 accumulate, bf16 out ─
def fp8_operands(rng, M, N, K):
    a = F.encode_e4m3(rng.standard_normal((M, K)).astype(np.float32))
    b = F.encode_e4m3(rng.standard_normal((N, K)).astype(np.float32))
    return a, b


def test_encode_e4m3_host_matches_oracle():
    rng = np.random.default_rng(50)
    x = (rng.standard_normal(50000) * 3).astype(np.float32)
    x[:10] = [500, -500, 448, -448, 0, 1e-9, 2 ** -9, 2 ** -10, 0.0625, -0.0625]
    assert np.array_equal(F.encode_e4m3(x), O.e4m3_encode(np.clip(x, -448, 448)))


@pytest.mark.parametrize("M", [1, 7, 16, 17, 40, 63, 64])
def test_config5_fp8_reduced_size_vs_oracle(M):
    rng = np.random.default_rng(5 + M)
    N, K = (504 if M in (7, 17, 63) else 512), 4096  # 504 = 31.5 row tiles of 16
    a, b = fp8_operands(rng, M, N, K)
    sa, sb = np.float32(0.731), np.float32(1.37)
    lin = FP8Linear(K, N)
    lin.set_weight(b, float(sb))
    xs = torch.tensor([sa], dtype=torch.float32, device="cuda")
    y = lin.forward(torch.from_numpy(a).cuda(), xs)
    assert y.dtype == torch.bfloat16
    y64, ybf = O.fp8_forward_f64(a, b, sa, sb)
    # The bar (1e-2 of RMS) is applied to the fp32 accumulator-times-scale value.  bf16 itself
    # carries up to 2^-8 relative rounding, i.e. up to 1.5e-2 of RMS on a 4-sigma output, so the
    # bf16 output is held to a tighter, exact statement instead: it is the round-to-nearest-even
    # bf16 of that fp32 value.
    yf = lin.forward(torch.from_numpy(a).cuda(), xs, out_dtype=torch.float32).cpu().numpy()
    assert rel_rms(yf, y64) < TOL_RMS_FP8
    # far inside the bar: the matrix cores add fp8 products in fp32 (their internal alignment
    # costs a little against a serial fp32 chain: ~6e-5 of RMS at K = 4096)
    assert rel_rms(yf, y64) < 3e-4
    gb = y.view(torch.int16).cpu().numpy().view(np.uint16)
    assert np.array_equal(gb, O.bf16_bits(yf))
    # and so it sits within bf16's own half-step (2^-9 relative) of the exact value, plus the
    # accumulation error above
    rms = np.sqrt((y64 ** 2).mean())
    assert (np.abs(O.bf16_value(gb).astype(np.float64) - y64) <= np.abs(y64) * 2.0 ** -8 + 3e-4 * rms).all()


def test_config5_fp8_gemv_full_size_sampled():
    """M = 1 at the full K = 4096, N = 11008: every output against the oracle
    (45 MB of weights, 45 MFLOP: the oracle finishes in well under a second)."""
    rng = np.random.default_rng(55)
    N, K = 11008, 4096
    a, b = fp8_operands(rng, 1, N, K)
    lin = FP8Linear(K, N)
    lin.set_weight(b, 1.0)
    xs = torch.ones(1, dtype=torch.float32, device="cuda")
    y = lin.forward(torch.from_numpy(a).cuda(), xs, out_dtype=torch.float32).cpu().numpy()
    y64, _ = O.fp8_forward_f64(a, b, 1.0, 1.0, want_bf16=False)
    assert rel_rms(y, y64) < 3e-4  # MFMA fp32 accumulation; the bar is 1e-2
    # repeated calls return the same bits (fixed-order K split)
    y2 = lin.forward(torch.from_numpy(a).cuda(), xs, out_dtype=torch.float32).cpu().numpy()
    assert np.array_equal(y.view(np.uint32), y2.view(np.uint32))


@pytest.mark.parametrize("M,K,N", [(1, 128, 16), (3, 384, 40), (16, 2560, 100), (2, 8192, 33),
                                   (1, 784, 37), (1, 1024, 5), (1, 2576, 130), (1, 8192, 19), (1, 8208, 9),
                                   (3, 400, 40), (40, 1040, 100), (200, 16, 24), (1, 48, 7),
                                   (300, 960, 2600), (130, 1040, 2600), (520, 1024, 1288)])
def test_fp8_small_m_bias_relu_and_shapes(M, K, N):
    """fp8 x fp8 at 1..520 rows: ragged N, K from a fraction of one MFMA step to several rounds of the K split,
    fp32 bias and ReLU fused; checked against the float64 oracle.  The last three take the tile kernel with
    four, two and four weight tiles per workgroup (K 64 short of a step, 16 past one, a multiple of it)."""
    rng = np.random.default_rng(1000 + M + K)
    a, b = fp8_operands(rng, M, N, K)
    sa, sb = np.float32(0.5), np.float32(0.25)
    bias = rng.standard_normal(N).astype(np.float32)
    lin = FP8Linear(K, N)
    lin.set_weight(b, float(sb))
    xs = torch.tensor([sa], dtype=torch.float32, device="cuda")
    y = lin.forward(torch.from_numpy(a).cuda(), xs, bias=torch.from_numpy(bias).cuda(), epilogue="relu",
                    out_dtype=torch.float32).cpu().numpy()
    y64, _ = O.fp8_forward_f64(a, b, sa, sb, want_bf16=False)
    ref = np.maximum(y64 + bias.astype(np.float64), 0.0)
    rms = np.sqrt(((y64 + bias) ** 2).mean())
    assert np.abs(y - ref).max() <= 3e-4 * rms


@pytest.mark.parametrize("N", [4096, 11008])
def test_config5_fp8_gemm_full_size_sampled(N):
    """M = 8192, K = 4096 at full size through the MFMA GEMM.  The oracle cannot
    do 2.7e11 MACs in seconds, so parity is checked (a) on a seeded sample of
    whole rows, against the oracle, (b) on every element for holes (pre-poisoned
    output), (c) against the M = 1 GEMV path on the same rows."""
    M, K = 8192, 4096
    g = torch.Generator().manual_seed(N)
    b = torch.randn((N, K), generator=g).clamp_(-448, 448).to(torch.float8_e4m3fn).view(torch.uint8)
    a = torch.randn((M, K), generator=g).clamp_(-448, 448).to(torch.float8_e4m3fn).view(torch.uint8)
    sa, sb = np.float32(0.5), np.float32(0.25)
    lin = FP8Linear(K, N)
    lin.set_weight(b.numpy(), float(sb))
    xs = torch.tensor([sa], dtype=torch.float32, device="cuda")
    ad = a.cuda()
    yf = torch.full((M, N), float("nan"), dtype=torch.float32, device="cuda")
    lin.forward(ad, xs, out=yf, out_dtype=torch.float32)
    assert not torch.isnan(yf).any()
    ybf = lin.forward(ad, xs)
    assert torch.equal(ybf, yf.to(torch.bfloat16))          # bf16 output = RNE of the fp32 value
    rows = np.random.default_rng(N).choice(M, 24, replace=False)
    rows[:4] = [0, 255, 256, M - 1]
    y64, _ = O.fp8_forward_f64(a.numpy()[rows], b.numpy(), sa, sb, want_bf16=False)
    got = yf[torch.from_numpy(rows).cuda()].cpu().numpy()
    assert rel_rms(got, y64) < TOL_RMS_FP8
    assert rel_rms(got, y64) < 3e-4
    gemv = lin.forward(ad[int(rows[5])].reshape(1, K).contiguous(), xs, out_dtype=torch.float32).cpu().numpy()
    assert rel_rms(gemv, y64[5:6]) < 3e-4


@pytest.mark.parametrize("M,K,N", [(4096, 256, 256), (300, 384, 520), (64, 128, 8), (1000, 1024, 264),
                                   (5, 128, 24), (63, 4096, 100), (1, 512, 48),
                                   (4096, 64, 256), (300, 960, 520), (5, 80, 24), (70, 16, 40),
                                   (1, 784, 37), (1, 4096, 130), (1, 8192, 19), (1, 2576, 5),
                                   (1100, 1024, 2296), (300, 960, 2600), (130, 1040, 2600),
                                   (2100, 512, 2296), (2100, 512, 2300)])
def test_int8_gemm_bit_exact(M, K, N):
    """W8A8 on the int8 matrix cores: int32 accumulators equal the oracle's bit for bit, ragged
    M / N edges included; the fused epilogue matches the oracle's fp32 expression.  The first
    seven shapes run on the 16-row tile kernel (few rows, or too few 256 x 256 tiles to fill the
    chip), the next four too, with K not a multiple of the kernel's 128-wide step (64 is the actor's
    first layer), then four single rows of 768 .. 8192 codes on the one-row kernel, then three on the
    tile kernel with four, four and two weight tiles per workgroup (ragged M and N, K a multiple of the
    step, 64 short of it, 16 past it), the last two on the large-tile GEMM (81 tiles, the last row and
    column of tiles cut short, N a multiple of 8 and not)."""
    rng = np.random.default_rng(M + K + N)
    lin, w, s = w8_layer(rng, K, N)
    xq = rng.integers(-127, 128, (M, K), dtype=np.int8)
    sx = rng.uniform(1e-3, 1e-1, M).astype(np.float32)
    bias = (rng.standard_normal(N) * 0.02).astype(np.float32)
    xd, sd = torch.from_numpy(xq).cuda(), torch.from_numpy(sx).cuda()
    acc = torch.full((M, N), -7, dtype=torch.int32, device="cuda")
    lin.forward_a8(xd, sd, out=acc, out_dtype=torch.int32)
    acc_o = O.w8a8_acc_i32(xq, w)
    assert np.array_equal(acc.cpu().numpy(), acc_o)
    y = lin.forward_a8(xd, sd, bias=torch.from_numpy(bias).cuda(), epilogue="relu").cpu().numpy()
    want = O.w8a8_epilogue(acc_o, sx, s, bias, relu=True)
    assert rel_rms(y, want) < 1e-5   # fp32 epilogue: a fused multiply-add against the oracle's two roundings
    yb = lin.forward_a8(xd, sd, bias=torch.from_numpy(bias).cuda(), out_dtype=torch.bfloat16)
    want_b = O.w8a8_epilogue(acc_o, sx, s, bias)
    assert np.abs(yb.float().cpu().numpy() - want_b).max() <= np.abs(want_b).max() * 2.0 ** -8


@pytest.mark.parametrize("N", [2296, 2300])
def test_fp8_gemm_ragged_tiles_vs_oracle(N):
    """fp8 x fp8 through the large-tile GEMM at a size the oracle finishes in seconds: 9 x 9 tiles of
    256 x 256 with the last row and column of tiles cut short; every element against the oracle."""
    M, K = 2100, 512
    rng = np.random.default_rng(N)
    a, b = fp8_operands(rng, M, N, K)
    sa, sb = np.float32(0.5), np.float32(0.25)
    bias = rng.standard_normal(N).astype(np.float32)
    lin = FP8Linear(K, N)
    lin.set_weight(b, float(sb))
    xs = torch.tensor([sa], dtype=torch.float32, device="cuda")
    yf = torch.full((M, N), float("nan"), dtype=torch.float32, device="cuda")
    lin.forward(torch.from_numpy(a).cuda(), xs, bias=torch.from_numpy(bias).cuda(), out=yf, out_dtype=torch.float32)
    y64, _ = O.fp8_forward_f64(a, b, sa, sb, want_bf16=False)
    ref = y64 + bias.astype(np.float64)
    rms = np.sqrt((ref ** 2).mean())
    assert np.abs(yf.cpu().numpy() - ref).max() <= 3e-4 * rms
    yb = lin.forward(torch.from_numpy(a).cuda(), xs, bias=torch.from_numpy(bias).cuda())
    assert torch.equal(yb, yf.to(torch.bfloat16))


def test_config4_w8a8_actor_fused_single_launch():
    """The same MLP as one launch (nq_mlp3_w8a8_forward) against the layer-by-layer oracle."""
    from noeira_amd.qlinear import mlp3_w8a8_forward
    rng = np.random.default_rng(4)
    layers = actor_layers(rng)
    for M in (4096, 1, 37):
        x = rng.standard_normal((M, 64)).astype(np.float32)
        want, _ = oracle_actor(layers, x)
        bs = [torch.from_numpy(l[3]).cuda() for l in layers]
        y = torch.full((M, 8), float("nan"), device="cuda")
        mlp3_w8a8_forward(layers[0][0], layers[1][0], layers[2][0], torch.from_numpy(x).cuda(), bs[0], bs[1], bs[2],
                          out=y)
        got = y.cpu().numpy()
        assert not np.isnan(got).any()
        assert rel_rms(got, want) < TOL_RMS, rel_rms(got, want)
        # no requantisation flips at all on this seed: the fused path equals the unfused oracle to fp32 rounding
        assert rel_rms(got, want) < 1e-5


def test_config4_actor_fused_quantizer_on_ties():
    """The fused kernel's quantizer must give the codes of the true division v / s.  Inputs that sit on and next
    to the half-way points k + 0.5 of their token's scale: a quotient off by one ulp there flips a code, and a
    flipped code shows as 1e-3."""
    from noeira_amd.qlinear import mlp3_w8a8_forward
    rng = np.random.default_rng(44)
    layers = actor_layers(rng)
    M = 512
    s = rng.uniform(0.5, 2.0, M).astype(np.float32) * np.float32(2.0) ** rng.integers(-20, 20, M).astype(np.float32)
    k = rng.integers(-127, 127, (M, 64)).astype(np.float32)
    x = ((k + np.float32(0.5)) * s[:, None]).astype(np.float32)
    step = rng.integers(-2, 3, (M, 64))
    for d in (1, 2):  # one and two ulps to either side
        x = np.where(step == d, np.nextafter(x, np.float32(np.inf)), x)
        x = np.where(step == -d, np.nextafter(x, np.float32(-np.inf)), x)
    x[:, 0] = np.float32(127.0) * s  # the token's absmax: its scale is s up to one rounding
    want, _ = oracle_actor(layers, x)
    bs = [torch.from_numpy(l[3]).cuda() for l in layers]
    y = mlp3_w8a8_forward(layers[0][0], layers[1][0], layers[2][0], torch.from_numpy(x).cuda(), bs[0], bs[1], bs[2])
    assert rel_rms(y.cpu().numpy(), want) < 1e-5


@pytest.mark.parametrize("dims", [[(48, 112), (112, 80), (80, 7)], [(256, 256), (256, 240), (240, 255)]])
def test_mlp3_widths_off_every_multiple(dims):
    """A last layer whose width is no multiple of 4 (channel scales and biases fetched one by one) or of 16 (a last
    tile cut short), inner widths that are no multiple of 64 (a last k-step cut short), against the layer-by-layer
    oracle."""
    from noeira_amd.qlinear import mlp3_w8a8_forward
    rng = np.random.default_rng(43)
    layers = []
    for K, N in dims:
        lin, w, s = w8_layer(rng, K, N)
        layers.append((lin, w, s, (rng.standard_normal(N) * 0.02).astype(np.float32)))
    x = rng.standard_normal((77, dims[0][0])).astype(np.float32)
    h = x
    for i, (_, w, s, b) in enumerate(layers):
        hq, sx = O.quantize_rows_i8(h)
        h = O.w8a8_epilogue(O.w8a8_acc_i32(hq, w), sx, s, b, relu=(i < 2))
    bs = [torch.from_numpy(l[3]).cuda() for l in layers]
    y = mlp3_w8a8_forward(layers[0][0], layers[1][0], layers[2][0], torch.from_numpy(x).cuda(), bs[0], bs[1], bs[2])
    assert rel_rms(y.cpu().numpy(), h) < TOL_RMS


def test_mlp3_other_shapes_and_errors():
    from noeira_amd import _lib as L
    from noeira_amd.qlinear import mlp3_w8a8_forward
    rng = np.random.default_rng(41)
    dims = [(48, 112), (112, 64), (64, 24)]      # K not a multiple of 64, N not a multiple of 64
    layers = []
    for K, N in dims:
        lin, w, s = w8_layer(rng, K, N)
        layers.append((lin, w, s, (rng.standard_normal(N) * 0.02).astype(np.float32)))
    x = rng.standard_normal((50, 48)).astype(np.float32)
    h = x
    for i, (_, w, s, b) in enumerate(layers):
        hq, sx = O.quantize_rows_i8(h)
        h = O.w8a8_epilogue(O.w8a8_acc_i32(hq, w), sx, s, b, relu=True)
    bs = [torch.from_numpy(l[3]).cuda() for l in layers]
    y = mlp3_w8a8_forward(layers[0][0], layers[1][0], layers[2][0], torch.from_numpy(x).cuda(), bs[0], bs[1], bs[2],
                          final_relu=True).cpu().numpy()
    assert rel_rms(y, h) < TOL_RMS
    with pytest.raises(L.NQError, match="do not chain"):
        mlp3_w8a8_forward(layers[0][0], layers[2][0], layers[1][0], torch.from_numpy(x).cuda())


# ── the two tile sizes of the 8-bit GEMM ────────────────────────────────────────────────────────────────────────
def _gemm8(lin, tile, x, x_dt, x_scale, M, out_dtype, bias=None, epilogue="none"):
    """The 8-bit GEMM on the 128 x 128 (`tile` = 128) or the 256 x 256 tile kernel (256; 2564 / 2568: on four / eight
    wavefronts; 1282: its 128 x 256 tile form), whatever nq_forward would choose."""
    import ctypes as C
    from noeira_amd import _lib as L
    out = torch.full((M, lin.OUT), 7, dtype=out_dtype, device="cuda")
    y_dt = {torch.float32: L.DT_F32, torch.bfloat16: L.DT_BF16, torch.int32: L.DT_I32}[out_dtype]
    L.check(L.lib().nq_diag_forward_gemm8(lin._h, C.c_void_p(x.data_ptr()), x_dt, C.c_void_p(x_scale.data_ptr()),
                                          C.c_void_p(out.data_ptr()), y_dt, M, C.c_void_p(bias.data_ptr()) if bias is not None else None,
                                          L.DT_F32, L.EPI_RELU if epilogue == "relu" else L.EPI_NONE, tile, None))
    return out


def test_gemm_tile_forms_on_random_ragged_shapes():
    """Every tile form of the 8-bit GEMM (128 x 128, 128 x 256, 256 x 256 on four and on eight wavefronts) on a dozen
    seeded random shapes - M from 64, any N from 1, K = 128 .. 640 in steps of 128 (one stage up to five: the stage
    buffers' wrap-around for two, three and four buffers) - against the oracle's int32 accumulators, bit for bit,
    with a sentinel under every output."""
    from noeira_amd import _lib as L
    rng = np.random.default_rng(20240611)
    shapes = [(int(rng.integers(64, 700)), 128 * int(rng.integers(1, 6)), int(rng.integers(1, 900))) for _ in range(10)]
    shapes += [(64, 128, 1), (65, 640, 257), (129, 512, 129), (513, 384, 511)]
    for M, K, N in shapes:
        lin, w, s = w8_layer(rng, K, N)
        xq_h = rng.integers(-127, 128, (M, K), dtype=np.int8)
        xq = torch.from_numpy(xq_h).cuda()
        sx = torch.from_numpy(rng.uniform(1e-3, 1e-1, M).astype(np.float32)).cuda()
        want = O.w8a8_acc_i32(xq_h, w)
        for tile in (128, 1282, 2564, 2568):
            got = _gemm8(lin, tile, xq, L.DT_I8, sx, M, torch.int32).cpu().numpy()
            assert np.array_equal(got, want), (M, K, N, tile)


@pytest.mark.parametrize("M,K,N", [(2048, 128, 8704), (2304, 256, 15360), (2240, 128, 15300), (2100, 128, 8500), (8192, 128, 11008)])
def test_gemm_leftover_tiles_on_the_half_tile_kernel(M, K, N):
    """More than a round of 256 x 256 tiles with at most half a round left over: nq_forward gives the full rounds to
    the 256 x 256 kernel and the leftover - whole columns of the last band of row tiles - to the 128 x 256 form in a
    second launch ((2048, 8704): 16 tiles = 2 columns of 8; (2304, 15360): the last band is one row of tiles, 28
    columns of it; (2240, 15300): the same with ragged edges in both directions; (2100, 8500): 50 leftover tiles that
    are no rectangle of the one-row last band's 34, so one launch; (8192, 11008): the config-5 shape, 96 = 12 columns
    of 8).  int32 accumulators equal the oracle's bit for bit and every element is written once (a sentinel
    survives nowhere); fp8 returns the bits of the single-kernel form."""
    from noeira_amd import _lib as L
    rng = np.random.default_rng(M + K + N)
    lin, w, s = w8_layer(rng, K, N)
    xq_h = rng.integers(-127, 128, (M, K), dtype=np.int8)
    sx_h = rng.uniform(1e-3, 1e-1, M).astype(np.float32)
    xq, sx = torch.from_numpy(xq_h).cuda(), torch.from_numpy(sx_h).cuda()
    out = torch.full((M, N), -2 ** 31, dtype=torch.int32, device="cuda")
    lin.forward_a8(xq, sx, out=out, out_dtype=torch.int32)
    assert np.array_equal(out.cpu().numpy(), O.w8a8_acc_i32(xq_h, w))
    bias = torch.from_numpy((rng.standard_normal(N) * 0.02).astype(np.float32)).cuda()
    assert torch.equal(lin.forward_a8(xq, sx, bias=bias, epilogue="relu", out_dtype=torch.bfloat16),
                       _gemm8(lin, 2564, xq, L.DT_I8, sx, M, torch.bfloat16, bias, "relu"))
    a, b = fp8_operands(rng, M, N, K)
    f8 = FP8Linear(K, N)
    f8.set_weight(b, 0.25)
    xs = torch.tensor([0.5], dtype=torch.float32, device="cuda")
    ad = torch.from_numpy(a).cuda()
    for dt in (torch.float32, torch.bfloat16):
        assert torch.equal(f8.forward(ad, xs, out_dtype=dt), _gemm8(f8, 2564, ad, L.DT_FP8_E4M3, xs, M, dt)), dt


@pytest.mark.parametrize("M,K,N", [(520, 1024, 2296), (1000, 512, 520), (2100, 512, 2300), (300, 4096, 1024), (64, 128, 8)])
def test_gemm_tile_sizes_against_the_oracle_and_each_other(M, K, N):
    """Both tile sizes on the same ragged problems (last row and column of tiles cut short, N a multiple of 8 and not,
    a single tile): int32 accumulators equal the oracle's bit for bit, the fused epilogue its fp32 expression, fp8
    the float64 oracle; and since both kernels add a row's K in the same order and apply the same epilogue, they
    return the same bits - int32, fp32 and bf16."""
    from noeira_amd import _lib as L
    rng = np.random.default_rng(M + K + N)
    lin, w, s = w8_layer(rng, K, N)
    xq_h = rng.integers(-127, 128, (M, K), dtype=np.int8)
    sx_h = rng.uniform(1e-3, 1e-1, M).astype(np.float32)
    bias_h = (rng.standard_normal(N) * 0.02).astype(np.float32)
    xq, sx, bias = torch.from_numpy(xq_h).cuda(), torch.from_numpy(sx_h).cuda(), torch.from_numpy(bias_h).cuda()
    acc_o = O.w8a8_acc_i32(xq_h, w)
    want = O.w8a8_epilogue(acc_o, sx_h, s, bias_h, relu=True)
    for tile in (128, 2564, 2568, 1282):  # (256: whichever of the last three nq_forward takes)
        assert np.array_equal(_gemm8(lin, tile, xq, L.DT_I8, sx, M, torch.int32).cpu().numpy(), acc_o), tile
        assert rel_rms(_gemm8(lin, tile, xq, L.DT_I8, sx, M, torch.float32, bias, "relu").cpu().numpy(), want) < 1e-5, tile
    for dt in (torch.float32, torch.bfloat16):
        for tile in (2564, 2568, 1282):
            assert torch.equal(_gemm8(lin, 128, xq, L.DT_I8, sx, M, dt, bias, "relu"), _gemm8(lin, tile, xq, L.DT_I8, sx, M, dt, bias, "relu")), (dt, tile)
    a, b = fp8_operands(rng, M, N, K)
    f8 = FP8Linear(K, N)
    f8.set_weight(b, 0.25)
    xs = torch.tensor([0.5], dtype=torch.float32, device="cuda")
    ad = torch.from_numpy(a).cuda()
    y64, _ = O.fp8_forward_f64(a, b, np.float32(0.5), np.float32(0.25), want_bf16=False)
    ref = y64 + bias_h.astype(np.float64)
    for tile in (128, 2564, 2568, 1282):
        got = _gemm8(f8, tile, ad, L.DT_FP8_E4M3, xs, M, torch.float32, bias).cpu().numpy()
        assert np.abs(got - ref).max() <= 3e-4 * np.sqrt((ref ** 2).mean()), tile
    for dt in (torch.float32, torch.bfloat16):
        for tile in (2564, 2568, 1282):
            assert torch.equal(_gemm8(f8, 128, ad, L.DT_FP8_E4M3, xs, M, dt, bias), _gemm8(f8, tile, ad, L.DT_FP8_E4M3, xs, M, dt, bias)), (dt, tile)
    # what nq_forward itself returns for the call (whichever kernel it takes): the oracle's accumulators
    assert np.array_equal(lin.forward_a8(xq, sx, out_dtype=torch.int32).cpu().numpy(), acc_o)
