"""Gates that close what the other GPU files leave open: the stand-alone dequantise of the int8 and fp8 layers
bit for bit against the oracle (other tests use it as their reference), the ReLU rule of every kernel family on
the values that tell its variants apart, the path from a blocks file to a forward, the loaders that take
`Linear`'s [IN, OUT] parameters, and the shared dequantise scratch."""
import ctypes as C
import os

import numpy as np
import pytest
import torch

from noeira_amd import _lib as L
from noeira_amd import formats as F
from noeira_amd.qlinear import (FP8Linear, QLinear, W4GroupLinear, W8Linear, mlp3_w8a8_forward, quantize_rows_i8)
from noeira_amd.safetensors_io import SafeTensors, SafeTensorsWriter, load_q4_blocks, q4_blocks_key
from oracle import oracle as O
import refw

pytestmark = pytest.mark.gpu


# ── nq_dequantize of W8_CHANNEL and FP8_E4M3: float(code) * scale, one fp32 multiply ──
@pytest.mark.parametrize("K,N", [(256, 256), (3200, 512), (4096, 1030), (16, 3)])
def test_w8_dequantize_bitwise(K, N):
    rng = np.random.default_rng(K + N)
    w = rng.integers(-128, 128, (N, K), dtype=np.int8)
    s = rng.uniform(1e-3, 1e-2, N).astype(np.float32)
    s[0] = np.float32(-3.5e-4)  # a negative and an irregular scale
    lin = W8Linear(K, N)
    lin.set_weight(w, s)
    want = w.astype(np.float32) * s[:, None]
    assert np.array_equal(lin.dequantized_dev().cpu().numpy().view(np.uint32), want.view(np.uint32))


@pytest.mark.parametrize("K,N", [(256, 256), (4096, 600), (16, 5)])
def test_fp8_dequantize_bitwise(K, N):
    rng = np.random.default_rng(K * 3 + N)
    codes = rng.integers(0, 256, (N, K), dtype=np.uint8)
    codes[(codes & 0x7F) == 0x7F] = 0x38  # (e4m3fn's two NaN codes: compared separately)
    scale = np.float32(0.0625) * np.float32(1.37)
    lin = FP8Linear(K, N)
    lin.set_weight(codes, float(scale))
    want = O.e4m3_decode_table()[codes].astype(np.float32) * scale
    assert np.array_equal(lin.dequantized_dev().cpu().numpy().view(np.uint32), want.view(np.uint32))
    nan_codes = np.full((N, K), 0x38, np.uint8)
    nan_codes[0, 0], nan_codes[N - 1, K - 1] = 0x7F, 0xFF
    lin.set_weight(nan_codes, 1.0)
    d = lin.dequantized_dev().cpu().numpy()
    assert np.isnan(d[0, 0]) and np.isnan(d[N - 1, K - 1]) and np.isnan(d).sum() == 2


# ── ReLU: z > 0 ? z : 0 (ops/relu_op.mojo:29-31): NaN -> 0, -0.0 -> +0.0, negative -> 0 ──
# With x = 0 the pre-activation is the bias, so one pattern of biases drives the rule through every kernel's
# own copy of the epilogue; the shapes are chosen for the kernel they reach.
PATTERN = np.array([np.nan, -0.0, -1.0, 2.0, 0.0, -np.inf, np.inf, 1e-30], np.float32)
WANT = np.array([0.0, 0.0, 0.0, 2.0, 0.0, 0.0, np.inf, 1e-30], np.float32)

FAMILIES = [
    # (name, format, K, N, M, x dtype, tile copy)
    ("gemv_m1 q4_0", "q4_0", 960, 320, 1, torch.float32, True),
    ("gemv_m1 w8", "w8", 512, 3200, 1, torch.bfloat16, True),
    ("gemv_m1 w4g", "w4g", 960, 2560, 1, torch.bfloat16, True),
    ("gemv (fallback) w4g64", "w4g64", 992, 70, 3, torch.float32, True),
    ("gemv_tile4 q4_0", "q4_0", 4096, 1040, 1, torch.float32, True),
    ("gemv_tile4 w4g", "w4g", 4096, 1040, 1, torch.bfloat16, True),
    ("gemv_tile8", "w8", 4096, 1040, 1, torch.bfloat16, True),
    ("gemv_row4 q4_0", "q4_0", 4096, 1040, 1, torch.float32, False),
    ("gemv_row4 w4g", "w4g", 4096, 1040, 1, torch.bfloat16, False),
    ("gemv_row8", "w8", 8192, 520, 1, torch.float32, False),
    ("gemv_split8", "w8", 4096, 4100, 1, torch.bfloat16, False),
    ("gemm_a16 q4_0", "q4_0", 960, 2560, 135, torch.float32, True),
    ("gemm_a16 w8", "w8", 3200, 512, 100, torch.bfloat16, True),
    ("gemm_a16 w4g", "w4g", 960, 960, 256, torch.bfloat16, True),
    ("gemm_a16_big q4_0", "q4_0", 960, 2560, 1120, torch.bfloat16, True),
    ("gemm_a16_big w8", "w8", 1024, 2048, 2048, torch.float32, True),
]


def _make(fmt, K, N, rng, tile_copy):
    if fmt == "q4_0":
        lin = QLinear(K, N, tile_copy=tile_copy)
        blocks = rng.integers(0, 256, (N, K // 32, 18), dtype=np.uint8)
        sc = rng.uniform(1e-3, 1e-2, (N, K // 32)).astype(np.float16).view(np.uint16)
        blocks[:, :, 0], blocks[:, :, 1] = sc & 0xFF, sc >> 8
        lin.set_blocks(blocks.reshape(-1))
    elif fmt == "w8":
        lin = W8Linear(K, N, tile_copy=tile_copy)
        lin.set_weight(rng.integers(-127, 128, (N, K), dtype=np.int8), rng.uniform(1e-3, 1e-2, N).astype(np.float32))
    else:
        group = 128 if fmt == "w4g" else 64
        G = -(-K // group)
        codes, zps = F.pack_w4g(rng.integers(0, 16, (N, K), dtype=np.uint8), rng.integers(0, 16, (N, G), dtype=np.uint8))
        lin = W4GroupLinear(K, N, group, tile_copy=tile_copy)
        lin.set_weight(codes, rng.uniform(1e-3, 1e-2, (N, G)).astype(np.float16), zps)
    return lin


def _bias_and_want(N):
    reps = -(-N // len(PATTERN))
    return np.tile(PATTERN, reps)[:N].copy(), np.tile(WANT, reps)[:N].copy()


@pytest.mark.parametrize("name,fmt,K,N,M,xdt,tile_copy", FAMILIES, ids=[f[0] for f in FAMILIES])
def test_relu_rule_float_activations(name, fmt, K, N, M, xdt, tile_copy):
    rng = np.random.default_rng(len(name) + K + N)
    lin = _make(fmt, K, N, rng, tile_copy)
    b, want = _bias_and_want(N)
    bias = torch.from_numpy(b).cuda()
    x = torch.zeros((M, K), dtype=xdt, device="cuda")
    y = lin.forward(x, bias=bias, epilogue="relu").cpu().numpy()
    for m in (0, M - 1):
        assert np.array_equal(y[m].view(np.uint32), want.view(np.uint32)), (name, m)  # (+0.0 bit for bit)
    ybf = lin.forward(x, bias=bias, epilogue="relu", out_dtype=torch.bfloat16).float().cpu().numpy()
    wbf = torch.from_numpy(want).to(torch.bfloat16).float().numpy()
    assert np.array_equal(ybf[0].view(np.uint32), wbf.view(np.uint32)), name
    # without the epilogue the bias comes back as it is (NaN stays NaN, -0.0 keeps its sign or meets +0.0)
    y0 = lin.forward(x, bias=bias).cpu().numpy()[0]
    assert np.isnan(y0[0]) and y0[2] == -1.0 and np.isneginf(y0[5])


@pytest.mark.parametrize("name,M,K,N", [("gemv8_row i8", 1, 4096, 1040), ("tile8 i8", 16, 512, 200),
                                        ("tile8 i8 many", 256, 1024, 1040), ("gemm8 i8", 1024, 256, 520),
                                        ("tile8 i8 short K", 3, 208, 37)])
def test_relu_rule_int8_activations(name, M, K, N):
    rng = np.random.default_rng(M + K + N)
    lin = W8Linear(K, N)
    lin.set_weight(rng.integers(-127, 128, (N, K), dtype=np.int8), rng.uniform(1e-3, 1e-2, N).astype(np.float32))
    b, want = _bias_and_want(N)
    xq = torch.zeros((M, K), dtype=torch.int8, device="cuda")
    sx = torch.ones((M,), dtype=torch.float32, device="cuda")
    y = lin.forward_a8(xq, sx, bias=torch.from_numpy(b).cuda(), epilogue="relu").cpu().numpy()
    for m in (0, M - 1):
        assert np.array_equal(y[m].view(np.uint32), want.view(np.uint32)), (name, m)


@pytest.mark.parametrize("name,M,K,N", [("gemv8_row fp8", 1, 4096, 1040), ("tile8 fp8", 16, 512, 200),
                                        ("gemm8 fp8", 1024, 256, 520)])
def test_relu_rule_fp8_activations(name, M, K, N):
    rng = np.random.default_rng(M + K + N + 1)
    lin = FP8Linear(K, N)
    lin.set_weight(F.encode_e4m3(rng.standard_normal((N, K)).astype(np.float32)), 0.0625)
    b, want = _bias_and_want(N)
    xc = torch.zeros((M, K), dtype=torch.uint8, device="cuda")
    sa = torch.ones((1,), dtype=torch.float32, device="cuda")
    y = lin.forward(xc, sa, bias=torch.from_numpy(b).cuda(), epilogue="relu", out_dtype=torch.float32).cpu().numpy()
    for m in (0, M - 1):
        assert np.array_equal(y[m].view(np.uint32), want.view(np.uint32)), (name, m)


def test_relu_rule_fused_actor():
    rng = np.random.default_rng(4)
    dims = [(64, 256), (256, 256), (256, 8)]
    lins = []
    for K, N in dims:
        lin = W8Linear(K, N)
        lin.set_weight(rng.integers(-127, 128, (N, K), dtype=np.int8), rng.uniform(1e-3, 1e-2, N).astype(np.float32))
        lins.append(lin)
    x = torch.zeros((4096, 64), dtype=torch.float32, device="cuda")
    b3 = torch.from_numpy(PATTERN.copy()).cuda()
    y = mlp3_w8a8_forward(lins[0], lins[1], lins[2], x, None, None, b3, final_relu=True).cpu().numpy()
    for m in (0, 4095):
        assert np.array_equal(y[m].view(np.uint32), WANT.view(np.uint32)), m


# ── file -> load_q4_blocks -> set_blocks -> forward (layer_weights.mojo:820-866) ──
def test_blocks_file_to_forward(tmp_path):
    rng = np.random.default_rng(8)
    shapes = {"model.layers.0.self_attn.q_proj.weight": (960, 960), "model.layers.0.self_attn.k_proj.weight": (960, 320),
              "model.layers.0.mlp.down_proj.weight": (2560, 960)}
    ws = {name: (rng.standard_normal((OUT, IN)) * 0.05).astype(np.float32) for name, (IN, OUT) in shapes.items()}
    wr = SafeTensorsWriter()
    for name, (IN, OUT) in shapes.items():
        blocks = O.rtn_q4_0_blocks(ws[name])
        wr.add_u8(q4_blocks_key(name), [OUT, (IN // 32) * 18], blocks)
    path = os.path.join(tmp_path, "text_q4.safetensors")
    wr.save(path)
    f = SafeTensors(path)
    for name, (IN, OUT) in shapes.items():
        blocks = load_q4_blocks(f, name, IN, OUT)
        lin = QLinear.make(IN, OUT, "gpu")
        lin.set_blocks(blocks)
        for T in (1, 135):
            x = rng.standard_normal((T, IN)).astype(np.float32)
            y = lin.forward(torch.from_numpy(x).cuda()).cpu().numpy()
            assert O.rel_max(y, O.qlinear_forward_cpu(blocks, IN, OUT, x)) < 1e-5, (name, T)
        assert np.array_equal(lin.blocks(), blocks)
    # a projection of another shape under the same key is refused before anything is loaded
    with pytest.raises(ValueError, match=r"expected \[320, 540\]"):
        load_q4_blocks(f, "model.layers.0.self_attn.q_proj.weight", 960, 320)
    with pytest.raises(KeyError):
        load_q4_blocks(f, "model.layers.0.self_attn.v_proj.weight", 960, 320)
    # and bytes of the wrong length are refused by the layer itself (qlinear.mojo:276-281)
    lin = QLinear.make(960, 320, "gpu")
    with pytest.raises(L.NQError, match="bytes, expected 172800"):
        lin.set_blocks(load_q4_blocks(f, "model.layers.0.self_attn.q_proj.weight", 960, 960))


# ── loaders for `Linear[IN, OUT]`'s parameters (linear.mojo:970-971, qlinear_common.mojo:86-91) ──
@pytest.mark.parametrize("kind", ["w8", "fp8", "w4g", "q4_0"])
def test_from_linear_is_x_at_w_plus_b(kind):
    rng = np.random.default_rng(sum(map(ord, kind)))
    IN, OUT, M = 256, 192, 5
    w = (rng.standard_normal((IN, OUT)) * 0.05).astype(np.float32)  # Linear's orientation
    b = (rng.standard_normal(OUT) * 0.1).astype(np.float32)
    x = rng.standard_normal((M, IN)).astype(np.float32)
    dense = x.astype(np.float64) @ w.astype(np.float64) + b  # y = x @ W + b
    rms = np.sqrt((dense ** 2).mean())
    xd = torch.from_numpy(x).cuda()
    if kind == "w8":
        lin = W8Linear.from_linear(w, b)
        q, s = F.quantize_w8_channel(np.ascontiguousarray(w.T))
        want = O.w8_forward_f64(q, s, x, b)
        y = lin.forward(xd).cpu().numpy()
        tol_q = 6e-2
    elif kind == "fp8":
        lin = FP8Linear.from_linear(w, b)
        # the loader's rule restated with the oracle's encoder: one scale absmax / 448, codes of w / scale
        sc8 = float(np.abs(w).max()) / 448.0
        deq = refw.fp8(O.e4m3_encode(np.ascontiguousarray(w.T) / np.float32(sc8)), sc8).cpu().numpy()
        xc = torch.from_numpy(x).to(torch.float8_e4m3fn)
        want = xc.double().numpy() @ deq.T + b
        y = lin.forward(xc.view(torch.uint8).cuda(), torch.ones(1, device="cuda"), out_dtype=torch.float32).cpu().numpy()
        dense = xc.double().numpy() @ w.astype(np.float64) + b
        tol_q = 2e-1
    elif kind == "w4g":
        lin = W4GroupLinear.from_linear(w, b, group=128)
        q4g, s4g, z4g = F.quantize_w4g_asym(np.ascontiguousarray(w.T), 128)
        c4g, zp4g = F.pack_w4g(q4g, z4g)
        want = x.astype(np.float64) @ refw.w4g(c4g, s4g, zp4g, OUT, IN, 128).cpu().numpy().T + b
        y = lin.forward(xd).cpu().numpy()
        tol_q = 5e-1
    else:
        lin = QLinear.from_linear(w, b)
        want = O.dense_forward_f64(O.dequantize_q4_0(O.rtn_q4_0_blocks(np.ascontiguousarray(w.T)), OUT, IN), x) + b
        y = lin.forward(xd).cpu().numpy()
        tol_q = 5e-1
    assert y.shape == (M, OUT)
    assert np.abs(y - want).max() < 1e-3 * rms, kind          # the layer's own arithmetic
    # and the dense Linear it stands in for, to the format's quantisation error (a weight read in the wrong
    # orientation is off by more than the output's RMS)
    assert np.abs(y - dense).max() < tol_q * rms, kind
    # LinearAct[..., ReLU]
    if kind != "fp8":
        yr = lin.forward(xd, epilogue="relu").cpu().numpy()
        assert np.abs(yr - np.maximum(want, 0)).max() < 1e-3 * rms
    with pytest.raises(L.NQError, match="expected Linear's"):
        W8Linear(IN, OUT)._linear_params(w.T, None, IN, OUT, "W8Linear.from_linear")


def test_quantize_w8_channel_is_symmetric_absmax():
    rng = np.random.default_rng(3)
    w = rng.standard_normal((7, 33)).astype(np.float32)
    w[2] = 0.0
    w[3, 5] = 4.0  # an exact tie somewhere below
    q, s = F.quantize_w8_channel(w)
    for n in range(7):
        am = np.abs(w[n]).max()
        sn = np.float32(am / np.float32(127)) if am > 0 else np.float32(1)
        assert s[n] == sn
        for k in range(33):
            want = int(np.clip(O.round_half_even(float(np.float32(w[n, k]) / sn)), -127, 127))
            assert int(q[n, k]) == want, (n, k)
    assert np.abs(q).max() == 127


# ── nq_dequantize at the full-size layer (4096 -> 11008, 45 M weights), bit for bit against the oracle ──
@pytest.mark.parametrize("fmt,tile_copy", [("q4_0", True), ("q4_0", False), ("w4g", True), ("w4g", False), ("w8", True),
                                           ("w8", False), ("fp8", True)])
def test_dequantize_bitwise_at_full_size(fmt, tile_copy):
    """Whatever device layout the layer keeps (row-ordered codes, the tile-ordered copy), `nq_dequantize` returns
    the fp32 values the CPU oracle computes from the codes the test drew, every one of the 45 M bit for bit; the forward
    tests at this size take their reference weights from the oracle, and this ties the library's own view to them."""
    rng = np.random.default_rng(sum(map(ord, fmt)) + tile_copy)
    K, N = 4096, 11008
    if fmt == "q4_0":
        blocks = rng.integers(0, 256, (N, K // 32, 18), dtype=np.uint8)
        sc = (rng.uniform(1e-3, 1e-2, (N, K // 32)) * rng.choice([-1.0, 1.0], (N, K // 32))).astype(np.float16).view(np.uint16)
        blocks[:, :, 0], blocks[:, :, 1] = sc & 0xFF, sc >> 8
        lin = QLinear(K, N, tile_copy=tile_copy)
        lin.set_blocks(blocks.reshape(-1))
        want = O.dequantize_q4_0(blocks.reshape(-1), N, K)
    elif fmt == "w4g":
        G = K // 128
        codes, zps = F.pack_w4g(rng.integers(0, 16, (N, K), dtype=np.uint8), rng.integers(0, 16, (N, G), dtype=np.uint8))
        sg = rng.uniform(1e-3, 1e-2, (N, G)).astype(np.float16)
        lin = W4GroupLinear(K, N, 128, tile_copy=tile_copy)
        lin.set_weight(codes, sg, zps)
        want = O.w4g_dequantize(codes, sg.view(np.uint16), zps, N, K, 128)
    elif fmt == "w8":
        w = rng.integers(-128, 128, (N, K), dtype=np.int8)
        sw = (rng.uniform(1e-3, 1e-2, N) * rng.choice([-1.0, 1.0], N)).astype(np.float32)
        lin = W8Linear(K, N, tile_copy=tile_copy)
        lin.set_weight(w, sw)
        want = w.astype(np.float32) * sw[:, None]  # one fp32 multiply per weight
    else:
        codes = rng.integers(0, 256, (N, K), dtype=np.uint8)
        codes[(codes & 0x7F) == 0x7F] = 0x38  # (the two NaN codes are compared in test_fp8_dequantize_bitwise)
        scale = np.float32(0.0625) * np.float32(1.37)
        lin = FP8Linear(K, N)
        lin.set_weight(codes, float(scale))
        want = O.e4m3_decode_table()[codes].astype(np.float32) * scale
    got = lin.dequantized_dev()
    assert torch.equal(got.view(torch.int32), torch.from_numpy(want).cuda().view(torch.int32))


# ── share_scratch: dequantized_dev() writes the shared buffer (qlinear.mojo:330-340) ──
def test_share_scratch_receives_the_dequantised_weight():
    rng = np.random.default_rng(9)
    a, b = QLinear(960, 320), QLinear(320, 960)
    for lin in (a, b):
        lin.set_weight((rng.standard_normal((lin.OUT, lin.IN)) * 0.05).astype(np.float32))
    shared = torch.full((960 * 320 + 100,), float("nan"), dtype=torch.float32, device="cuda")
    a.share_scratch(shared, shared.numel())
    b.share_scratch(shared, shared.numel())
    own_a = a.dequantized_dev(torch.empty((320, 960), dtype=torch.float32, device="cuda"))
    got = a.dequantized_dev()
    assert got.data_ptr() == shared.data_ptr()
    assert torch.equal(shared[: 960 * 320].view(320, 960), own_a)  # the bytes are in the shared buffer
    assert bool(torch.isnan(shared[960 * 320:]).all())              # and nothing past the weight was touched
    got_b = b.dequantized_dev()                                     # the next layer reuses the same memory
    assert got_b.data_ptr() == shared.data_ptr() and got_b.shape == (960, 320)
    assert np.array_equal(got_b.cpu().numpy(), O.dequantize_q4_0(b.blocks().reshape(960, -1), 960, 320))
    with pytest.raises(L.NQError, match="share_scratch"):
        a.share_scratch(shared, 960 * 320 - 1)


@pytest.mark.parametrize("xdt", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("M,K,N", [(1, 512, 3200), (2, 512, 3200), (7, 784, 40), (100, 3200, 512), (256, 4096, 1000),
                                   (600, 512, 3200), (2050, 1040, 650)])
def test_fp8_weights_under_16bit_activations(M, K, N, xdt):
    """e4m3fn weights with fp32 / bf16 activations at every M: one row on the GEMV, from two rows on the bf16
    matrix-core kernels (the codes decode to bf16 exactly, fp32 activations enter as three exact bf16 terms), so
    the result is the fp64 product over the weights the oracle's decode table gives for the codes the test drew,
    to fp32 accumulation accuracy.  With bias, ReLU and bf16 out; a NaN code poisons
    its own output channel and no other."""
    rng = np.random.default_rng(M + K + N)
    lin = FP8Linear(K, N)
    wt = torch.from_numpy(rng.standard_normal((N, K)).astype(np.float32)).to(torch.float8_e4m3fn)
    codes = wt.view(torch.uint8).numpy().copy()
    lin.set_weight(codes, 1.0 / 16)
    deq = refw.fp8(codes, 1.0 / 16)
    x = torch.from_numpy(rng.standard_normal((M, K)).astype(np.float32)).cuda().to(xdt)
    bias = torch.from_numpy((rng.standard_normal(N) * 0.5).astype(np.float32)).cuda()
    want = x.double() @ deq.T
    y = lin.forward_a16(x)
    assert y.dtype == torch.float32 and y.shape == (M, N)
    assert float((y.double() - want).abs().max()) <= 1e-5 * float(want.abs().max())
    assert torch.equal(lin.forward_a16(x), y)
    yr = lin.forward_a16(x, bias=bias, epilogue="relu")
    want_r = (want + bias.double()).clamp_min(0)
    assert float((yr.double() - want_r).abs().max()) <= 1e-5 * float(want_r.abs().max())
    yb = lin.forward_a16(x, bias=bias, out_dtype=torch.bfloat16)
    want_b = want + bias.double()
    assert float((yb.double() - want_b).abs().max()) <= 2.0 ** -8 * float(want_b.abs().max())
    codes[N // 2, K // 3] = 0x7F  # NaN
    lin.set_weight(codes, 1.0 / 16)
    yn = lin.forward_a16(x)
    assert bool(torch.isnan(yn[:, N // 2]).all())
    keep = torch.ones(N, dtype=torch.bool, device="cuda")
    keep[N // 2] = False
    assert torch.equal(yn[:, keep], y[:, keep])


def test_gemm8_timeline_diagnostic_reports_ordered_stamps_and_the_same_output():
    """nq_diag_gemm8_timeline: the call nq_forward would make, with every workgroup of the large-tile kernel
    reporting its four readings of the constant clock and two of the shader clock: ordered, all written, a
    plausible clock between them, and y as without them."""
    import ctypes as C

    from noeira_amd import _lib as L

    M, K, N = 2048, 512, 2304   # 8 x 9 tiles
    rng = np.random.default_rng(3)
    lin = FP8Linear(K, N)
    wt = torch.from_numpy(rng.standard_normal((N, K)).astype(np.float32)).to(torch.float8_e4m3fn)
    lin.set_weight(wt.view(torch.uint8).numpy(), 0.25)
    xc = torch.from_numpy(rng.standard_normal((M, K)).astype(np.float32)).to(torch.float8_e4m3fn).view(torch.uint8).cuda()
    sa = torch.tensor([0.5], dtype=torch.float32, device="cuda")
    want = lin.forward(xc, sa)
    y = torch.zeros_like(want)
    tiles = 8 * 9
    stamps = torch.zeros((tiles, 6), dtype=torch.int64, device="cuda")
    args = (lin._h, C.c_void_p(xc.data_ptr()), L.DT_FP8_E4M3, C.c_void_p(sa.data_ptr()), C.c_void_p(y.data_ptr()),
            L.DT_BF16, M, C.c_void_p(stamps.data_ptr()))
    assert L.lib().nq_diag_gemm8_timeline(*args, tiles - 1, C.c_void_p(0)) == L.NQ_ERR_INVALID
    L.check(L.lib().nq_diag_gemm8_timeline(*args, tiles, C.c_void_p(0)))
    assert torch.equal(y, want)
    t = stamps.cpu().numpy()
    assert (t > 0).all() and (np.diff(t[:, :4], axis=1) >= 0).all()
    assert (t[:, 3] - t[:, 0]).max() < 100000   # under a millisecond of 10 ns ticks
    ghz = (t[:, 5] - t[:, 4]) / np.maximum(t[:, 2] - t[:, 1], 1) / 10.0   # cycles per 10 ns tick -> GHz
    assert 0.3 < np.median(ghz) < 3.0
    # and the next ordinary call writes no stamps
    stamps.zero_()
    lin.forward(xc, sa)
    torch.cuda.synchronize()
    assert int(stamps.abs().sum()) == 0


def test_stream_read_diagnostic_really_reads():
    """nq_diag_stream_read is the floor bench.py prints beside the large GEMVs: it must move the bytes.  256 MiB
    cannot come out of HBM in less than 256 MiB / 8 TB/s = 33.5 us (the published peak), whatever the clocks."""
    import ctypes as C

    from noeira_amd import _lib as L

    nbytes = 256 << 20
    bufs = [torch.full((nbytes,), 0x5A, dtype=torch.uint8, device="cuda") for _ in range(3)]   # > the 256 MB cache
    lib = L.lib()
    s = C.c_void_p(torch.cuda.current_stream().cuda_stream)
    for b in bufs:
        L.check(lib.nq_diag_stream_read(C.c_void_p(b.data_ptr()), nbytes, s))
    torch.cuda.synchronize()
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    e0.record()
    for _ in range(4):
        for b in bufs:
            L.check(lib.nq_diag_stream_read(C.c_void_p(b.data_ptr()), nbytes, s))
    e1.record()
    torch.cuda.synchronize()
    us = e0.elapsed_time(e1) * 1e3 / 12
    assert us > 33.5, f"a plain read of 256 MiB took {us:.1f} us: the loads were not issued"
    assert us < 200


def test_a16_shape_changes_no_bits():
    """nq_diag_forward_a16 runs one forward on the 16-row tile kernel under a tile shape of the caller's choice
    (bench.py times a grid of calls under each shape with it).  A shape decides which workgroup computes an output,
    not the order of its sum: every shape returns the bits of nq_forward's own choice, for each format and
    activation type; shapes that do not exist are refused, and nothing of the call outlasts it (the forward that
    follows is the library's own again)."""
    lib = L.lib()
    rng = np.random.default_rng(61)
    null = C.c_void_p(0)
    for fmt, K, N, M in (("q4_0", 960, 1000, 135), ("w4g", 2560, 520, 40), ("w8", 3200, 512, 100), ("w4g64", 992, 300, 77)):
        lin = _make(fmt, K, N, rng, False)
        for xdt, xc in ((torch.float32, L.DT_F32), (torch.bfloat16, L.DT_BF16)):
            x = torch.from_numpy(rng.standard_normal((M, K)).astype(np.float32)).to(xdt).cuda()
            want = lin.forward(x)
            for mw, nw in ((1, 1), (1, 2), (1, 4), (2, 2), (2, 4)):
                y = torch.full((M, N), float("nan"), dtype=torch.float32, device="cuda")
                rc = lib.nq_diag_forward_a16(lin._h, C.c_void_p(x.data_ptr()), xc, C.c_void_p(y.data_ptr()), L.DT_F32, M, mw, nw, null)
                if xdt == torch.float32 and (mw, nw) == (2, 4):
                    assert rc == L.NQ_ERR_INVALID and "shapes are" in L.last_error()
                    continue
                L.check(rc)
                assert torch.equal(y.view(torch.int32), want.view(torch.int32)), (fmt, xdt, mw, nw)
            assert torch.equal(lin.forward(x).view(torch.int32), want.view(torch.int32))
    x = torch.zeros((4, 960), dtype=torch.bfloat16, device="cuda")
    y = torch.zeros((4, 1000), dtype=torch.float32, device="cuda")
    lin = _make("q4_0", 960, 1000, rng, False)
    for mw, nw in ((2, 1), (3, 2), (1, 3), (0, 1), (-1, -1), (0, 0)):
        assert lib.nq_diag_forward_a16(lin._h, C.c_void_p(x.data_ptr()), L.DT_BF16, C.c_void_p(y.data_ptr()), L.DT_F32, 4, mw, nw, null) == L.NQ_ERR_INVALID
        assert "shapes are" in L.last_error()
    assert lib.nq_diag_forward_a16(lin._h, C.c_void_p(x.data_ptr()), L.DT_BF16, C.c_void_p(y.data_ptr()), L.DT_F32, 1, 1, 1, null) == L.NQ_ERR_UNSUPPORTED


def test_device_bytes_one_copy_where_no_kernel_reads_a_second():
    """`keep_only_repacked` keeps exactly one device copy of the weights in the reference (qlinear.mojo:342-356; "int4
    buys memory", docs-site/src/content/docs/nn/peft-quant.mdx:194-199).  Here a second, tile-ordered copy exists only
    where a kernel of the default dispatch reads it: nq_device_bytes bounds it.  The narrow SmolVLA projections
    (q, k, v, o, down) hold 0.5625 bytes per weight, the wide ones (gate, up: the M-tile kernel's) 1.16 (IN = 960 pads to 1024 in tile order) unless made
    with NQ_FLAG_NO_TILE_COPY; the forward's bits do not depend on keep_only_repacked."""
    rng = np.random.default_rng(77)
    for K, N, wide in ((960, 960, False), (960, 320, False), (2560, 960, False), (960, 2560, True)):
        lin = _make("q4_0", K, N, rng, True)
        x = torch.from_numpy(rng.standard_normal((135, K)).astype(np.float32)).cuda()
        before = {T: lin.forward(x[:T]).clone() for T in (135, 16, 7, 1)}
        per_weight = lin.device_bytes() / (K * N)
        assert (1.0 < per_weight < 1.17) if wide else (0.5625 <= per_weight <= 0.60), (K, N, per_weight)
        lin.keep_only_repacked()
        assert lin.device_bytes() / (K * N) == per_weight
        for T, want in before.items():
            assert torch.equal(lin.forward(x[:T]).view(torch.int32), want.view(torch.int32)), (K, N, T)
        lean = _make("q4_0", K, N, rng, False)  # NQ_FLAG_NO_TILE_COPY
        assert 0.5625 <= lean.device_bytes() / (K * N) <= 0.60
    assert QLinear(960, 320).device_bytes() == 0  # nothing loaded
    w8 = _make("w8", 3200, 512, rng, True)
    assert 1.0 <= w8.device_bytes() / (3200 * 512) <= 1.01
