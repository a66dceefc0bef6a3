"""Pins the oracle's extension formats (int8 per-channel, per-token int8
activations, uint4 group-wise asymmetric, fp8 e4m3fn).  The reference
implements none of these, so there are no reference vectors: each function is
pinned against a library routine (numpy integer matmul, numpy float16,
torch.float8_e4m3fn, numpy.round) or a brute-force numpy re-derivation written
independently of the C code.
"""
import numpy as np
import pytest
import torch

from oracle import oracle as O


def test_w8a8_int32_accumulators_vs_numpy():
    rng = np.random.default_rng(0)
    for M, N, K in [(1, 256, 256), (9, 8, 64), (5, 33, 4096)]:
        xq = rng.integers(-127, 128, (M, K), dtype=np.int8)
        w = rng.integers(-127, 128, (N, K), dtype=np.int8)
        want = xq.astype(np.int32) @ w.astype(np.int32).T
        assert np.array_equal(O.w8a8_acc_i32(xq, w), want)
    # the extreme: every product 127*127 at K = 4096 stays inside int32
    xq = np.full((1, 4096), 127, np.int8)
    w = np.full((2, 4096), -127, np.int8)
    assert (O.w8a8_acc_i32(xq, w) == -4096 * 127 * 127).all()


def test_quantize_rows_i8_vs_numpy():
    rng = np.random.default_rng(1)
    x = rng.standard_normal((17, 64)).astype(np.float32)
    x[3] = 0.0                      # absmax 0 -> scale 1, codes 0
    x[4, :] = np.float32(0.5) * np.arange(64, dtype=np.float32) - 16   # ties at scale 1?  see below
    x[4, 0] = -127.0                # absmax 127 -> scale exactly 1 -> halves are exact ties
    q, s = O.quantize_rows_i8(x)
    amax = np.abs(x).max(axis=1)
    s_want = (amax / np.float32(127)).astype(np.float32)
    s_want[s_want == 0] = 1
    assert np.array_equal(s.view(np.uint32), s_want.view(np.uint32))
    q_want = np.clip(np.round(x / s_want[:, None]), -127, 127).astype(np.int8)  # np.round: ties to even
    assert np.array_equal(q, q_want)
    assert not q[3].any() and s[3] == 1.0
    assert q[4, 1] == -16 and q[4, 2] == -15  # -15.5 -> -16 (even), -15.0
    assert (np.abs(q.astype(np.int32)) <= 127).all() and (np.abs(q).max(axis=1)[amax > 0] == 127).all()


def test_w8_forward_fp32_and_fp64():
    rng = np.random.default_rng(2)
    M, N, K = 3, 40, 512
    w = rng.integers(-127, 128, (N, K), dtype=np.int8)
    s = rng.uniform(1e-3, 1e-2, N).astype(np.float32)
    x = rng.standard_normal((M, K)).astype(np.float32)
    b = (rng.standard_normal(N) * 0.02).astype(np.float32)
    exact = (x.astype(np.float64) @ w.astype(np.float64).T) * s.astype(np.float64) + b.astype(np.float64)
    y64 = O.w8_forward_f64(w, s, x, b)
    assert np.abs(y64 - exact).max() <= 1e-12 * np.abs(exact).max()
    y = O.w8_forward_f32(w, s, x, b)
    assert np.abs(y - exact).max() / np.sqrt((exact ** 2).mean()) < 1e-5
    yr = O.w8_forward_f32(w, s, x, b, relu=True)
    assert np.array_equal(yr, np.where(y > 0, y, np.float32(0)))
    assert np.array_equal(O.w8_forward_f64(w, s, x, b, relu=True), np.where(y64 > 0, y64, 0.0))
    # small integers: fp32 arithmetic is exact, so the result equals the integer closed form
    xi = rng.integers(-4, 5, (M, K)).astype(np.float32)
    yi = O.w8_forward_f32(w, np.ones(N, np.float32), xi)
    assert np.array_equal(yi, (xi.astype(np.int64) @ w.astype(np.int64).T).astype(np.float32))


def test_w8a8_epilogue_closed_form():
    rng = np.random.default_rng(3)
    M, N = 6, 10
    acc = rng.integers(-2 ** 20, 2 ** 20, (M, N), dtype=np.int32)
    sx = rng.uniform(1e-3, 1e-1, M).astype(np.float32)
    sw = rng.uniform(1e-3, 1e-2, N).astype(np.float32)
    b = rng.standard_normal(N).astype(np.float32)
    want = acc.astype(np.float32) * (sx[:, None] * sw[None, :]) + b[None, :]
    assert np.array_equal(O.w8a8_epilogue(acc, sx, sw, b), want)
    assert np.array_equal(O.w8a8_epilogue(acc, sx, sw, b, relu=True), np.where(want > 0, want, np.float32(0)))
    assert np.array_equal(O.w8a8_epilogue(acc, sx, sw), acc.astype(np.float32) * (sx[:, None] * sw[None, :]))


@pytest.mark.parametrize("K,group", [(960, 128), (2560, 128), (128, 32), (64, 128)])
def test_w4g_dequantize_vs_bruteforce(K, group):
    rng = np.random.default_rng(K + group)
    N = 5
    G = -(-K // group)
    q = rng.integers(0, 16, (N, K), dtype=np.uint8)
    z = rng.integers(0, 16, (N, G), dtype=np.uint8)
    s = rng.uniform(1e-3, 1e-1, (N, G)).astype(np.float16)
    codes = (q[:, 0::2] | (q[:, 1::2] << 4)).astype(np.uint8)
    zp = np.zeros((N, (G + 1) // 2), np.uint8)
    for g in range(G):
        zp[:, g // 2] |= (z[:, g] << (4 * (g & 1))).astype(np.uint8)
    got = O.w4g_dequantize(codes, s.view(np.uint16), zp, N, K, group)
    want = np.empty((N, K), np.float32)
    for n in range(N):
        for k in range(K):
            g = k // group
            want[n, k] = (np.float32(q[n, k]) - np.float32(z[n, g])) * np.float32(s[n, g])
    assert np.array_equal(got.view(np.uint32), want.view(np.uint32))
    if K == 960:
        assert G == 8  # ragged: the 8th group is 64 wide


def test_e4m3_decode_all_codes_vs_torch():
    codes = torch.arange(256, dtype=torch.uint8)
    want = codes.view(torch.float8_e4m3fn).float().numpy()
    got = O.e4m3_decode_table()
    nan = np.isnan(want)
    assert nan.sum() == 2 and np.array_equal(np.isnan(got), nan)  # 0x7F and 0xFF only: no infinities
    assert np.array_equal(got[~nan].view(np.uint32), want[~nan].view(np.uint32))
    assert got[0x7E] == 448.0 and got[0xFE] == -448.0 and got[0x01] == 2.0 ** -9


def test_e4m3_encode_vs_torch_in_range_and_saturation():
    rng = np.random.default_rng(4)
    tbl = O.e4m3_decode_table()
    fin = np.sort(tbl[:0x7F])
    mids = ((fin[:-1].astype(np.float64) + fin[1:].astype(np.float64)) / 2).astype(np.float32)  # exact ties
    x = np.concatenate([
        np.clip(rng.standard_normal(40000).astype(np.float32), -448, 448),
        (rng.standard_normal(20000) * 100).clip(-448, 448).astype(np.float32),
        (rng.standard_normal(20000) * 1e-2).astype(np.float32),
        fin, -fin, mids, -mids, np.nextafter(mids, np.float32(0)), np.nextafter(mids, np.float32(1e9)),
        np.array([0.0, -0.0, 448.0, -448.0, 2.0 ** -10, 2.0 ** -10 * 1.001, 2.0 ** -9, 1e-9], np.float32),
    ])
    x = x[np.abs(x) <= 448]
    want = torch.from_numpy(x).to(torch.float8_e4m3fn).view(torch.uint8).numpy()
    got = O.e4m3_encode(x)
    assert np.array_equal(got, want), np.flatnonzero(got != want)[:10]
    # saturating above the largest finite (BASELINE: "clipped to the e4m3 range")
    big = np.array([449.0, 464.0, 480.0, 1e6, np.inf, -500.0, -np.inf], np.float32)
    assert np.array_equal(O.e4m3_encode(big), np.array([0x7E, 0x7E, 0x7E, 0x7E, 0x7E, 0xFE, 0xFE], np.uint8))
    assert (O.e4m3_encode(np.array([np.nan], np.float32))[0] & 0x7F) == 0x7F
    # encode ∘ decode is the identity on every non-NaN code (−0 keeps its sign)
    ok = ~np.isnan(tbl)
    assert np.array_equal(O.e4m3_encode(tbl[ok]), np.arange(256, dtype=np.uint8)[ok])


def test_fp8_forward_vs_numpy():
    rng = np.random.default_rng(5)
    M, N, K = 4, 9, 256
    a = O.e4m3_encode(np.clip(rng.standard_normal((M, K)), -448, 448).astype(np.float32))
    b = O.e4m3_encode(np.clip(rng.standard_normal((N, K)), -448, 448).astype(np.float32))
    sa, sb = np.float32(0.37), np.float32(1.9)
    fa = torch.from_numpy(a).view(torch.float8_e4m3fn).double().numpy()
    fb = torch.from_numpy(b).view(torch.float8_e4m3fn).double().numpy()
    want = (fa @ fb.T) * np.float64(sa * sb)
    y64, ybf = O.fp8_forward_f64(a, b, sa, sb)
    assert np.abs(y64 - want).max() <= 1e-12 * np.abs(want).max()
    want_bf = torch.from_numpy(want.astype(np.float32)).to(torch.bfloat16).view(torch.int16).numpy().view(np.uint16)
    assert np.array_equal(ybf, want_bf)


# ── LoRA forward_add (lora.mojo:292-318) ───────────────────────────────────
def test_lora_forward_add_against_numpy():
    rng = np.random.default_rng(12)
    T, IN, OUT, R = 4, 13, 7, 5
    x = rng.standard_normal((T, IN)).astype(np.float32)
    a = rng.standard_normal((IN, R)).astype(np.float32)
    b = rng.standard_normal((R, OUT)).astype(np.float32)
    y0 = rng.standard_normal((T, OUT)).astype(np.float32)
    y = O.lora_forward_add(x, a, b, 0.4, y0.copy())
    want = y0.astype(np.float64) + 0.4 * (x.astype(np.float64) @ a.astype(np.float64)) @ b.astype(np.float64)
    assert np.abs(y - want).max() <= 1e-6 * np.abs(want).max()
    # B = 0 is a no-op, bit for bit (test_lora.mojo [1]); a swapped A / B or a dropped scale is not
    assert np.array_equal(O.lora_forward_add(x, a, np.zeros_like(b), 0.4, y0.copy()), y0)
    assert np.abs(O.lora_forward_add(x, a, b, 1.0, y0.copy()) - want).max() > 1e-2
    # rank padding is exact: zero columns of A / rows of B change nothing (lora.mojo:28-41)
    ap = np.concatenate([a, np.zeros((IN, 11), np.float32)], axis=1)
    bp = np.concatenate([b, np.zeros((11, OUT), np.float32)], axis=0)
    assert np.array_equal(O.lora_forward_add(x, ap, bp, 0.4, y0.copy()), y)


# ── the three-term int8 split of an activation row (nq_gemv_split.hip), restated in numpy fp32 ──
def _split3(x, fused):
    """x fp32 [K] -> (s, q1, q2, q3) with x ~ s (q1 + q2 / 254 + q3 / 254^2).  `fused` rounds the exact
    products r * 254 (one fma each, what the kernel does); without it the products are rounded to fp32 first.
    The bounds must hold either way."""
    f32, f64 = np.float32, np.float64
    absmax = f32(np.abs(x).max())
    inv_s = f32(127.0) / absmax if absmax > 1e-30 else f32(0.0)
    t = (x * inv_s).astype(f32)
    q1 = np.rint(t).astype(f32)
    r1 = (t - q1).astype(f32)                      # exact
    if fused:
        q2 = np.rint(r1.astype(f64) * 254.0).astype(f32)
        r2 = (r1.astype(f64) * 254.0 - q2.astype(f64)).astype(f32)
        q3 = np.rint(r2.astype(f64) * 254.0).astype(f32)
    else:
        t2 = (r1 * f32(254.0)).astype(f32)
        q2 = np.rint(t2).astype(f32)
        r2 = (t2 - q2).astype(f32)
        q3 = np.rint((r2 * f32(254.0)).astype(f32)).astype(f32)
    s = absmax * f32(1.0 / 127.0) if inv_s != 0 else f32(0.0)
    return s, q1, q2, q3


@pytest.mark.parametrize("fused", [False, True])
@pytest.mark.parametrize("kind", ["normal", "bf16", "outlier", "ties"])
def test_three_term_int8_split_bounds(kind, fused):
    rng = np.random.default_rng(5)
    x = rng.standard_normal(1 << 16).astype(np.float32)
    if kind == "bf16":    # few significand bits: leftovers land on exact halves far more often
        x = torch.from_numpy(x).to(torch.bfloat16).float().numpy()
    if kind == "outlier":
        x[7] = 300.0
    if kind == "ties":    # every multiple of 1 / 508 of the scale: all the .5 cases of the second term
        x = (np.arange(-127 * 508, 127 * 508 + 1, dtype=np.float64) / 508.0).astype(np.float32)
    s, q1, q2, q3 = _split3(x, fused)
    for q in (q1, q2, q3):  # every term fits an int8, the range the byte packing keeps
        assert np.abs(q).max() <= 127
    rec = s.astype(np.float64) * (q1.astype(np.float64) + q2 / 254.0 + q3 / 254.0 ** 2)
    bound = np.abs(x).max() / (127.0 * 254.0 ** 2 * 2.0)
    assert np.abs(rec - x.astype(np.float64)).max() <= bound * 1.05 + np.abs(x).max() * 2.0 ** -23


def test_three_term_int8_split_zero_and_tiny():
    for x in (np.zeros(64, np.float32), np.full(64, 1e-38, np.float32)):
        s, q1, q2, q3 = _split3(x, False)
        assert s == 0 and not q1.any() and not q2.any() and not q3.any()


def test_w8_qlinear_forward_cpu_is_dequantize_then_the_serial_loop():
    """The function bench.py times as the CPU baseline: a fresh dequantise (float(code) * scale) into an fp32
    [OUT, IN] scratch, then the reference's serial triple loop (cpu_gemm.mojo:88-98), then the bias."""
    rng = np.random.default_rng(12)
    N, K, M = 37, 96, 3
    w = rng.integers(-127, 128, (N, K), dtype=np.int8)
    s = rng.uniform(1e-3, 1e-2, N).astype(np.float32)
    x = rng.standard_normal((M, K)).astype(np.float32)
    b = rng.standard_normal(N).astype(np.float32)
    y = O.w8_qlinear_forward_cpu(w, s, x, b)
    deq = w.astype(np.float32) * s[:, None]
    want = np.empty((M, N), np.float32)
    for m in range(M):
        for n in range(N):
            acc = np.float32(0)
            for k in range(K):  # k ascending, one fp32 accumulator, multiply and add rounded separately or fused
                acc = np.float32(acc + np.float32(x[m, k] * deq[n, k]))
            want[m, n] = np.float32(acc + b[n])
    exact = x.astype(np.float64) @ deq.astype(np.float64).T + b
    assert np.abs(y - exact).max() <= 1e-5 * np.abs(exact).max()
    # the serial order itself: equal to the loop above unless the C compiler fused multiply and add (then within an ulp or two)
    assert np.abs(y - want).max() <= 4e-7 * np.abs(exact).max()
    assert np.array_equal(O.w8_qlinear_forward_cpu(w, s, x), O.w8_qlinear_forward_cpu(w, s, x, np.zeros(N, np.float32)))


def test_swiglu_is_u_times_v_sigmoid_v():
    """Pinned by the closed form in fp64 and by the values that tell a wrong variant apart: silu(0) = 0,
    silu(v) -> v for large v, -> 0 for very negative v, (u, v) not interchangeable."""
    rng = np.random.default_rng(4)
    u = rng.standard_normal(4000).astype(np.float32) * 3
    v = rng.standard_normal(4000).astype(np.float32) * 4
    got = O.swiglu(u, v)
    want = u.astype(np.float64) * v.astype(np.float64) / (1.0 + np.exp(-v.astype(np.float64)))
    assert np.abs(got - want).max() <= 4e-7 * np.abs(want).max()
    assert np.abs(got - want).max() > 0  # fp32 arithmetic, not the fp64 formula retyped
    assert np.array_equal(O.swiglu(np.float32([2, 2, 2, -3]), np.float32([0, 100, -100, 1])),
                          np.float32([0, 200, -0.0, -3 * 0.7310585786]).astype(np.float32))
    assert not np.allclose(O.swiglu(u, v), O.swiglu(v, u))
    # the reference's grouping: u * (v * s), not (u * v) * s (they differ in the last bit now and then)
    s32 = np.float32(1) / (np.float32(1) + np.exp(-v).astype(np.float32))
    regroup = (u * v) * s32
    assert np.abs(got - regroup).max() <= 2e-7 * np.abs(want).max()


def test_fp8_cpu_forward_restatement_pinned():
    """`fp8_qlinear_forward_cpu` (the CPU baseline bench.py times: dequantize to an fp32 scratch, then the serial
    gemm_cpu, qlinear.mojo:416-426 / cpu_gemm.mojo:88-98, for e4m3 operands) against what fixes it: small-integer
    codes whose products and sums are exact in fp32 (so any order of summation gives the same bits as numpy's integer
    matmul), and the fp64 forward on random codes within fp32 summation error; a transposed operand or a dropped
    scale fails both."""
    rng = np.random.default_rng(5)
    table = O.e4m3_decode_table()
    ints = np.array([c for c in range(256) if np.isfinite(table[c]) and table[c] == np.round(table[c]) and abs(table[c]) <= 8], np.uint8)
    M, N, K = 3, 7, 64
    a = ints[rng.integers(0, len(ints), (M, K))]
    w = ints[rng.integers(0, len(ints), (N, K))]
    y = O.fp8_qlinear_forward_cpu(w, 2.0, a, 0.5)
    want = (table[a].astype(np.int64) @ table[w].astype(np.int64).T).astype(np.float32)  # 2.0 * 0.5 = 1
    assert np.array_equal(y, want)
    # random codes (NaN codes excluded), scales that are not powers of two
    codes = np.array([c for c in range(256) if np.isfinite(table[c])], np.uint8)
    M, N, K = 2, 33, 4096
    a = codes[rng.integers(0, len(codes), (M, K))]
    w = codes[rng.integers(0, len(codes), (N, K))]
    sa, sb = 0.013, 0.07
    y, ob = O.fp8_qlinear_forward_cpu(w, sb, a, sa, want_bf16=True)
    y64, _ = O.fp8_forward_f64(a, w, sa, sb, want_bf16=False)
    assert np.abs(y - y64).max() <= 2e-5 * np.abs(y64).max()
    assert np.array_equal(ob, O.bf16_bits(y))
