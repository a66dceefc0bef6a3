"""Pins the CPU oracle's Q4_0 half against the reference's golden vectors and
against library routines / closed forms.

The gates mirror the reference's own (tests/nn/quant/test_q4_0.mojo [1]-[4],
tests/nn/quant/test_qlinear.mojo): same fixture, same invariants, same bands.
Independent checkers used here: numpy's float16 (IEEE half), torch's bfloat16
cast, numpy's argmax / round / float64 matmul, and exact small-integer GEMMs.
"""
import os

import numpy as np
import pytest
import torch

from noeira_amd.safetensors_io import SafeTensors, SafeTensorsWriter, load_q4_blocks, q4_blocks_key
from oracle import oracle as O

FIX = "q4_0_rtn.safetensors"
FIX_SHA256 = "5ef9efac14f225cd6b2ed2fb37b6593d3eb22d2245f27f6eec7acad782a319d9"


@pytest.fixture(scope="module")
def fix(golden_dir):
    import hashlib
    path = os.path.join(golden_dir, FIX)
    assert hashlib.sha256(open(path, "rb").read()).hexdigest() == FIX_SHA256
    f = SafeTensors(path)
    return f.read_f32("w"), f.read("q"), f.read_f32("d")


def test_fixture_shapes(fix):
    w, q, d = fix
    assert w.shape == (25, 128) and q.shape == (25, 128) and d.shape == (25, 4)
    assert q.dtype == np.uint8 and q.max() <= 15


# [1] RTN == the reference's codes and scale BITS (test_q4_0.mojo:32-54)
def test_rtn_matches_reference_fixture(fix):
    w, q_ref, d_ref = fix
    q, d = O.quantize_rtn_q4_0(w)
    assert np.array_equal(q, q_ref), f"{(q != q_ref).sum()} codes differ"
    assert np.array_equal(d.view(np.uint32), d_ref.view(np.uint32)), "scale bits differ"


def test_rtn_fixture_edges_are_load_bearing(fix):
    """Each rule the fixture was built to pin really changes codes/scales when
    broken (numpy re-derivation with one rule flipped)."""
    w, q_ref, d_ref = fix
    g = w.reshape(25, 4, 32)

    def grid(first_max=True, trunc_bf16=False, recip=False, half_away=False):
        a = np.abs(g)
        idx = np.argmax(a, axis=2) if first_max else (31 - np.argmax(a[..., ::-1], axis=2))
        d = np.take_along_axis(g, idx[..., None], axis=2)[..., 0] / np.float32(-8)
        d = np.where(d == 0, np.float32(1e-8), d).astype(np.float32)
        b = d.view(np.uint32).astype(np.uint64)
        b = (b & 0xFFFF0000) if trunc_bf16 else ((b + 0x7FFF + ((b >> 16) & 1)) & 0xFFFF0000)
        d = b.astype(np.uint32).view(np.float32)
        t = (g * (np.float32(1) / d[..., None])) if recip else (g / d[..., None])
        r = (np.sign(t) * np.floor(np.abs(t) + np.float32(0.5))) if half_away else np.round(t)
        q = np.clip(r + np.float32(8), 0, 15).astype(np.uint8).reshape(25, 128)
        return q, d

    q0, d0 = grid()
    assert np.array_equal(q0, q_ref) and np.array_equal(d0.view(np.uint32), d_ref.view(np.uint32))
    for kw in (dict(first_max=False), dict(trunc_bf16=True), dict(recip=True), dict(half_away=True)):
        q1, d1 = grid(**kw)
        assert (q1 != q_ref).any() or (d1.view(np.uint32) != d_ref.view(np.uint32)).any(), kw


# scalar pieces vs library routines
def test_f16_value_exhaustive_vs_numpy():
    bits = np.arange(65536, dtype=np.uint16)
    got = O.f16_value(bits)
    want = bits.view(np.float16).astype(np.float32)
    nan = np.isnan(want)
    assert np.array_equal(np.isnan(got), nan)
    assert np.array_equal(got[~nan].view(np.uint32), want[~nan].view(np.uint32))


def test_f16_bits_vs_numpy():
    rng = np.random.default_rng(1)
    x = np.concatenate([
        rng.standard_normal(20000).astype(np.float32) * np.float32(10) ** rng.integers(-9, 6, 20000).astype(np.float32),
        np.array([0.0, -0.0, 65504.0, 65519.9, 65520.0, 65536.0, 1e9, -1e9, np.inf, -np.inf,
                  2.0 ** -24, 2.0 ** -25, 2.0 ** -25 * 1.0001, 2.0 ** -14, 2.0 ** -14 * 0.9999,
                  1e-8, 6.1e-5, 5.96e-8, 1.0009765625, 1.00048828125, 1.00146484375], np.float32),
        # every fp16 value and the midpoints between neighbours
        np.arange(0, 0x7C00, dtype=np.uint16).view(np.float16).astype(np.float32),
    ])
    h = np.arange(0, 0x7BFF, dtype=np.uint16)
    mid = (h.view(np.float16).astype(np.float64) + (h + 1).astype(np.uint16).view(np.float16).astype(np.float64)) / 2
    x = np.concatenate([x, mid.astype(np.float32), -mid.astype(np.float32)])
    with np.errstate(over="ignore"):
        want = x.astype(np.float16).view(np.uint16)
    got = O.f16_bits(x)
    assert np.array_equal(got, want), np.flatnonzero(got != want)[:10]
    # NaN stays a NaN
    assert (O.f16_bits(np.array([np.nan], np.float32))[0] & 0x7C00) == 0x7C00
    assert (O.f16_bits(np.array([np.nan], np.float32))[0] & 0x03FF) != 0


def test_bf16_round_vs_torch():
    rng = np.random.default_rng(2)
    x = rng.standard_normal(50000).astype(np.float32) * np.float32(10) ** rng.integers(-20, 20, 50000).astype(np.float32)
    ties = (np.arange(0x3E80, 0x3E90, dtype=np.uint32) << 16 | 0x8000).view(np.float32)
    x = np.concatenate([x, ties, -ties, np.array([0, -0.0, np.inf, -np.inf, 3.4e38], np.float32)])
    want = torch.from_numpy(x).to(torch.bfloat16).view(torch.int16).numpy().view(np.uint16)
    assert np.array_equal(O.bf16_bits(x), want)
    assert O.bf16_bits(np.array([np.nan], np.float32))[0] == 0x7FC0  # safetensors.mojo:584
    assert np.array_equal(O.bf16_round(x).view(np.uint32), want.astype(np.uint32) << 16)


def test_round_half_even_vs_numpy():
    xs = np.concatenate([np.arange(-20, 20, 0.25), np.random.default_rng(3).uniform(-9, 9, 2000)]).astype(np.float32)
    for v in xs:
        assert O.round_half_even(v) == np.round(np.float32(v)), v


# [2] pack ∘ unpack identity incl. NaN / inf / subnormal scales (test_q4_0.mojo:57-100)
def test_pack_unpack_identity():
    rng = np.random.default_rng(7)
    for t in range(6):
        n, k = 1 + t, 32 * (1 + 2 * t)
        nb = n * O.q4_0_row_bytes(k)
        blocks = rng.integers(0, 256, nb, dtype=np.uint8)
        blocks[0:2] = [0x01, 0x7E]  # fp16 NaN 0x7E01
        if nb >= 36:
            blocks[18:20] = [0x00, 0x7C]  # +inf
        if nb >= 54:
            blocks[36:38] = [0x03, 0x00]  # subnormal
        q, bits = O.unpack_q4_0(blocks, n, k)
        again = O.pack_q4_0(q, bits)
        assert np.array_equal(again.ravel(), blocks)
        q2 = rng.integers(0, 16, (n, k), dtype=np.uint8)
        b2 = rng.integers(0, 65536, (n, k // 32), dtype=np.uint16)
        q3, b3 = O.unpack_q4_0(O.pack_q4_0(q2, b2), n, k)
        assert np.array_equal(q3, q2) and np.array_equal(b3, b2)


def test_block_layout_by_hand():
    """One block written out by hand from the format text (q4_0.mojo:1-8):
    scale LE fp16, byte j = element j (low nibble) | element j+16 (high)."""
    q = np.arange(32, dtype=np.uint8).reshape(1, 32) % 16
    q[0, 16:] = (q[0, 16:] + 5) % 16
    bits = np.array([[0x3C00 | 0x0123]], np.uint16)
    blk = O.pack_q4_0(q, bits).ravel()
    assert blk[0] == 0x23 and blk[1] == 0x3D
    for j in range(16):
        assert blk[2 + j] == (q[0, j] | (q[0, j + 16] << 4))
    # the three restatements of q4_0_value in the reference's benchmarks
    # (noeira_max/qmatmul/bench_qint4_orin.mojo:38-44) give the same element
    d = np.array([0x3D23], np.uint16).view(np.float16).astype(np.float32)[0]
    deq = O.dequantize_q4_0(blk, 1, 32)
    for j in range(32):
        byte = blk[2 + (j % 16)]
        nib = (byte & 0xF) if j < 16 else (byte >> 4)
        assert deq[0, j] == (np.float32(nib) - np.float32(8)) * d


# [3] dequantize == (q - 8) d bitwise; RTN within d/2 (test_q4_0.mojo:103-156)
def test_dequantize_closed_form_and_rtn_error(fix):
    w, _, _ = fix
    n, k = w.shape
    blocks = O.rtn_q4_0_blocks(w)
    assert blocks.size == n * O.q4_0_row_bytes(k)
    deq = O.dequantize_q4_0(blocks, n, k)
    q, bits = O.unpack_q4_0(blocks, n, k)
    d_np = bits.view(np.float16).astype(np.float32)  # numpy's half decode, independent of the oracle's
    want = (q.astype(np.float32).reshape(n, k // 32, 32) - np.float32(8)) * d_np[..., None]
    assert np.array_equal(deq.view(np.uint32), want.reshape(n, k).view(np.uint32))
    q_rtn, d_rtn = O.quantize_rtn_q4_0(w)
    moved = d_np != d_rtn
    assert (np.abs(d_rtn[moved]) < 6.103515625e-05).all()  # only below fp16's normal range
    dd = np.repeat(d_np, 32, axis=1)
    ok = (dd != 0) & (np.repeat(~moved, 32, axis=1)) & (q != 0) & (q != 15)
    err = np.abs(deq.astype(np.float64) - w.astype(np.float64))[ok] / np.abs(dd.astype(np.float64))[ok]
    assert err.max() <= 0.5 + 1e-6


def test_zero_scale_group_decodes_to_zero():
    """d = 0 decodes to 0 whatever the nibbles (qlinear.mojo:32-34)."""
    rng = np.random.default_rng(11)
    blocks = rng.integers(0, 256, 4 * 18, dtype=np.uint8)
    blocks[0::18] = 0
    blocks[1::18] = 0
    assert not O.dequantize_q4_0(blocks, 1, 128).any()


# [4] U8 safetensors round trip (test_q4_0.mojo:159-178)
def test_u8_safetensors_round_trip(tmp_path):
    n, k = 3, 64
    blocks = np.array([(i * 37 + 11) % 256 for i in range(n * O.q4_0_row_bytes(k))], np.uint8)
    wr = SafeTensorsWriter()
    wr.add_u8(q4_blocks_key("proj"), [n, O.q4_0_row_bytes(k)], blocks)
    path = str(tmp_path / "u8.safetensors")
    wr.save(path)
    f = SafeTensors(path)
    assert f.dtype_of("proj.q4_0") == "U8" and f.shape("proj.q4_0") == [n, O.q4_0_row_bytes(k)]
    assert np.array_equal(f.read_raw("proj.q4_0"), blocks)
    assert np.array_equal(load_q4_blocks(f, "proj", k, n), blocks)
    with pytest.raises(ValueError, match=r"expected \[4, 36\]"):
        load_q4_blocks(f, "proj", k, 4)
    # the same bytes through the safetensors package's own reader
    from safetensors.numpy import load_file
    assert np.array_equal(load_file(path)["proj.q4_0"].ravel(), blocks)


# gemm_cpu (cpu_gemm.mojo:88-98)
def test_gemm_cpu_exact_on_small_integers():
    rng = np.random.default_rng(5)
    M, N, K = 5, 7, 33
    a = rng.integers(-8, 9, (M, K)).astype(np.float32)
    b = rng.integers(-8, 9, (K, N)).astype(np.float32)
    c0 = rng.integers(-8, 9, (M, N)).astype(np.float32)
    want = (2 * (a.astype(np.int64) @ b.astype(np.int64)) + 3 * c0.astype(np.int64)).astype(np.float32)
    for ta in (False, True):
        for tb in (False, True):
            A = np.ascontiguousarray(a.T) if ta else a
            B = np.ascontiguousarray(b.T) if tb else b
            c = c0.copy()
            O.gemm_cpu(ta, tb, M, N, K, 2.0, A, A.shape[1], B, B.shape[1], 3.0, c, N)
            assert np.array_equal(c, want), (ta, tb)
    # beta == 0 does not read c (NaNs in c must not leak)
    c = np.full((M, N), np.nan, np.float32)
    O.gemm_cpu(False, False, M, N, K, 1.0, a, K, b, N, 0.0, c, N)
    assert np.array_equal(c, (a.astype(np.int64) @ b.astype(np.int64)).astype(np.float32))


def test_gemm_cpu_is_serial_k_ascending():
    """One accumulator, k ascending: reproduces numpy's sequential fp32 sum."""
    rng = np.random.default_rng(6)
    K = 257
    a = rng.standard_normal((1, K)).astype(np.float32)
    b = rng.standard_normal((1, K)).astype(np.float32)
    acc = np.float32(0)
    for k in range(K):
        acc = np.float32(acc + np.float32(a[0, k] * b[0, k]))
    c = np.zeros((1, 1), np.float32)
    O.gemm_cpu(False, True, 1, 1, K, 1.0, a, K, b, K, 0.0, c, 1)
    assert c[0, 0] == acc


# QLinear.forward["cpu"] at the reference's shapes and band (test_qlinear.mojo:15-29)
@pytest.mark.parametrize("IN,OUT", [(960, 960), (960, 320), (960, 2560), (2560, 960)])
def test_qlinear_forward_cpu_vs_fp64_and_twin(IN, OUT):
    T = 7
    rng = np.random.default_rng(IN * 7 + OUT)
    w = (rng.standard_normal((OUT, IN)) * 0.05).astype(np.float32)
    x = rng.standard_normal((T, IN)).astype(np.float32)
    gy = rng.standard_normal((T, OUT)).astype(np.float32)
    blocks = O.rtn_q4_0_blocks(w)
    deq = O.dequantize_q4_0(blocks, OUT, IN)
    y = O.qlinear_forward_cpu(blocks, IN, OUT, x)
    exact = x.astype(np.float64) @ deq.astype(np.float64).T          # numpy fp64, not the oracle's loop
    assert np.abs(y - exact).max() / np.abs(exact).max() < 1e-5
    assert np.abs(O.dense_forward_f64(deq, x) - exact).max() <= 1e-9 * np.abs(exact).max()
    # the fp32 "Linear over deq(W)^T" twin: same GEMM, so bit-identical here
    twin = np.zeros((T, OUT), np.float32)
    O.gemm_cpu(False, False, T, OUT, IN, 1.0, x, IN, np.ascontiguousarray(deq.T), OUT, 0.0, twin, OUT)
    assert O.rel_max(y, twin) < 1e-5
    gx = O.qlinear_vjp_cpu(blocks, IN, OUT, gy)
    gexact = gy.astype(np.float64) @ deq.astype(np.float64)
    assert np.abs(gx - gexact).max() / np.abs(gexact).max() < 1e-5


def test_rel_max_metric():
    a = np.array([1.0, 2.0, -4.5], np.float32)
    b = np.array([1.0, 2.5, -4.0], np.float32)
    assert O.rel_max(a, b) == pytest.approx(0.5 / 4.0)
    assert O.rel_max(np.zeros(3, np.float32), np.zeros(3, np.float32)) == 0.0


def test_cast_pad_and_slice_cast():
    rng = np.random.default_rng(8)
    x = rng.standard_normal((5, 96)).astype(np.float32)
    xb = O.cast_pad_bf16(x, 128)
    want = torch.from_numpy(x).to(torch.bfloat16).view(torch.int16).numpy().view(np.uint16)
    assert np.array_equal(xb[:, :96], want) and not xb[:, 96:].any()
    back = O.slice_cast_f32(xb, 96)
    assert np.array_equal(back, torch.from_numpy(x).to(torch.bfloat16).float().numpy())
