"""The caller's side of the path (the SmolVLA text layer, noeira/deep_agents/smolvla/fused.mojo:287-363):
gate | up with the SwiGLU between them and `down` as one launch (nq_fuse_glu), against the oracle's restatements of
`QLinear.forward["cpu"]` and `SwiGLU.forward["cpu"]`; and the reference's two-layer tower gate
(tests/deep_agents/smolvla/q4_tower_common.mojo: every linear a QLinear against the fp32 tower over deq(W)), forward
half, with q | k | v and gate | up + SwiGLU fused.  Bands as the reference's: 1e-5 of the largest reference value for
the fp32 path, 3e-2 for bf16 activations (q4_tower_common.mojo:137-138)."""
import numpy as np
import pytest
import torch

from noeira_amd import _lib as L
from noeira_amd import formats as F
from noeira_amd.qlinear import FusedGLU, FusedRows, QLinear, W4GroupLinear, W8Linear
from oracle import oracle as O
import refw

pytestmark = pytest.mark.gpu


def q4(rng, IN, OUT, std=0.05):
    lin = QLinear(IN, OUT)
    w = (rng.standard_normal((OUT, IN)) * std).astype(np.float32)
    lin.set_weight(w)
    # deq(W) by the oracle alone: its round-to-nearest quantiser, then its dequantiser
    lin.ref_deq = lambda: refw.q4_0(O.rtn_q4_0_blocks(w), OUT, IN)
    return lin


def rel_max(a, b):
    return float((a.double() - b.double()).abs().max() / b.double().abs().max())


# ── gate | up + SwiGLU in one launch ─────────────────────────────────────────────────────────────
@pytest.mark.parametrize("M", [1, 7, 135])
def test_glu_q4_0_against_the_oracle(M):
    rng = np.random.default_rng(100 + M)
    IN, H = 960, 2560
    gate, up = q4(rng, IN, H), q4(rng, IN, H)
    glu = FusedGLU(gate, up)
    x = rng.standard_normal((M, IN)).astype(np.float32)
    y = glu.forward(torch.from_numpy(x).cuda()).cpu().numpy()
    g = O.qlinear_forward_cpu(gate.blocks(), IN, H, x)
    u = O.qlinear_forward_cpu(up.blocks(), IN, H, x)
    want = O.swiglu(u, g)
    assert y.shape == (M, H)
    assert O.rel_max(y, want) < 1e-5
    assert np.array_equal(glu.forward(torch.from_numpy(x).cuda()).cpu().numpy(), y)  # repeated call: same bits


@pytest.mark.parametrize("kind,IN,H,M", [("q4_0", 960, 2560, 600), ("q4_0", 960, 2560, 1120), ("q4_0", 2048, 304, 1),
                                         ("q4_0", 4096, 5504, 1), ("q4_0", 4096, 5504, 3), ("w8", 512, 1600, 1),
                                         ("w8", 512, 1600, 100), ("w4g", 960, 2560, 1), ("w4g", 960, 2560, 256),
                                         ("w4g", 2560, 960, 33)])
@pytest.mark.parametrize("xdt", [torch.float32, torch.bfloat16])
def test_glu_against_fp64_over_the_dequantised_weights(kind, IN, H, M, xdt):
    """Every kernel that carries the SwiGLU epilogue (one row: lane groups of 16, 32 and 64 lanes; a few rows; hundreds
    of rows), every format nq_fuse_glu takes."""
    rng = np.random.default_rng(IN + H + M)
    layers = []
    for _ in range(2):
        if kind == "q4_0":
            layers.append(q4(rng, IN, H))
        elif kind == "w8":
            lin = W8Linear(IN, H)
            wq, ws = F.quantize_w8_channel((rng.standard_normal((H, IN)) * 0.05).astype(np.float32))
            lin.set_weight(wq, ws)
            lin.ref_deq = lambda wq=wq, ws=ws: refw.w8(wq, ws)
            layers.append(lin)
        else:
            lin = W4GroupLinear(IN, H, 128)
            q, s, z = F.quantize_w4g_asym((rng.standard_normal((H, IN)) * 0.05).astype(np.float32), 128)
            codes, zps = F.pack_w4g(q, z)
            lin.set_weight(codes, s, zps)
            lin.ref_deq = lambda codes=codes, s=s, zps=zps: refw.w4g(codes, s, zps, H, IN, 128)
            layers.append(lin)
    gate, up = layers
    glu = FusedGLU(gate, up)
    x = torch.from_numpy(rng.standard_normal((M, IN)).astype(np.float32)).to(xdt).cuda()
    g = x.double() @ gate.ref_deq().T
    u = x.double() @ up.ref_deq().T
    want = u * (g * torch.sigmoid(g))
    y = glu.forward(x)
    assert y.shape == (M, H) and y.dtype == torch.float32
    assert rel_max(y, want) < 1e-5
    # the two halves as two outputs of one row-fused launch, then SwiGLU apart: the same values
    yg, yu = FusedRows([gate, up]).forward(x)
    apart = O.swiglu(yu.cpu().numpy(), yg.cpu().numpy())
    assert np.abs(y.cpu().numpy() - apart).max() <= 4e-6 * np.abs(apart).max()
    # bf16 out: the RNE bf16 of a value within the band
    yb = glu.forward(x, out_dtype=torch.bfloat16)
    assert float((yb.double() - want).abs().max()) <= 2.0 ** -8 * float(want.abs().max()) + 1e-5 * float(want.abs().max())


def test_glu_lifecycle_and_errors():
    rng = np.random.default_rng(5)
    gate, up = q4(rng, 64, 96), q4(rng, 64, 96)
    glu = FusedGLU(gate, up)
    x = torch.zeros((2, 64), device="cuda")
    lib = L.lib()
    import ctypes as C

    y = torch.empty((2, 96), device="cuda")
    null = C.c_void_p(0)

    def fwd(h, epi, bias=null):
        return lib.nq_forward(h, C.c_void_p(x.data_ptr()), L.DT_F32, null, C.c_void_p(y.data_ptr()), L.DT_F32, 2, bias,
                              L.DT_F32, epi, null)

    assert fwd(glu._h, L.EPI_NONE) == L.NQ_ERR_INVALID and "NQ_EPI_SWIGLU only" in L.last_error()
    assert fwd(gate._h, L.EPI_SWIGLU) == L.NQ_ERR_INVALID and "nq_fuse_glu" in L.last_error()
    assert fwd(glu._h, L.EPI_SWIGLU, C.c_void_p(y.data_ptr())) == L.NQ_ERR_INVALID and "no bias" in L.last_error()
    assert fwd(glu._h, L.EPI_SWIGLU) == L.NQ_OK
    with pytest.raises(L.NQError, match="share format, IN, OUT"):
        FusedGLU(gate, q4(rng, 64, 64))
    with pytest.raises(L.NQError, match="cannot be fused again"):
        FusedGLU(glu, up)
    buf = np.empty(10, np.uint8)
    assert lib.nq_get_blocks(glu._h, buf.ctypes.data_as(C.c_void_p), 10) == L.NQ_ERR_NO_BLOCKS
    # zero activations: silu(0) * up(0) = 0, and the sources may go
    del gate, up
    assert torch.equal(glu.forward(x), torch.zeros((2, 96), device="cuda"))


# ── the two-layer tower gate, forward half ───────────────────────────────────────────────────────
P, W, FF, HEADS, NKV, HD, LAYERS = 6, 64, 96, 2, 1, 32, 2
THETA = 100000.0


def rmsnorm(x, gamma):
    return x * torch.rsqrt(x.pow(2).mean(-1, keepdim=True) + 1e-5) * gamma


def rope(t, heads):
    """[P, heads * HD] -> rotated, half-split pairs, positions 0 .. P - 1."""
    t = t.view(P, heads, HD)
    half = HD // 2
    inv = THETA ** (-torch.arange(half, dtype=torch.float64, device=t.device) / half)
    ang = torch.arange(P, dtype=torch.float64, device=t.device)[:, None] * inv[None, :]
    c, s = torch.cos(ang).to(t.dtype)[:, None, :], torch.sin(ang).to(t.dtype)[:, None, :]
    a, b = t[..., :half], t[..., half:]
    return torch.cat([a * c - b * s, b * c + a * s], -1).reshape(P, heads * HD)


def attention(q, k, v):
    q, k, v = q.view(P, HEADS, HD), k.view(P, NKV, HD), v.view(P, NKV, HD)
    k, v = k.repeat_interleave(HEADS // NKV, 1), v.repeat_interleave(HEADS // NKV, 1)
    sc = torch.einsum("phd,qhd->hpq", q, k) / HD ** 0.5
    mask = torch.ones((P, P), dtype=torch.bool, device=q.device).tril()
    sc = sc.masked_fill(~mask, float("-inf"))
    return torch.einsum("hpq,qhd->phd", torch.softmax(sc, -1), v).reshape(P, HEADS * HD)


class Tower:
    """Every linear a QLinear (`quant`), or a dense fp64 matrix holding deq(W) (`dense`), zero bias either way."""

    def __init__(self, rng):
        self.layers = []
        for _ in range(LAYERS):
            lw = {n: q4(rng, i, o, 0.2) for n, (i, o) in dict(q=(W, HEADS * HD), k=(W, NKV * HD), v=(W, NKV * HD),
                                                               o=(HEADS * HD, W), gate=(W, FF), up=(W, FF),
                                                               down=(FF, W)).items()}
            lw["qkv"] = FusedRows([lw["q"], lw["k"], lw["v"]])
            lw["glu"] = FusedGLU(lw["gate"], lw["up"])
            lw["g1"] = torch.from_numpy(1 + 0.1 * rng.standard_normal(W)).cuda()
            lw["g2"] = torch.from_numpy(1 + 0.1 * rng.standard_normal(W)).cuda()
            self.layers.append(lw)
        self.gf = torch.from_numpy(1 + 0.1 * rng.standard_normal(W)).cuda()

    def run(self, x, mode):
        """mode: "dense" (fp64 over deq(W)), "f32" (the library, fp32 at every boundary), "bf16" (the library with
        bf16 in and bf16 out at every linear).  Returns (final norm, [(post-RoPE K, V) per layer])."""
        dt = {"dense": torch.float64, "f32": torch.float32, "bf16": torch.float32}[mode]
        x = x.to(dt)
        cache = []

        def lin(layer, h):
            if mode == "dense":
                return h @ layer.ref_deq().T
            if mode == "bf16":
                return layer.forward(h.to(torch.bfloat16).contiguous(), out_dtype=torch.bfloat16).float()
            return layer.forward(h.contiguous())

        for lw in self.layers:
            h = rmsnorm(x, lw["g1"].to(dt))
            if mode == "dense":
                q, k, v = lin(lw["q"], h), lin(lw["k"], h), lin(lw["v"], h)
            elif mode == "bf16":
                q, k, v = [t.float() for t in lw["qkv"].forward(h.to(torch.bfloat16).contiguous(), out_dtype=torch.bfloat16)]
            else:
                q, k, v = lw["qkv"].forward(h.contiguous())
            qr, kr = rope(q, HEADS), rope(k, NKV)
            cache.append((kr, v))
            x2 = x + lin(lw["o"], attention(qr, kr, v))
            h2 = rmsnorm(x2, lw["g2"].to(dt))
            if mode == "dense":
                g, u = lin(lw["gate"], h2), lin(lw["up"], h2)
                glu = u * (g * torch.sigmoid(g))
            elif mode == "bf16":
                glu = lw["glu"].forward(h2.to(torch.bfloat16).contiguous(), out_dtype=torch.bfloat16).float()
            else:
                glu = lw["glu"].forward(h2.contiguous())
            x = x2 + lin(lw["down"], glu)
        return rmsnorm(x, self.gf.to(dt)), cache


@pytest.mark.parametrize("mode,tol", [("f32", 1e-5), ("bf16", 3e-2)])
def test_two_layer_tower_against_the_dense_tower_over_deq_w(mode, tol):
    rng = np.random.default_rng(11)
    tower = Tower(rng)
    x = torch.from_numpy(rng.random((P, W)) - 0.5).cuda()
    out_d, cache_d = tower.run(x, "dense")
    out_q, cache_q = tower.run(x, mode)
    assert rel_max(out_q, out_d) < tol
    for (kq, vq), (kd, vd) in zip(cache_q, cache_d):
        assert rel_max(kq, kd) < tol and rel_max(vq, vd) < tol
    # a projection dispatched to the wrong layer shows as an O(1) difference: swap k and v of layer 0 and see it
    lw = tower.layers[0]
    lw["qkv"] = FusedRows([lw["q"], lw["v"], lw["k"]])
    out_w, _ = tower.run(x, mode)
    assert rel_max(out_w, out_d) > 10 * tol
