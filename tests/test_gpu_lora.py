"""A frozen LoRA adapter beside a quantized linear (QLoRA inference), on the GPU
through the C ABI, against the CPU oracle.

Gates as the reference's tests/nn/quant/test_qlora.mojo and
tests/nn/peft/test_lora.mojo [1]: B = 0 leaves the base layer's output bit for
bit; with a nonzero B the result equals LoRA over deq(W) within the fp32 band
(1e-5 of the largest reference value); rank padding is exact.
"""
import numpy as np
import pytest
import torch

from noeira_amd import _lib as L
from noeira_amd.lora import LoRAAdapter
from noeira_amd.qlinear import QLinear
from oracle import oracle as O

pytestmark = pytest.mark.gpu

BAND = 1e-5


def make(rng, IN, OUT, R, pad=16, zero_b=False):
    ad = LoRAAdapter(IN, OUT, R, PAD_R=pad, alpha=2.0 * R)
    bound = 1.0 / np.sqrt(IN)
    a = ((rng.random((IN, R)) * 2 - 1) * bound).astype(np.float32)       # PEFT's init (lora.mojo:232-237)
    b = np.zeros((R, OUT), np.float32) if zero_b else (rng.standard_normal((R, OUT)) * 0.05).astype(np.float32)
    ad.set_params(a, b)
    return ad, a, b


# the reference's shapes (test_qlora.mojo:15-19): small, k / v, down; T = 7; plus one token and a prefill
@pytest.mark.parametrize("IN,OUT,T,R", [(64, 96, 7, 4), (960, 320, 7, 16), (2560, 960, 7, 16),
                                          (960, 2560, 1, 16), (960, 960, 135, 8), (64, 300, 33, 40)])
@pytest.mark.parametrize("xdt", [torch.float32, torch.bfloat16])
def test_qlora_forward(IN, OUT, T, R, xdt):
    rng = np.random.default_rng(IN + OUT + T + R)
    w = (rng.standard_normal((OUT, IN)) * 0.05).astype(np.float32)
    base = QLinear(IN, OUT)
    base.set_weight(w)
    x = torch.from_numpy(rng.standard_normal((T, IN)).astype(np.float32)).to(xdt).cuda()
    y_base = base.forward(x)
    # B = 0: bit for bit the bare QLinear
    ad0, _, _ = make(rng, IN, OUT, R, zero_b=True)
    y0 = ad0.forward_add(x, y_base.clone())
    assert torch.equal(y0, y_base)
    # nonzero B: LoRA over deq(W) (qlora_common.mojo), oracle on the same inputs
    ad, a, b = make(rng, IN, OUT, R)
    assert ad.scale() == 2.0
    y = ad.forward_add(x, y_base.clone()).cpu().numpy()
    xf = x.float().cpu().numpy()
    want = O.qlinear_forward_cpu(base.blocks(), IN, OUT, xf)
    want = O.lora_forward_add(xf, a, b, ad.scale(), want)
    assert O.rel_max(y, want) < BAND, O.rel_max(y, want)
    # the adapter's share alone, against fp64
    share = 2.0 * (xf.astype(np.float64) @ a.astype(np.float64)) @ b.astype(np.float64)
    got = y.astype(np.float64) - y_base.cpu().numpy().astype(np.float64)
    assert np.abs(got - share).max() <= 2e-6 * max(np.abs(share).max(), np.abs(y).max())


def test_rank_padding_is_exact_and_rslora_scale():
    rng = np.random.default_rng(3)
    IN, OUT, T, R = 96, 70, 5, 3
    x = torch.from_numpy(rng.standard_normal((T, IN)).astype(np.float32)).cuda()
    y0 = torch.from_numpy(rng.standard_normal((T, OUT)).astype(np.float32)).cuda()
    padded, a, b = make(rng, IN, OUT, R, pad=16)
    bare = LoRAAdapter(IN, OUT, R, PAD_R=1, alpha=2.0 * R)
    bare.set_params(a, b)
    assert padded.R_PAD == 16 and bare.R_PAD == 3
    # (R_PAD = 16 takes the kernel with 16-byte loads, 3 the general one: the same values to the last bits' worth)
    yp, yb = padded.forward_add(x, y0.clone()), bare.forward_add(x, y0.clone())
    assert float((yp - yb).abs().max()) <= 2e-6 * float(yb.abs().max())
    # the pad is exact: B's pad rows are zero, so whatever A's pad columns hold adds exact zeros
    padded.lora_A[:, R:] = torch.from_numpy(rng.standard_normal((IN, 16 - R)).astype(np.float32)).cuda()
    assert torch.equal(padded.forward_add(x, y0.clone()), yp)
    rs = LoRAAdapter(IN, OUT, 4, RSLORA=True, alpha=8.0)
    assert rs.scale() == 4.0 and LoRAAdapter(IN, OUT, 4, alpha=8.0).scale() == 2.0


def test_merged_adapter_adds_nothing_and_errors():
    rng = np.random.default_rng(4)
    ad, _, _ = make(rng, 64, 32, 4)
    x = torch.from_numpy(rng.standard_normal((2, 64)).astype(np.float32)).cuda()
    y = torch.ones((2, 32), device="cuda")
    ad.merged = True
    assert torch.equal(ad.forward_add(x, y.clone()), y)
    ad.merged = False
    with pytest.raises(L.NQError, match="fp32"):
        ad.forward_add(x, y.to(torch.bfloat16))
    with pytest.raises(L.NQError, match=r"\[T, IN\]"):
        ad.forward_add(x[:, :63].contiguous(), y)
    with pytest.raises(L.NQError, match="rank"):
        LoRAAdapter(64, 32, 0)
    with pytest.raises(L.NQError, match="expected A"):
        ad.set_params(np.zeros((64, 5), np.float32), np.zeros((4, 32), np.float32))


# ---- the adapter folded into the base launch (nq_forward_lora) ---------------------------------------------
# the reference's shapes again, at T = 7 and at the prefill's 135 tokens, on layers that prefer the kernel the fold
# rides on (2 .. 512 rows), plus the default dispatch: folded on a wide layer at T = 135, two launches elsewhere
@pytest.mark.parametrize("IN,OUT,T,R,prefer", [(960, 320, 7, 16, True), (2560, 960, 7, 16, True), (960, 960, 135, 8, True),
                                                 (960, 2560, 135, 16, False), (960, 2560, 2, 16, True),
                                                 (960, 320, 135, 16, False), (64, 96, 7, 4, True), (992, 100, 33, 3, True),
                                                 (4096, 512, 40, 16, True), (4224, 64, 20, 16, True),
                                                 (2048, 10240, 33, 16, False)])  # (folded by default: bf16 x over a large layer)
@pytest.mark.parametrize("xdt", [torch.float32, torch.bfloat16])
def test_qlora_one_call(IN, OUT, T, R, prefer, xdt):
    rng = np.random.default_rng(IN + OUT + T + R + 1)
    w = (rng.standard_normal((OUT, IN)) * 0.05).astype(np.float32)
    base = QLinear(IN, OUT, prefer_tile=prefer)
    base.set_weight(w)
    bias = torch.from_numpy((rng.standard_normal(OUT) * 0.1).astype(np.float32)).cuda()
    x = torch.from_numpy(rng.standard_normal((T, IN)).astype(np.float32)).to(xdt).cuda()
    y_base = base.forward(x, bias=bias)
    # B = 0: bit for bit the bare QLinear (test_qlora.mojo: b0_fwd_diff == 0)
    ad0, _, _ = make(rng, IN, OUT, R, zero_b=True)
    assert torch.equal(ad0.forward_with(base, x, bias=bias), y_base)
    # nonzero B: LoRA over deq(W), oracle on the same inputs, band 1e-5
    ad, a, b = make(rng, IN, OUT, R)
    y = ad.forward_with(base, x, bias=bias)
    assert torch.equal(ad.forward_with(base, x, bias=bias), y)
    xf = x.float().cpu().numpy()
    want = O.qlinear_forward_cpu(base.blocks(), IN, OUT, xf) + bias.cpu().numpy()
    want = O.lora_forward_add(xf, a, b, ad.scale(), want)
    assert O.rel_max(y.cpu().numpy(), want) < BAND, O.rel_max(y.cpu().numpy(), want)
    # the adapter's share alone, against fp64
    share = 2.0 * (xf.astype(np.float64) @ a.astype(np.float64)) @ b.astype(np.float64)
    got = y.double().cpu().numpy() - y_base.double().cpu().numpy()
    assert np.abs(got - share).max() <= 2e-6 * max(np.abs(share).max(), np.abs(want).max())
    # and the two-launch form gives the same values
    two = ad.forward_add(x, y_base.clone())
    assert float((two - y).abs().max()) <= 2e-6 * float(two.abs().max())


@pytest.mark.parametrize("R,pad", [(8, 8), (3, 1), (16, 16)])
@pytest.mark.parametrize("xdt", [torch.float32, torch.bfloat16])
def test_qlora_one_call_rank_as_stored(R, pad, xdt):
    """The folded call reads A [IN, R_PAD] in 16-byte pieces when R_PAD is 16 and element by element otherwise (R_PAD
    8 and 3 here): the same values either way, B = 0 bit for bit the base."""
    rng = np.random.default_rng(R * 31 + pad)
    IN, OUT, T = 960, 2560, 135
    base = QLinear(IN, OUT)
    base.set_weight((rng.standard_normal((OUT, IN)) * 0.05).astype(np.float32))
    x = torch.from_numpy(rng.standard_normal((T, IN)).astype(np.float32)).to(xdt).cuda()
    y_base = base.forward(x)
    ad0, _, _ = make(rng, IN, OUT, R, pad=pad, zero_b=True)
    assert torch.equal(ad0.forward_with(base, x), y_base)
    ad, a, b = make(rng, IN, OUT, R, pad=pad)
    y = ad.forward_with(base, x)
    xf = x.float().cpu().numpy()
    want = O.lora_forward_add(xf, a, b, ad.scale(), O.qlinear_forward_cpu(base.blocks(), IN, OUT, xf))
    assert O.rel_max(y.cpu().numpy(), want) < BAND


def test_qlora_one_call_bf16_out_and_errors():
    rng = np.random.default_rng(5)
    IN, OUT, T = 960, 2560, 135
    base = QLinear(IN, OUT)
    base.set_weight((rng.standard_normal((OUT, IN)) * 0.05).astype(np.float32))
    ad, a, b = make(rng, IN, OUT, 16)
    x = torch.from_numpy(rng.standard_normal((T, IN)).astype(np.float32)).to(torch.bfloat16).cuda()
    y32 = ad.forward_with(base, x)
    yb = ad.forward_with(base, x, out_dtype=torch.bfloat16)       # folded: bf16 in, bf16 out
    assert torch.equal(yb, y32.to(torch.bfloat16))
    narrow = QLinear(IN, 320)
    narrow.set_weight((rng.standard_normal((320, IN)) * 0.05).astype(np.float32))
    adn, _, _ = make(rng, IN, 320, 16)
    # not folded here: the adapter adds into fp32 only.  The answer comes before anything is launched: y is untouched
    ybn = torch.full((T, 320), 7.0, dtype=torch.bfloat16, device="cuda")
    with pytest.raises(L.NQError, match="second launch"):
        adn.forward_with(narrow, x, out=ybn, out_dtype=torch.bfloat16)
    torch.cuda.synchronize()
    assert bool((ybn == 7.0).all())
    with pytest.raises(L.NQError, match="differ in shape"):
        adn.forward_with(base, x)


# ── adapters on row-fused layers: a decoder layer's projections with all seven adapters ─────────────────────────
def _q4(rng, IN, OUT):
    w = (rng.standard_normal((OUT, IN)) * 0.05).astype(np.float32)
    lin = QLinear(IN, OUT)
    lin.set_weight(w)
    return lin


def _oracle_proj(lin, x_host, ad):
    """`proj_fwd` on the CPU: the oracle's QLinear forward, then its adapter's share (a, b logical blocks)."""
    want = O.qlinear_forward_cpu(lin.blocks(), lin.IN, lin.OUT, x_host)
    if ad is not None:
        adapter, a, b = ad
        want = O.lora_forward_add(x_host, a, b, adapter.scale(), want)
    return want


@pytest.mark.parametrize("T", [1, 17, 135])
@pytest.mark.parametrize("xdt", [torch.float32, torch.bfloat16])
def test_fused_rows_with_an_adapter_per_part(T, xdt):
    """q | k | v of the caller's text layer (960 -> 960 / 320 / 320) with R = 16 adapters on all three: every output
    is `LoRAAdapter.forward_add` over `QLinear.forward` (oracle, 1e-5 of the largest value); B = 0 on every part, and
    no adapter at all, leave the bits of the adapter-free fused call; a part without an adapter keeps its base bits
    while its neighbours get their shares."""
    from noeira_amd.qlinear import FusedRows

    rng = np.random.default_rng(1000 + T)
    IN, outs = 960, (960, 320, 320)
    parts = [_q4(rng, IN, n) for n in outs]
    fused = FusedRows(parts)
    x = torch.from_numpy(rng.standard_normal((T, IN)).astype(np.float32)).to(xdt).cuda()
    xh = x.float().cpu().numpy()
    base = [y.clone() for y in fused.forward(x)]
    ads = [make(rng, IN, n, 16) for n in outs]
    got = fused.forward_lora(x, [ad[0] for ad in ads])
    for lin, ad, y in zip(parts, ads, got):
        want = _oracle_proj(lin, xh, ad)
        assert O.rel_max(y.cpu().numpy(), want) < BAND
    zero = [make(rng, IN, n, 16, zero_b=True)[0] for n in outs]
    for y, yb in zip(fused.forward_lora(x, zero), base):
        assert torch.equal(y, yb)
    for y, yb in zip(fused.forward_lora(x, [None, None, None]), base):
        assert torch.equal(y, yb)
    mixed = fused.forward_lora(x, [ads[0][0], None, ads[2][0]])
    assert torch.equal(mixed[1], base[1])
    assert torch.equal(mixed[0], got[0]) and torch.equal(mixed[2], got[2])
    # a repeated call returns the same bits
    for y, y2 in zip(fused.forward_lora(x, [ad[0] for ad in ads]), got):
        assert torch.equal(y, y2)


@pytest.mark.parametrize("T", [1, 135])
@pytest.mark.parametrize("gdt", [torch.float32, torch.bfloat16])
def test_gate_up_with_adapters_through_swiglu(T, gdt):
    """gate | up (960 -> 2560 each) with an adapter on both and the SwiGLU applied to the SUMS, as the reference's
    caller orders it (fused.mojo:337-353: `proj_fwd[LORA_GATE]`, `proj_fwd[LORA_UP]`, then `glu`): against the
    oracle's projections, adapters and `swiglu`; with B = 0 the result is the adapter-free pair's SwiGLU."""
    from noeira_amd.qlinear import FusedRows

    rng = np.random.default_rng(2000 + T)
    IN, H = 960, 2560
    gate, up = _q4(rng, IN, H), _q4(rng, IN, H)
    pair = FusedRows([gate, up])
    x = torch.from_numpy(rng.standard_normal((T, IN)).astype(np.float32)).cuda()
    xh = x.cpu().numpy()
    adg, adu = make(rng, IN, H, 16), make(rng, IN, H, 16)
    out = pair.forward_lora(x, [adg[0], adu[0]], glu_dtype=gdt)
    assert out.shape == (T, H) and out.dtype == gdt
    want = O.swiglu(_oracle_proj(up, xh, adu), _oracle_proj(gate, xh, adg))
    tol = BAND if gdt == torch.float32 else 2.0 ** -8 + BAND
    assert O.rel_max(out.float().cpu().numpy(), want) < tol
    g0, u0 = pair.forward(x)
    zg, zu = make(rng, IN, H, 16, zero_b=True)[0], make(rng, IN, H, 16, zero_b=True)[0]
    out0 = pair.forward_lora(x, [zg, zu], glu_dtype=torch.float32)
    # (the base projections' own bits through SwiGLU; the device's exp and the oracle's differ in the last bit)
    assert O.rel_max(out0.cpu().numpy(), O.swiglu(u0.cpu().numpy(), g0.cpu().numpy())) < 1e-6
    assert torch.equal(out0, pair.forward_lora(x, [None, None], glu_dtype=torch.float32))
    # only one of the two carries an adapter
    out1 = pair.forward_lora(x, [None, adu[0]], glu_dtype=torch.float32)
    want1 = O.swiglu(_oracle_proj(up, xh, adu), _oracle_proj(gate, xh, None))
    assert O.rel_max(out1.cpu().numpy(), want1) < BAND


@pytest.mark.parametrize("IN,H,R,pad", [(960, 2560, 16, 16), (2048, 2048, 5, 8)])
@pytest.mark.parametrize("T", [17, 135, 300])
@pytest.mark.parametrize("xdt", [torch.float32, torch.bfloat16])
def test_glu_layer_with_both_adapters_in_one_launch(T, xdt, IN, H, R, pad):
    """A gate | up layer made by nq_fuse_glu (960 -> 2560 each with rank 16, 2048 -> 2048 with rank 5 stored as 8; SwiGLU in the kernel's epilogue) with an adapter on both
    projections, in the layer's single launch: against the oracle's projections, adapters and `swiglu`
    (fused.mojo:337-353 orders them that way); B = 0 on both leaves the bits of the layer's plain forward wherever that
    runs on the same kernel, no adapters at all always; shapes the kernel does not take, and an adapter on one projection only, are refused before any launch."""
    from noeira_amd.qlinear import FusedGLU

    rng = np.random.default_rng(3000 + T + IN)
    gate, up = _q4(rng, IN, H), _q4(rng, IN, H)
    glu = FusedGLU(gate, up)
    xf = rng.standard_normal((T, IN)).astype(np.float32)
    x = torch.from_numpy(xf).cuda().to(xdt)
    xh = x.float().cpu().numpy()
    adg, adu = make(rng, IN, H, R, pad=pad), make(rng, IN, H, R, pad=pad)
    for odt in (torch.float32, torch.bfloat16):
        out = glu.forward_lora(x, adg[0], adu[0], out_dtype=odt)
        assert out.shape == (T, H) and out.dtype == odt
        want = O.swiglu(_oracle_proj(up, xh, adu), _oracle_proj(gate, xh, adg))
        tol = BAND if odt == torch.float32 else 2.0 ** -8 + BAND
        assert O.rel_max(out.float().cpu().numpy(), want) < tol, odt
    base = glu.forward(x)
    zg, zu = make(rng, IN, H, R, pad=pad, zero_b=True)[0], make(rng, IN, H, R, pad=pad, zero_b=True)[0]
    zero = glu.forward_lora(x, zg, zu)
    if T >= 135:  # (where the layer's plain forward runs on the same kernel; at 17 rows it takes another one)
        assert torch.equal(zero.view(torch.int32), base.view(torch.int32))
    else:
        assert O.rel_max(zero.cpu().numpy(), base.cpu().numpy()) < BAND
    assert torch.equal(glu.forward_lora(x, None, None).view(torch.int32), base.view(torch.int32))
    # a sentinel under the output: every element is written
    out = torch.full((T, H), float("nan"), dtype=torch.float32, device="cuda")
    glu.forward_lora(x, adg[0], adu[0], out=out)
    assert not torch.isnan(out).any()
    with pytest.raises(L.NQError, match="both projections"):
        glu.forward_lora(x, adg[0], None)
    for bad_T in (1, 600):
        xb = torch.from_numpy(rng.standard_normal((bad_T, IN)).astype(np.float32)).cuda().to(xdt)
        keep = torch.full((bad_T, H), 7.0, dtype=torch.float32, device="cuda")
        with pytest.raises(L.NQError, match="ahead of SwiGLU"):
            glu.forward_lora(xb, adg[0], adu[0], out=keep)
        assert bool((keep == 7.0).all())   # refused before anything ran


def test_fused_adapters_outside_the_fast_kernel_and_errors():
    """Ranks and widths the 16-byte kernel does not take (R_PAD = 8, a part 70 wide) go part by part through the
    general kernel, the SwiGLU through its own launch: the same values.  A GLU-fused layer needs its glu_out."""
    from noeira_amd.qlinear import FusedGLU, FusedRows

    rng = np.random.default_rng(77)
    IN, T = 96, 9
    a_, b_ = _q4(rng, IN, 70), _q4(rng, IN, 128)
    fused = FusedRows([a_, b_])
    x = torch.from_numpy(rng.standard_normal((T, IN)).astype(np.float32)).cuda()
    xh = x.cpu().numpy()
    ads = [make(rng, IN, 70, 3, pad=8), make(rng, IN, 128, 16)]
    for lin, ad, y in zip((a_, b_), ads, fused.forward_lora(x, [ad[0] for ad in ads])):
        assert O.rel_max(y.cpu().numpy(), _oracle_proj(lin, xh, ad)) < BAND
    g, u = _q4(rng, IN, 64), _q4(rng, IN, 64)
    pair = FusedRows([g, u])
    adg, adu = make(rng, IN, 64, 3, pad=8), make(rng, IN, 64, 3, pad=8)
    out = pair.forward_lora(x, [adg[0], adu[0]], glu_dtype=torch.float32)
    want = O.swiglu(_oracle_proj(u, xh, adu), _oracle_proj(g, xh, adg))
    assert O.rel_max(out.cpu().numpy(), want) < BAND
    with pytest.raises(L.NQError, match="equal width"):
        fused.forward_lora(x, [None, None], glu_dtype=torch.float32)
    with pytest.raises(L.NQError, match="per part"):
        fused.forward_lora(x, [None])
    glu = FusedGLU(g, u)
    table = (L.LoraPart * 1)(L.LoraPart(None, None, 0, 0.0))
    import ctypes as C
    ys = (C.c_void_p * 1)(out.data_ptr())
    rc = L.lib().nq_forward_fused_lora(glu._h, x.data_ptr(), L.DT_F32, ys, 1, T, None, L.DT_F32, table, None, L.DT_F32, None)
    assert rc == L.NQ_ERR_INVALID


def test_proj_fwd_taps_the_hessian_then_runs_base_and_adapter():
    """`DecoderLayerWeights.proj_fwd` (layer_weights.mojo:455-508): with calibration on, the projection's input goes
    into its Hessian first; then the base linear; then the adapter's share."""
    from noeira_amd.gptq import HessianAccumulator
    from noeira_amd.lora import proj_fwd

    rng = np.random.default_rng(31)
    IN, OUT, T = 192, 96, 11
    lin = _q4(rng, IN, OUT)
    ad = make(rng, IN, OUT, 4)
    x = torch.from_numpy(rng.standard_normal((T, IN)).astype(np.float32)).cuda()
    xh = x.cpu().numpy()
    hs = HessianAccumulator(IN)
    y = proj_fwd(lin, x, adapter=ad[0], hessian=hs)
    assert O.rel_max(y.cpu().numpy(), _oracle_proj(lin, xh, ad)) < BAND
    assert hs.rows == T
    want_h = O.hessian_add(np.zeros((IN, IN), np.float64), xh)
    assert np.array_equal(hs.h.view(np.uint64), want_h.view(np.uint64))
    # no adapter, no tap: the bare linear's bits
    assert torch.equal(proj_fwd(lin, x), lin.forward(x))
    ad[0].merged = True
    assert torch.equal(proj_fwd(lin, x, adapter=ad[0]), lin.forward(x))
