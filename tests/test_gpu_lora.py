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
