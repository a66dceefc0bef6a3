"""The capture rule of the reference's layer (noeira/nn/quant/qlinear.mojo:63-64, gate tests/nn/quant/
test_qlinear_gpu.mojo:55-130): after a first call at a row count a forward only enqueues kernels - no allocation,
no synchronisation, no host-side state that a replay would miss - so a caller may record it into a device graph.
Every kernel family's forward is recorded once and replayed several times over changing activations, with eager
work and synchronisations between the replays; each replay must return the bits of the eager call on the same
input.  The last test runs different layers on two streams at once (the boundary's threading rule: calls on
different handles on different streams are safe) against the same calls made one after the other."""
import numpy as np
import pytest
import torch

from noeira_amd import formats as F
from noeira_amd.lora import LoRAAdapter
from noeira_amd.qlinear import (FP8Linear, FusedGLU, FusedRows, QLinear, W4GroupLinear, W8Linear, mlp3_w8a8_forward,
                                quantize_rows_i8)

pytestmark = pytest.mark.gpu


def q4(rng, K, N, **kw):
    lin = QLinear(K, N, **kw)
    blocks = rng.integers(0, 256, (N, K // 32, 18), dtype=np.uint8)
    sc = rng.uniform(1e-3, 1e-2, (N, K // 32)).astype(np.float16).view(np.uint16)
    blocks[:, :, 0], blocks[:, :, 1] = sc & 0xFF, sc >> 8
    lin.set_blocks(blocks.reshape(-1))
    return lin


def w8(rng, K, N, **kw):
    lin = W8Linear(K, N, **kw)
    lin.set_weight(rng.integers(-127, 128, (N, K), dtype=np.int8), rng.uniform(1e-3, 1e-2, N).astype(np.float32))
    return lin


def w4g(rng, K, N, **kw):
    G = -(-K // 128)
    codes, zps = F.pack_w4g(rng.integers(0, 16, (N, K), dtype=np.uint8), rng.integers(0, 16, (N, G), dtype=np.uint8))
    lin = W4GroupLinear(K, N, 128, **kw)
    lin.set_weight(codes, rng.uniform(1e-3, 1e-2, (N, G)).astype(np.float16), zps)
    return lin


def fp8(rng, K, N):
    codes = rng.integers(0, 256, (N, K), dtype=np.uint8)
    codes[(codes & 0x7F) == 0x7F] = 0x38
    lin = FP8Linear(K, N)
    lin.set_weight(codes, 0.01)
    return lin


def replay_equals_eager(call, inputs, fresh):
    """`call(out)` runs the forward on the tensors of `inputs` into `out`; `fresh(i)` returns the i-th set of
    contents for them.  Recorded once, replayed over four sets of contents; every replay against the eager call."""
    for t, v in zip(inputs, fresh(0)):
        t.copy_(v)
    want = call(None)                      # the first call at this row count, outside any recording
    out = torch.empty_like(want)
    torch.cuda.synchronize()
    g = torch.cuda.CUDAGraph()
    with torch.cuda.graph(g):
        call(out)
    for i in (1, 2, 0, 3):
        for t, v in zip(inputs, fresh(i)):
            t.copy_(v)
        out.fill_(float("nan")) if out.dtype.is_floating_point else out.zero_()
        torch.cuda.synchronize()
        g.replay()
        torch.cuda.synchronize()
        want = call(None)
        torch.cuda.synchronize()
        assert torch.equal(out.view(torch.uint8), want.view(torch.uint8)), i


FLOAT_FAMILIES = [
    # (name, maker, K, N, M, x dtype, keyword arguments of the layer)
    ("gemv_m1 q4_0", q4, 960, 2560, 1, torch.float32, {}),
    ("gemv_m1 w8", w8, 512, 3200, 1, torch.bfloat16, {}),
    ("gemv_m1 w4g", w4g, 2560, 960, 1, torch.bfloat16, {}),
    ("gemv_tile4 q4_0", q4, 4096, 1040, 1, torch.float32, {}),
    ("gemv_tile4 rows w4g", w4g, 4096, 2064, 7, torch.bfloat16, {}),
    ("gemv_tile8 rows w8", w8, 4096, 1040, 5, torch.bfloat16, {}),
    ("gemv_row4 q4_0", q4, 4096, 1040, 1, torch.float32, {"tile_copy": False}),
    ("gemv_row8 w8", w8, 8192, 520, 1, torch.float32, {"tile_copy": False}),
    ("gemv_split8 w8", w8, 4096, 4100, 1, torch.bfloat16, {"tile_copy": False}),
    ("gemm_a16 q4_0 fp32", q4, 960, 960, 135, torch.float32, {}),
    ("gemm_a16 w8", w8, 3200, 512, 100, torch.bfloat16, {}),
    ("gemm_a16 w4g", w4g, 960, 960, 256, torch.bfloat16, {}),
    ("m tiles q4_0 bf16", q4, 960, 2560, 135, torch.bfloat16, {}),
    ("m tiles q4_0 fp32", q4, 960, 2560, 135, torch.float32, {}),
    ("m tiles w4g large", w4g, 2048, 11008, 33, torch.bfloat16, {}),
    ("gemm_a16_big q4_0", q4, 960, 2560, 1120, torch.bfloat16, {}),
]


@pytest.mark.parametrize("name,maker,K,N,M,xdt,kw", FLOAT_FAMILIES, ids=[f[0] for f in FLOAT_FAMILIES])
def test_recorded_forward_float_activations(name, maker, K, N, M, xdt, kw):
    rng = np.random.default_rng(K + N + M)
    lin = maker(rng, K, N, **kw)
    xs = [torch.from_numpy(rng.standard_normal((M, K)).astype(np.float32)).to(xdt).cuda() for _ in range(4)]
    bias = torch.from_numpy(rng.standard_normal(N).astype(np.float32)).cuda()
    x = torch.empty_like(xs[0])
    if maker is q4:
        call = lambda out: lin.forward(x, out=out)
    else:
        call = lambda out: lin.forward(x, bias=bias, epilogue="relu", out=out)
    replay_equals_eager(call, [x], lambda i: [xs[i]])


@pytest.mark.parametrize("M,K,N", [(1, 4096, 1040), (16, 512, 200), (256, 1024, 1040), (1024, 256, 520), (2048, 128, 8704), (1536, 256, 2304)])
def test_recorded_forward_int8_and_fp8_activations(M, K, N):
    """gemv8_row, tile8 and gemm8 under int8 and e4m3 activations, and the row quantiser that feeds the first.
    ((2048, 128, 8704): the GEMM as two launches, full rounds of 256 x 256 tiles and the leftover on 128 x 256 tiles;
    (1536, 256, 2304): all of it on 128 x 256 or 128 x 128 tiles.)"""
    rng = np.random.default_rng(M + K + N)
    lin, lin8 = w8(rng, K, N), fp8(rng, K, N)
    xs = [torch.from_numpy(rng.standard_normal((M, K)).astype(np.float32)).cuda() for _ in range(4)]
    x = torch.empty_like(xs[0])
    xq = torch.empty((M, K), dtype=torch.int8, device="cuda")
    sx = torch.empty((M,), dtype=torch.float32, device="cuda")

    def call_i8(out):
        quantize_rows_i8(x, q=xq, scales=sx)
        return lin.forward_a8(xq, sx, out=out)
    replay_equals_eager(call_i8, [x], lambda i: [xs[i]])

    cs = [torch.from_numpy(rng.integers(0, 0x78, (M, K), dtype=np.uint8) | (rng.integers(0, 2, (M, K), dtype=np.uint8) << 7)).cuda()
          for _ in range(4)]
    xc = torch.empty_like(cs[0])
    xscale = torch.tensor([0.02], dtype=torch.float32, device="cuda")
    replay_equals_eager(lambda out: lin8.forward(xc, xscale, out=out), [xc], lambda i: [cs[i]])


@pytest.mark.parametrize("M", [1, 135])
@pytest.mark.parametrize("xdt", [torch.float32, torch.bfloat16])
def test_recorded_fused_calls(M, xdt):
    """q | k | v through the part table, gate | up with the SwiGLU in the launch, and the adapter folded into the
    base call: the calls of one decoder layer (noeira/deep_agents/smolvla/fused.mojo:255-384)."""
    rng = np.random.default_rng(M)
    IN = 960
    xs = [torch.from_numpy(rng.standard_normal((M, IN)).astype(np.float32)).to(xdt).cuda() for _ in range(4)]
    x = torch.empty_like(xs[0])
    qkv = FusedRows([q4(rng, IN, 960), q4(rng, IN, 320), q4(rng, IN, 320)])

    # (the parts' outputs are separate [M, OUT_i] tensors: compared as one flat buffer)
    flat = lambda outs: torch.cat([o.reshape(-1) for o in outs])
    x.copy_(xs[0])
    outs = [torch.empty((M, n), device="cuda") for n in (960, 320, 320)]
    qkv.forward(x)
    torch.cuda.synchronize()
    g = torch.cuda.CUDAGraph()
    with torch.cuda.graph(g):
        qkv.forward(x, outs=outs)
    for i in (1, 2, 0):
        x.copy_(xs[i])
        for o in outs:
            o.fill_(float("nan"))
        torch.cuda.synchronize()
        g.replay()
        torch.cuda.synchronize()
        assert torch.equal(flat(outs).view(torch.int32), flat(qkv.forward(x)).view(torch.int32)), i

    glu = FusedGLU(q4(rng, IN, 2560), q4(rng, IN, 2560))
    replay_equals_eager(lambda out: glu.forward(x, out=out), [x], lambda i: [xs[i]])

    base = q4(rng, IN, 2560)
    ad = LoRAAdapter(IN, 2560, 8)
    ad.set_params(rng.standard_normal((IN, 8)).astype(np.float32) * 0.05, rng.standard_normal((8, 2560)).astype(np.float32) * 0.05)

    def call_lora(out):
        y = ad.forward_with(base, x)
        if out is None:
            return y
        out.copy_(y)       # (forward_with returns its own tensor: inside the recording the copy is part of the graph)
        return out
    replay_equals_eager(call_lora, [x], lambda i: [xs[i]])

    def call_lora_two(out):
        y = base.forward(x, out=out)
        return ad.forward_add(x, y)
    replay_equals_eager(call_lora_two, [x], lambda i: [xs[i]])


def test_recorded_actor_mlp():
    """The three-layer W8A8 actor as one launch (64 -> 256 -> 256 -> 8), M = 4096 and a ragged 77."""
    rng = np.random.default_rng(4)
    l1, l2, l3 = w8(rng, 64, 256), w8(rng, 256, 256), w8(rng, 256, 8)
    bs = [torch.from_numpy(rng.standard_normal(n).astype(np.float32)).cuda() for n in (256, 256, 8)]
    for M in (4096, 77):
        xs = [torch.from_numpy(rng.standard_normal((M, 64)).astype(np.float32)).cuda() for _ in range(4)]
        x = torch.empty_like(xs[0])
        replay_equals_eager(lambda out: mlp3_w8a8_forward(l1, l2, l3, x, *bs, out=out), [x], lambda i: [xs[i]])


def test_two_streams_different_layers():
    """Different handles on different streams at the same time - two small layers, two large 4-bit layers on the
    persistent tile kernel, a 16-row call beside a single-row one - return what the same calls return one by one."""
    rng = np.random.default_rng(8)
    pairs = [((q4, 960, 2560, 1, torch.float32), (w8, 512, 3200, 1, torch.bfloat16)),
             ((q4, 4096, 4096, 1, torch.float32), (w4g, 4096, 4096, 1, torch.bfloat16)),
             ((w4g, 4096, 2064, 16, torch.bfloat16), (w8, 4096, 1040, 1, torch.bfloat16)),
             ((q4, 960, 2560, 135, torch.bfloat16), (q4, 960, 960, 135, torch.float32))]
    s1, s2 = torch.cuda.Stream(), torch.cuda.Stream()
    for a, b in pairs:
        la, lb = a[0](rng, a[1], a[2]), b[0](rng, b[1], b[2])
        xa = torch.from_numpy(rng.standard_normal((a[3], a[1])).astype(np.float32)).to(a[4]).cuda()
        xb = torch.from_numpy(rng.standard_normal((b[3], b[1])).astype(np.float32)).to(b[4]).cuda()
        wa, wb = la.forward(xa), lb.forward(xb)
        oa, ob = torch.empty_like(wa), torch.empty_like(wb)
        torch.cuda.synchronize()
        for _ in range(20):
            oa.fill_(float("nan"))
            ob.fill_(float("nan"))
            torch.cuda.synchronize()
            with torch.cuda.stream(s1):
                for _ in range(4):
                    la.forward(xa, out=oa)
            with torch.cuda.stream(s2):
                for _ in range(4):
                    lb.forward(xb, out=ob)
            torch.cuda.synchronize()
            assert torch.equal(oa.view(torch.int32), wa.view(torch.int32))
            assert torch.equal(ob.view(torch.int32), wb.view(torch.int32))
