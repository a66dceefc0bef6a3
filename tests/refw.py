"""Reference weights for the forward tests: deq(W) as fp64 on the device, computed from the host-side codes the
test itself drew, by the CPU oracle's dequantisers (oracle/nq_oracle.c) or, for int8 and e4m3, by the exact product
code x scale in fp64.  Nothing here asks the library under test what its weights are, so a forward test that
compares with `x @ refw.*(...).T` stands on the oracle alone; `nq_dequantize` is pinned separately, bit for bit,
against these same values."""
import numpy as np
import torch

from oracle import oracle as O


def q4_0(blocks, N, K):
    """(code - 8) * d per block of 32 (q4_0.mojo:242-266 restated in the oracle); exact in fp32."""
    return torch.from_numpy(O.dequantize_q4_0(np.ascontiguousarray(blocks, dtype=np.uint8).reshape(-1), N, K)).cuda().double()


def w4g(codes, scales_f16, zps, N, K, group):
    """(q - z) * s per group along K; exact in fp32."""
    s = np.ascontiguousarray(scales_f16)
    if s.dtype == np.float16:
        s = s.view(np.uint16)
    return torch.from_numpy(O.w4g_dequantize(codes, s, zps, N, K, group)).cuda().double()


def w8(w_i8, scales_f32):
    """int8 code x fp32 channel scale, exact in fp64."""
    w = torch.from_numpy(np.ascontiguousarray(w_i8, dtype=np.int8)).cuda().double()
    return w * torch.from_numpy(np.ascontiguousarray(scales_f32, dtype=np.float32)).cuda().double()[:, None]


def fp8(codes_u8, scale):
    """e4m3fn code decoded by the oracle's table x the fp32 tensor scale, exact in fp64."""
    table = torch.from_numpy(O.e4m3_decode_table().astype(np.float64)).cuda()
    c = torch.from_numpy(np.ascontiguousarray(codes_u8, dtype=np.uint8)).cuda().long()
    return table[c] * float(np.float32(scale))


def f32_bits(t):
    """fp32 tensor or array -> its bit patterns on the host, for bitwise comparisons."""
    a = t.detach().cpu().numpy() if isinstance(t, torch.Tensor) else np.asarray(t)
    return np.ascontiguousarray(a, dtype=np.float32).view(np.uint32)
