"""Host-side packing of the quantized weight formats (numpy; load time only).

Q4_0 is the reference's format (noeira/nn/quant/q4_0.mojo:1-8); its packing on
the host lives in the library's device RTN kernel and in ``QLinear.set_blocks``.
The helpers here build the byte layouts of the extension formats that
``W8Linear`` / ``W4GroupLinear`` / ``FP8Linear`` load:

  W4_GROUP  codes  [N, K/2]  byte i of a row = element 2i (low nibble) | element 2i+1 (high)
            scales [N, G] fp16, G = ceil(K / group) (a ragged last group is allowed)
            zps    [N, ceil(G/2)]  byte i = group 2i (low nibble) | group 2i+1 (high)
            value  = (q - z) * fp32(s)
  FP8_E4M3  OCP e4m3fn codes (max finite 448, no infinities), one fp32 scale
"""
from __future__ import annotations

import numpy as np


def pack_u4_pairs(q: np.ndarray) -> np.ndarray:
    """[..., 2n] values in 0..15 -> [..., n] bytes, even index in the low nibble."""
    q = np.ascontiguousarray(q, dtype=np.uint8)
    if q.shape[-1] % 2:
        q = np.concatenate([q, np.zeros(q.shape[:-1] + (1,), np.uint8)], axis=-1)
    return ((q[..., 0::2] & 0xF) | ((q[..., 1::2] & 0xF) << 4)).astype(np.uint8)


def pack_w4g(q: np.ndarray, zps: np.ndarray):
    """codes [N, K] (0..15) and zero-points [N, G] (0..15) -> (codes [N, K/2], zps [N, ceil(G/2)])."""
    return pack_u4_pairs(q), pack_u4_pairs(zps)


def quantize_w4g_asym(w: np.ndarray, group: int = 128):
    """Min/max asymmetric uint4 quantisation of an fp32 [N, K] weight, group-wise
    along K (ragged last group allowed): returns (q [N, K], scales fp16 [N, G],
    zps [N, G])."""
    w = np.asarray(w, np.float32)
    N, K = w.shape
    G = -(-K // group)
    q = np.empty((N, K), np.uint8)
    s = np.empty((N, G), np.float16)
    z = np.empty((N, G), np.uint8)
    for g in range(G):
        blk = w[:, g * group:(g + 1) * group]
        lo = np.minimum(blk.min(axis=1), 0.0)
        hi = np.maximum(blk.max(axis=1), 0.0)
        sc = ((hi - lo) / np.float32(15)).astype(np.float16)
        sc[sc == 0] = np.float16(1.0)
        s32 = sc.astype(np.float32)
        zp = np.clip(np.round(-lo / s32), 0, 15).astype(np.uint8)
        q[:, g * group:(g + 1) * group] = np.clip(np.round(blk / s32[:, None]) + zp[:, None], 0, 15).astype(np.uint8)
        s[:, g], z[:, g] = sc, zp
    return q, s, z


def quantize_w8_channel(w: np.ndarray):
    """Symmetric per-output-channel int8: s = absmax / 127, q = round(w / s)."""
    w = np.asarray(w, np.float32)
    s = (np.abs(w).max(axis=1) / np.float32(127)).astype(np.float32)
    s[s == 0] = 1.0
    q = np.clip(np.round(w / s[:, None]), -127, 127).astype(np.int8)
    return q, s


def encode_e4m3(x: np.ndarray) -> np.ndarray:
    """fp32 -> OCP e4m3fn codes, clipped to +-448 first, round to nearest even."""
    import torch

    t = torch.from_numpy(np.ascontiguousarray(x, dtype=np.float32)).clamp_(-448.0, 448.0)
    return t.to(torch.float8_e4m3fn).view(torch.uint8).numpy()
