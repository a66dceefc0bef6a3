"""Host-side mirror of the reference's GPTQ quantizer over the C ABI.

``HessianAccumulator`` (noeira/nn/quant/hessian.mojo:24-77), ``gptq_q4_0`` and
``q4_0_objective`` (noeira/nn/quant/gptq.mojo:62-189) and ``hinv_upper_f64``
(noeira/nn/quant/dense.mojo:355-363) with the reference's names, argument
meaning and error sentences.  Every computation runs on the device inside
libnoeira_qlinear.so; there is no CPU path.
"""
from __future__ import annotations

import ctypes as C
from dataclasses import dataclass
from typing import Optional

import numpy as np
import torch

from . import _lib as L
from .qlinear import Q4_GROUP, QLinear, _dev_ptr, _stream_ptr, _TORCH_DT


@dataclass
class GPTQStats:
    """What one ``gptq_q4_0`` call saw: the dead inputs and the damping (gptq.mojo:52-60)."""

    dead: int = 0
    damp: float = 0.0


class HessianAccumulator:
    """H = sum x x^T over every row a linear reads during calibration, in fp64, on the device."""

    def __init__(self, n: int):
        self.n = int(n)
        self._h = C.c_void_p()
        L.check(L.lib().nq_hessian_create(C.byref(self._h), self.n))

    def __del__(self):
        h = getattr(self, "_h", None)
        if h:
            try:
                L.lib().nq_hessian_destroy(h)
            except Exception:
                pass
            self._h = None

    @property
    def rows(self) -> int:
        return int(L.lib().nq_hessian_rows(self._h))

    def add(self, x: torch.Tensor, rows: Optional[int] = None):
        """H += X^T X for the first `rows` rows of the device slab `x` ([rows, n] row-major)."""
        if x.dtype not in _TORCH_DT or not x.is_cuda or not x.is_contiguous():
            raise L.NQError(L.NQ_ERR_INVALID, "HessianAccumulator.add: x must be a contiguous fp32/bf16 device tensor")
        if rows is None:
            rows = x.numel() // self.n
        if x.numel() < rows * self.n:  # hessian.mojo:54-60
            raise L.NQError(L.NQ_ERR_SIZE, f"HessianAccumulator.add: the slab holds {x.numel()} values, "
                                           f"[{rows}, {self.n}] need {rows * self.n}")
        L.check(L.lib().nq_hessian_add(self._h, _dev_ptr(x), _TORCH_DT[x.dtype], rows, _stream_ptr()))

    @property
    def h(self) -> np.ndarray:
        out = np.empty((self.n, self.n), np.float64)
        L.check(L.lib().nq_hessian_get(self._h, out.ctypes.data_as(C.c_void_p), out.size))
        return out

    def set(self, h, rows: int = 0):
        """Load a Hessian computed elsewhere ([n, n], widened to fp64)."""
        a = np.ascontiguousarray(h, dtype=np.float64)
        L.check(L.lib().nq_hessian_set(self._h, a.ctypes.data_as(C.c_void_p), a.size, rows))
        return self


def hinv_upper_f64(h) -> np.ndarray:
    """U, upper triangular with U^T U = h^-1 (dense.mojo:355-363)."""
    a = np.ascontiguousarray(h, dtype=np.float64)
    n = a.shape[0]
    u = np.empty((n, n), np.float64)
    L.check(L.lib().nq_hinv_upper_f64(a.ctypes.data_as(C.c_void_p), n, u.ctypes.data_as(C.c_void_p), _stream_ptr()))
    return u


def hinv_upper_f64_dev(h: torch.Tensor, u: Optional[torch.Tensor] = None, pivot: Optional[torch.Tensor] = None):
    """`hinv_upper_f64` without any allocation inside the library (nq_hinv_upper_f64_dev): `h`, `u` are [n, n] fp64
    device tensors, `pivot` a device int32.  Only enqueues; returns (u, pivot).  n <= 1024; calls that overlap
    on one GPU race (they share the library's fixed scratch)."""
    if h.dtype != torch.float64 or not h.is_cuda or not h.is_contiguous() or h.dim() != 2 or h.shape[0] != h.shape[1]:
        raise L.NQError(L.NQ_ERR_INVALID, "hinv_upper_f64_dev: h must be a contiguous [n, n] fp64 device tensor")
    n = h.shape[0]
    if u is None:
        u = torch.empty_like(h)
    if pivot is None:
        pivot = torch.empty((1,), dtype=torch.int32, device=h.device)
    L.check(L.lib().nq_hinv_upper_f64_dev(_dev_ptr(h), n, _dev_ptr(u), _dev_ptr(pivot), _stream_ptr()))
    return u, pivot


def set_weight_gptq(layer: QLinear, w, hess: HessianAccumulator, damp_frac: float = 0.01) -> GPTQStats:
    """Quantize the fp32 [OUT, IN] weight with GPTQ against `hess` and load the layer with it."""
    w = np.ascontiguousarray(w, dtype=np.float32)
    dead, damp = C.c_int64(0), C.c_double(0)
    L.check(L.lib().nq_set_weight_gptq(layer._h, w.ctypes.data_as(C.c_void_p), w.size, hess._h, damp_frac,
                                       C.byref(dead), C.byref(damp), _stream_ptr()))
    layer._loaded = True
    return GPTQStats(dead.value, damp.value)


def gptq_q4_0(w, n: int, k: int, h, damp_frac: float = 0.01):
    """(codes [n, k] uint8, scales [n, k/32] fp32 with bf16 values, stats) for a row-major [n, k]
    fp32 weight and the [k, k] Hessian of its inputs (gptq.mojo:62-150)."""
    if k % Q4_GROUP != 0:
        raise L.NQError(L.NQ_ERR_INVALID, f"gptq_q4_0: k = {k} is not a multiple of 32")
    w = np.ascontiguousarray(w, dtype=np.float32)
    hh = np.ascontiguousarray(h, dtype=np.float64)
    if w.size < n * k or hh.size < k * k:
        raise L.NQError(L.NQ_ERR_SIZE, "gptq_q4_0: w or h is smaller than [n, k] / [k, k]")
    layer = QLinear(k, n)
    acc = HessianAccumulator(k).set(hh.reshape(-1)[:k * k].reshape(k, k))
    stats = set_weight_gptq(layer, w.reshape(-1)[:n * k], acc, damp_frac)
    blocks = layer.blocks().reshape(n, k // Q4_GROUP, 18)
    nib = blocks[:, :, 2:]
    q = np.concatenate([nib & 0xF, nib >> 4], axis=2).reshape(n, k)
    d = np.ascontiguousarray(blocks[:, :, :2]).view(np.float16).astype(np.float32).reshape(n, k // Q4_GROUP)
    return q, d, stats


def q4_0_objective(layer: QLinear, w, hess: HessianAccumulator) -> float:
    """tr((W - What) H (W - What)^T) in fp64 for the layer's weights What (gptq.mojo:152-189)."""
    w = np.ascontiguousarray(w, dtype=np.float32)
    out = C.c_double(0)
    L.check(L.lib().nq_q4_0_objective(layer._h, w.ctypes.data_as(C.c_void_p), w.size, hess._h, C.byref(out),
                                      _stream_ptr()))
    return out.value
