"""Host-side mirror of the reference's LoRA adapter for inference, over the C ABI.

``LoRAAdapter`` keeps what `LoRAAdapter[IN, OUT, R, PAD_R, RSLORA]`
(noeira/nn/peft/lora.mojo:152-349) needs to serve a frozen adapter beside a
quantized linear: the rank-padded parameters on the device, ``alpha``,
``scale()``, ``merged`` and ``forward_add``.  Training (``vjp_add``, the
optimizer walks) and merging into an fp32 base weight are not part of the
inference path and are not here.
"""
from __future__ import annotations

import ctypes as C
import math

import numpy as np
import torch

from . import _lib as L
from .qlinear import _TORCH_DT, _dev_ptr, _stream_ptr


class LoRAAdapter:
    """``s * (x A) B`` beside a linear [IN -> OUT]; A [IN, R_PAD], B [R_PAD, OUT] fp32, the logical R
    columns / rows first and zeros after (lora.mojo:28-41)."""

    def __init__(self, IN: int, OUT: int, R: int, PAD_R: int = 16, RSLORA: bool = False, alpha: float | None = None):
        if R < 1 or PAD_R < 1:  # the comptime asserts of lora.mojo:198-199
            raise L.NQError(L.NQ_ERR_INVALID, "LoRA rank must be at least 1" if R < 1 else "PAD_R must be at least 1")
        self.IN, self.OUT, self.R, self.RSLORA = IN, OUT, R, RSLORA
        self.R_PAD = (R + PAD_R - 1) // PAD_R * PAD_R
        self.alpha = float(R if alpha is None else alpha)
        self.merged = False
        self.lora_A = torch.zeros((IN, self.R_PAD), dtype=torch.float32, device="cuda")
        self.lora_B = torch.zeros((self.R_PAD, OUT), dtype=torch.float32, device="cuda")

    def scale(self) -> float:
        return self.alpha / math.sqrt(self.R) if self.RSLORA else self.alpha / self.R

    def set_params(self, a, b):
        """Load the logical blocks: a [IN, R], b [R, OUT] (the pad stays zero)."""
        a = np.ascontiguousarray(a, dtype=np.float32)
        b = np.ascontiguousarray(b, dtype=np.float32)
        if a.shape != (self.IN, self.R) or b.shape != (self.R, self.OUT):
            raise L.NQError(L.NQ_ERR_SIZE, f"LoRAAdapter.set_params: expected A [{self.IN}, {self.R}] and "
                                           f"B [{self.R}, {self.OUT}]")
        self.lora_A.zero_()
        self.lora_B.zero_()
        self.lora_A[:, :self.R] = torch.from_numpy(a).cuda()
        self.lora_B[:self.R] = torch.from_numpy(b).cuda()

    def forward_add(self, x: torch.Tensor, y: torch.Tensor):
        """``y[T, OUT] += s * (x[T, IN] A) B``, called with the base linear's own input and output right
        after its forward.  Nothing once merged (lora.mojo:292-303)."""
        if self.merged:
            return y
        if x.dtype not in _TORCH_DT or not x.is_cuda or not x.is_contiguous() or x.numel() % self.IN:
            raise L.NQError(L.NQ_ERR_INVALID, "LoRAAdapter.forward_add: x must be a contiguous fp32/bf16 device "
                                              "tensor of [T, IN] values")
        T = x.numel() // self.IN
        if y.dtype != torch.float32 or not y.is_cuda or not y.is_contiguous() or y.numel() != T * self.OUT:
            raise L.NQError(L.NQ_ERR_INVALID, "LoRAAdapter.forward_add: y must be the base layer's fp32 [T, OUT] output")
        L.check(L.lib().nq_lora_forward_add(_dev_ptr(self.lora_A), _dev_ptr(self.lora_B), self.IN, self.OUT,
                                            self.R_PAD, C.c_float(self.scale()), _dev_ptr(x), _TORCH_DT[x.dtype],
                                            _dev_ptr(y), T, _stream_ptr()))
        return y

    def forward_with(self, base, x: torch.Tensor, bias: torch.Tensor | None = None,
                     out_dtype: torch.dtype = torch.float32, out: torch.Tensor | None = None) -> torch.Tensor:
        """``base.forward(x)`` and this adapter's share in one call (`nq_forward_lora`): one launch where the base
        call runs on the kernel that keeps its rows' activations resident, the two of `forward` + `forward_add`
        elsewhere.  B = 0 returns the bits of ``base.forward(x)``."""
        if self.merged:
            return base.forward(x, bias=bias, out_dtype=out_dtype)
        if x.dtype not in _TORCH_DT or not x.is_cuda or not x.is_contiguous() or x.dim() != 2 or x.shape[1] != self.IN:
            raise L.NQError(L.NQ_ERR_INVALID, "LoRAAdapter.forward_with: x must be a contiguous fp32/bf16 device [T, IN] tensor")
        if base.IN != self.IN or base.OUT != self.OUT:
            raise L.NQError(L.NQ_ERR_INVALID, "LoRAAdapter.forward_with: the adapter and the base layer differ in shape")
        T = x.shape[0]
        y = out if (out is not None and out.dtype == out_dtype and out.numel() >= T * self.OUT and out.is_cuda) else \
            torch.empty((T, self.OUT), dtype=out_dtype, device=x.device)
        null = C.c_void_p(0)
        L.check(L.lib().nq_forward_lora(base._h, _dev_ptr(x), _TORCH_DT[x.dtype], _dev_ptr(y), _TORCH_DT[out_dtype], T,
                                        _dev_ptr(bias) if bias is not None else null,
                                        _TORCH_DT[bias.dtype] if bias is not None else L.DT_F32,
                                        _dev_ptr(self.lora_A), _dev_ptr(self.lora_B), self.R_PAD,
                                        C.c_float(self.scale()), _stream_ptr()))
        return y


def proj_fwd(base, x: torch.Tensor, adapter: "LoRAAdapter | None" = None, hessian=None, bias: torch.Tensor | None = None,
             out: torch.Tensor | None = None) -> torch.Tensor:
    """One projection of the decoder layer as the reference's caller runs it, `DecoderLayerWeights.proj_fwd`
    (noeira/deep_agents/smolvla/layer_weights.mojo:455-508): when calibrating, the projection's input is added to
    its Hessian first (`HessianAccumulator.add`, hessian.mojo:41-77: `hessian` is a `noeira_amd.gptq.HessianAccumulator` or
    None); then the base linear; then the adapter's share, if the projection carries an unmerged one.  x: fp32 or
    bf16 [T, IN] on the device; returns fp32 [T, OUT]."""
    if hessian is not None:
        hessian.add(x)
    if adapter is None or adapter.merged:
        return base.forward(x, bias=bias, out=out) if bias is not None or out is not None else base.forward(x)
    return adapter.forward_with(base, x, bias=bias, out=out)
