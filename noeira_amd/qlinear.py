"""Host-side mirror of the reference's quantized linear operator over the C ABI.

``QLinear`` keeps the public surface of ``QLinear[IN, OUT]``
(noeira/nn/quant/qlinear.mojo:208-524): ``make``, ``set_weight``,
``set_blocks``, ``blocks``, ``dequantized``, ``share_scratch``,
``keep_only_repacked``, ``forward``, ``vjp``, ``release_buffers`` with the
same argument meaning and the same error sentences, so the gates read like the
reference's (tests/nn/quant/test_qlinear_gpu.mojo).  ``W8Linear``,
``W4GroupLinear`` and ``FP8Linear`` are the int8 / group-wise uint4 / fp8
layers BASELINE names, in the shape of ``Linear`` / ``LinearAct`` (a bias and an
optional ReLU, noeira/nn/primitives/linear_act.mojo:81-115) but holding the
weight as [OUT, IN] like ``QLinear`` does.

torch is used only for device memory and streams; every computation is a call
into libnoeira_qlinear.so.  There is no CPU path: ``target="cpu"`` raises.
"""
from __future__ import annotations

import ctypes as C
from typing import Optional

import numpy as np
import torch

from . import _lib as L

Q4_GROUP = 32
Q4_BLOCK = 18

_TORCH_DT = {torch.float32: L.DT_F32, torch.bfloat16: L.DT_BF16}


def _stream_ptr() -> C.c_void_p:
    return C.c_void_p(torch.cuda.current_stream().cuda_stream)


def _need_gpu(target: str):
    if target != "gpu":
        raise L.NQError(L.NQ_ERR_UNSUPPORTED,
                        "noeira_amd has no CPU path: target must be \"gpu\" (got \"" + str(target) + "\")")
    if not torch.cuda.is_available():
        raise L.NQError(L.NQ_ERR_HIP, "noeira_amd: no HIP device is visible")


def _dev_ptr(t: Optional[torch.Tensor]) -> C.c_void_p:
    return C.c_void_p(t.data_ptr()) if t is not None else C.c_void_p(0)


def _check_x(x: torch.Tensor, IN: int, what: str):
    if not x.is_cuda or not x.is_contiguous():
        raise L.NQError(L.NQ_ERR_INVALID, what + ": x must be a contiguous device tensor")
    if x.numel() % IN != 0:
        raise L.NQError(L.NQ_ERR_INVALID, f"{what}: x has {x.numel()} values, not a multiple of IN = {IN}")
    return x.numel() // IN


class _Layer:
    """Owns one nq_handle."""

    FORMAT = -1

    def __init__(self, IN: int, OUT: int, group: int = 0, tile_copy: bool = True, prefer_tile: bool = False):
        """tile_copy=False (NQ_FLAG_NO_TILE_COPY): a large layer does not keep the second,
        matrix-core-ordered copy of its codes that its single-row calls stream faster."""
        self.IN, self.OUT, self.group = int(IN), int(OUT), int(group)
        h = C.c_void_p()
        flags = (0 if tile_copy else L.FLAG_NO_TILE_COPY) | (L.FLAG_PREFER_TILE if prefer_tile else 0)
        L.check(L.lib().nq_create(C.byref(h), self.FORMAT, self.IN, self.OUT, self.group, flags))
        self._h = h
        self._loaded = False
        self.bias: Optional[torch.Tensor] = None  # `Linear`'s fp32 [OUT] bias, set by from_linear

    def __del__(self):
        h = getattr(self, "_h", None)
        if h is not None and h.value:
            try:
                L.lib().nq_destroy(h)
            except Exception:
                pass
            self._h = None

    @staticmethod
    def _linear_params(w_in_out, bias, IN: int, OUT: int, what: str):
        """`Linear[IN, OUT]` keeps W as [IN, OUT] row-major fp32 and an fp32 [OUT] bias
        (noeira/nn/primitives/linear.mojo:970-971): the opposite orientation from the [OUT, IN] this library (and
        `QLinear`) holds, so a drop-in transposes at load, as the reference's own gates do
        (tests/nn/quant/qlinear_common.mojo:86-91).  Returns (W^T [OUT, IN] contiguous fp32, device bias or None)."""
        w = np.asarray(w_in_out, dtype=np.float32)
        if w.shape != (IN, OUT):
            raise L.NQError(L.NQ_ERR_SIZE, f"{what}: the weight is {list(w.shape)}, expected Linear's [IN, OUT] = [{IN}, {OUT}]")
        b = None
        if bias is not None:
            bh = np.ascontiguousarray(bias, dtype=np.float32)
            if bh.shape != (OUT,):
                raise L.NQError(L.NQ_ERR_SIZE, f"{what}: the bias has {bh.size} values, expected OUT = {OUT}")
            b = torch.from_numpy(bh).cuda()
        return np.ascontiguousarray(w.T), b

    # shared by every format ------------------------------------------------
    def _forward(self, x: torch.Tensor, x_dtype: int, x_scale: Optional[torch.Tensor], out: Optional[torch.Tensor],
                 out_dtype: torch.dtype, bias: Optional[torch.Tensor], epilogue: str, what: str) -> torch.Tensor:
        M = _check_x(x, self.IN, what)
        if bias is None:
            bias = self.bias
        if out is None or out.numel() < M * self.OUT or out.dtype != out_dtype:
            out = torch.empty((M, self.OUT), dtype=out_dtype, device=x.device)
        y_dt = {torch.float32: L.DT_F32, torch.bfloat16: L.DT_BF16, torch.int32: L.DT_I32}[out_dtype]
        b_dt = L.DT_F32
        if bias is not None:
            if bias.dtype not in _TORCH_DT or bias.numel() != self.OUT or not bias.is_cuda:
                raise L.NQError(L.NQ_ERR_INVALID, what + ": bias must be a device fp32/bf16 tensor of OUT values")
            b_dt = _TORCH_DT[bias.dtype]
        epi = {"none": L.EPI_NONE, "relu": L.EPI_RELU}[epilogue]
        L.check(L.lib().nq_forward(self._h, _dev_ptr(x), x_dtype, _dev_ptr(x_scale), _dev_ptr(out), y_dt, M,
                                   _dev_ptr(bias), b_dt, epi, _stream_ptr()))
        return out

    def device_bytes(self) -> int:
        """Device memory the layer's weights occupy: codes, scales, zero points and every re-ordered copy a kernel
        reads (nq_device_bytes); 0 before a weight is set."""
        return int(L.lib().nq_device_bytes(self._h))

    def dequantized_dev(self, out: Optional[torch.Tensor] = None) -> torch.Tensor:
        """deq(W) [OUT, IN] fp32 on the device (`dequant_q4_0_kernel`, q4_0.mojo:242-266).  Without `out` it is
        written into the buffer handed to `share_scratch`, if any (its first OUT*IN values, returned as a
        [OUT, IN] view), else into a new tensor."""
        if out is None:
            shared = getattr(self, "deq", None)
            if shared is not None:
                # (the library writes the workspace it was handed by nq_set_workspace)
                L.check(L.lib().nq_dequantize(self._h, None, 0, _stream_ptr()))
                return shared.view(-1)[: self.OUT * self.IN].view(self.OUT, self.IN)
            else:
                out = torch.empty((self.OUT, self.IN), dtype=torch.float32, device="cuda")
        L.check(L.lib().nq_dequantize(self._h, _dev_ptr(out), out.numel(), _stream_ptr()))
        return out


class QLinear(_Layer):
    """A frozen Q4_0 linear: y[T, OUT] = x[T, IN] @ deq(W)^T, W [OUT, IN]
    (qlinear.mojo:1-11).  fp32 activations at its boundary, no bias, no Param."""

    FORMAT = L.FMT_Q4_0
    ARITY = 1

    def __init__(self, IN: int, OUT: int, tile_copy: bool = True, prefer_tile: bool = False):
        if IN % Q4_GROUP != 0:  # the comptime assert of qlinear.mojo:243-245
            raise L.NQError(L.NQ_ERR_INVALID, "QLinear: IN must be a multiple of 32 (one Q4_0 group)")
        super().__init__(IN, OUT, Q4_GROUP, tile_copy, prefer_tile)
        self.W_SIZE = IN * OUT
        self.ROW_BYTES = (IN // Q4_GROUP) * Q4_BLOCK
        self.BYTES = OUT * self.ROW_BYTES
        self.deq: Optional[torch.Tensor] = None  # shared dequantize scratch (share_scratch)

    @staticmethod
    def display_label() -> str:
        return "QLinear"

    @classmethod
    def make(cls, IN: int, OUT: int, target: str = "gpu", ctx=None) -> "QLinear":
        """An empty layer: weights come from set_weight or set_blocks, never
        from an initializer (qlinear.mojo:253-260)."""
        _need_gpu(target)
        return cls(IN, OUT)

    @classmethod
    def from_linear(cls, w_in_out, bias=None, tile_copy: bool = True) -> "QLinear":
        """A Q4_0 layer from `Linear[IN, OUT]`'s parameters: W [IN, OUT] is transposed to [OUT, IN] and quantized
        by RTN (set_weight); the fp32 bias, if any, is kept on the device and added by forward."""
        IN, OUT = np.asarray(w_in_out).shape
        lin = cls(IN, OUT, tile_copy=tile_copy)
        wt, lin.bias = cls._linear_params(w_in_out, bias, IN, OUT, "QLinear.from_linear")
        lin.set_weight(wt)
        return lin

    # ── weights ────────────────────────────────────────────────────────────
    def set_weight(self, w, target: str = "gpu", ctx=None):
        """Quantize an fp32 [OUT, IN] weight by RTN on the Q4_0 grid and load it
        (qlinear.mojo:264-269)."""
        _need_gpu(target)
        w = np.ascontiguousarray(w, dtype=np.float32)
        L.check(L.lib().nq_set_weight_f32(self._h, w.ctypes.data_as(C.c_void_p), w.size, _stream_ptr()))
        self._loaded = True

    def set_blocks(self, blocks, target: str = "gpu", ctx=None):
        """Load Q4_0 blocks [OUT, IN/32*18] (qlinear.mojo:271-320)."""
        _need_gpu(target)
        b = np.ascontiguousarray(blocks, dtype=np.uint8)
        L.check(L.lib().nq_set_blocks(self._h, b.ctypes.data_as(C.c_void_p), b.size, _stream_ptr()))
        self._loaded = True

    def blocks(self) -> np.ndarray:
        """A copy of the Q4_0 blocks (for a file) (qlinear.mojo:322-324)."""
        out = np.empty(self.BYTES, np.uint8)
        L.check(L.lib().nq_get_blocks(self._h, out.ctypes.data_as(C.c_void_p), out.size))
        return out

    def dequantized(self) -> np.ndarray:
        """deq(W) [OUT, IN] fp32 on the host (for gates) (qlinear.mojo:326-328)."""
        self.blocks()  # the `_need_blocks` rule: raises once the blocks were dropped
        return self.dequantized_dev().cpu().numpy()

    def share_scratch(self, buf: torch.Tensor, n: int):
        """Use `buf` (n fp32 values on the device, at least OUT*IN) as the dequantize scratch
        (qlinear.mojo:330-340).  This build's forward never materialises deq(W), so the forward does not
        touch it; it is where `dequantized_dev()` and `dequantized()` write deq(W) from now on."""
        if n < self.W_SIZE or buf.numel() < n:
            raise L.NQError(L.NQ_ERR_SIZE,
                            f"QLinear.share_scratch: {min(n, buf.numel())} values for a [{self.OUT}, {self.IN}] weight")
        if buf.dtype != torch.float32 or not buf.is_cuda or not buf.is_contiguous():
            raise L.NQError(L.NQ_ERR_INVALID, "QLinear.share_scratch: the scratch must be a contiguous fp32 device tensor")
        L.check(L.lib().nq_set_workspace(self._h, _dev_ptr(buf), 4 * n))
        self.deq = buf

    def keep_only_repacked(self):
        """Drop the logical blocks, keep the device layout the forward reads
        (qlinear.mojo:342-356).  blocks(), dequantized() and vjp raise after."""
        L.check(L.lib().nq_keep_only_repacked(self._h))

    # ── Module ─────────────────────────────────────────────────────────────
    def forward(self, x: torch.Tensor, out: Optional[torch.Tensor] = None, target: str = "gpu",
                ctx=None, bias: Optional[torch.Tensor] = None, epilogue: str = "none",
                out_dtype: torch.dtype = torch.float32) -> torch.Tensor:
        """y[B, OUT] = x[B, IN] @ deq(W)^T (qlinear.mojo:407-477).  x fp32 (the
        reference's boundary) or bf16; y fp32.  Beyond the reference's surface: `bias` / `epilogue`
        (`LinearAct`'s, linear_act.mojo:81-115) and `out_dtype=torch.bfloat16` (a bf16-flow tower takes
        bf16 in and hands bf16 on, without the boundary casts of qlinear.mojo:430-463)."""
        _need_gpu(target)
        if x.dtype not in _TORCH_DT:
            raise L.NQError(L.NQ_ERR_INVALID, "QLinear.forward: x must be fp32 or bf16")
        if out_dtype not in _TORCH_DT:
            raise L.NQError(L.NQ_ERR_INVALID, "QLinear.forward: y must be fp32 or bf16")
        return self._forward(x, _TORCH_DT[x.dtype], None, out, out_dtype, bias, epilogue, "QLinear.forward")

    def vjp(self, forward_input: torch.Tensor, grad_output: torch.Tensor,
            grad_input: Optional[torch.Tensor] = None, target: str = "gpu", ctx=None) -> torch.Tensor:
        """grad_input = grad_output @ deq(W), overwriting it (qlinear.mojo:479-518)."""
        _need_gpu(target)
        M = _check_x(grad_output, self.OUT, "QLinear.vjp")
        if grad_output.dtype != torch.float32:
            raise L.NQError(L.NQ_ERR_INVALID, "QLinear.vjp: grad_output must be fp32")
        if grad_input is None or grad_input.numel() < M * self.IN:
            grad_input = torch.empty((M, self.IN), dtype=torch.float32, device=grad_output.device)
        L.check(L.lib().nq_grad_input(self._h, _dev_ptr(grad_output), _dev_ptr(grad_input), M, _stream_ptr()))
        return grad_input

    def release_buffers(self):
        """The reference drops its bf16 activation staging here
        (qlinear.mojo:520-524); this build has none to drop."""


class W8Linear(_Layer):
    """int8 weight [OUT, IN] with one fp32 scale per output channel.
    Activations fp32/bf16 (W8A32 / W8A16) or int8 with per-token scales (W8A8)."""

    FORMAT = L.FMT_W8_CHANNEL

    @classmethod
    def from_linear(cls, w_in_out, bias=None, tile_copy: bool = True) -> "W8Linear":
        """A drop-in for `Linear[IN, OUT]` / `LinearAct`: W [IN, OUT] fp32 is transposed to [OUT, IN] and quantized
        per output channel (symmetric int8, s = absmax / 127); the fp32 bias, if any, is kept on the device and
        added by forward (pass epilogue="relu" for `LinearAct[..., ReLU]`)."""
        from . import formats as F

        IN, OUT = np.asarray(w_in_out).shape
        lin = cls(IN, OUT, tile_copy=tile_copy)
        wt, lin.bias = cls._linear_params(w_in_out, bias, IN, OUT, "W8Linear.from_linear")
        q, s = F.quantize_w8_channel(wt)
        lin.set_weight(q, s)
        return lin

    def set_weight(self, w_i8, scales):
        w = np.ascontiguousarray(w_i8, dtype=np.int8)
        s = np.ascontiguousarray(scales, dtype=np.float32)
        if w.size != self.IN * self.OUT or s.size != self.OUT:
            raise L.NQError(L.NQ_ERR_SIZE, f"W8Linear.set_weight: expected [{self.OUT}, {self.IN}] codes and "
                                           f"{self.OUT} scales")
        L.check(L.lib().nq_set_weight_i8(self._h, w.ctypes.data_as(C.c_void_p), s.ctypes.data_as(C.c_void_p),
                                         _stream_ptr()))
        self._loaded = True

    def forward(self, x, bias=None, epilogue="none", out=None, out_dtype=torch.float32):
        if x.dtype not in _TORCH_DT:
            raise L.NQError(L.NQ_ERR_INVALID, "W8Linear.forward: x must be fp32 or bf16")
        return self._forward(x, _TORCH_DT[x.dtype], None, out, out_dtype, bias, epilogue, "W8Linear.forward")

    def forward_a8(self, xq, x_scales, bias=None, epilogue="none", out=None, out_dtype=torch.float32):
        """int8 activations [M, IN] with per-token scales [M]: int32
        accumulation, then epi(acc * sx * sw + bias).  out_dtype=torch.int32
        returns the raw accumulators."""
        if xq.dtype != torch.int8:
            raise L.NQError(L.NQ_ERR_INVALID, "W8Linear.forward_a8: xq must be int8")
        return self._forward(xq, L.DT_I8, x_scales, out, out_dtype, bias, epilogue, "W8Linear.forward_a8")


class W4GroupLinear(_Layer):
    """Asymmetric uint4, group-wise along IN: codes [OUT, IN/2] (low nibble =
    even k), fp16 scales [OUT, G], packed uint4 zero-points [OUT, ceil(G/2)]."""

    FORMAT = L.FMT_W4_GROUP

    def __init__(self, IN, OUT, group=128, tile_copy: bool = True, prefer_tile: bool = False):
        super().__init__(IN, OUT, group, tile_copy, prefer_tile)
        self.G = -(-IN // group)

    @classmethod
    def from_linear(cls, w_in_out, bias=None, group: int = 128, tile_copy: bool = True) -> "W4GroupLinear":
        """`Linear[IN, OUT]`'s W [IN, OUT] transposed and quantized to asymmetric uint4, group-wise along IN
        (min / max per group); the fp32 bias, if any, is kept on the device and added by forward."""
        from . import formats as F

        IN, OUT = np.asarray(w_in_out).shape
        lin = cls(IN, OUT, group, tile_copy=tile_copy)
        wt, lin.bias = cls._linear_params(w_in_out, bias, IN, OUT, "W4GroupLinear.from_linear")
        q, s, z = F.quantize_w4g_asym(wt, group)
        codes, zps = F.pack_w4g(q, z)
        lin.set_weight(codes, s, zps)
        return lin

    def set_weight(self, codes, scales_f16, zps):
        c = np.ascontiguousarray(codes, dtype=np.uint8)
        s = np.ascontiguousarray(scales_f16)
        if s.dtype == np.float16:
            s = s.view(np.uint16)
        s = np.ascontiguousarray(s, dtype=np.uint16)
        z = np.ascontiguousarray(zps, dtype=np.uint8)
        if c.size != self.OUT * self.IN // 2 or s.size != self.OUT * self.G or z.size != self.OUT * ((self.G + 1) // 2):
            raise L.NQError(L.NQ_ERR_SIZE, "W4GroupLinear.set_weight: inconsistent sizes")
        L.check(L.lib().nq_set_weight_w4g(self._h, c.ctypes.data_as(C.c_void_p), s.ctypes.data_as(C.c_void_p),
                                          z.ctypes.data_as(C.c_void_p), _stream_ptr()))
        self._loaded = True

    def forward(self, x, bias=None, epilogue="none", out=None, out_dtype=torch.float32):
        if x.dtype not in _TORCH_DT:
            raise L.NQError(L.NQ_ERR_INVALID, "W4GroupLinear.forward: x must be fp32 or bf16")
        return self._forward(x, _TORCH_DT[x.dtype], None, out, out_dtype, bias, epilogue, "W4GroupLinear.forward")


class FP8Linear(_Layer):
    """OCP e4m3fn weight [OUT, IN] with one fp32 scale; activations e4m3fn with
    one fp32 scale (or fp32/bf16); fp32 accumulation; bf16 or fp32 output."""

    FORMAT = L.FMT_FP8_E4M3

    @classmethod
    def from_linear(cls, w_in_out, bias=None) -> "FP8Linear":
        """`Linear[IN, OUT]`'s W [IN, OUT] transposed and encoded as e4m3fn under one scale (absmax / 448); the
        fp32 bias, if any, is kept on the device and added by forward."""
        from . import formats as F

        IN, OUT = np.asarray(w_in_out).shape
        lin = cls(IN, OUT)
        wt, lin.bias = cls._linear_params(w_in_out, bias, IN, OUT, "FP8Linear.from_linear")
        amax = float(np.abs(wt).max())
        scale = amax / 448.0 if amax > 0 else 1.0
        lin.set_weight(F.encode_e4m3(wt / np.float32(scale)), scale)
        return lin

    def set_weight(self, w_codes, scale: float):
        w = np.ascontiguousarray(w_codes, dtype=np.uint8)
        if w.size != self.IN * self.OUT:
            raise L.NQError(L.NQ_ERR_SIZE, f"FP8Linear.set_weight: expected [{self.OUT}, {self.IN}] codes")
        L.check(L.lib().nq_set_weight_fp8(self._h, w.ctypes.data_as(C.c_void_p), C.c_float(scale), _stream_ptr()))
        self._loaded = True

    def forward(self, x_codes, x_scale, bias=None, epilogue="none", out=None, out_dtype=torch.bfloat16):
        """x_codes: uint8 (or torch.float8_e4m3fn) [M, IN]; x_scale: device fp32 [1]."""
        if x_codes.dtype == torch.float8_e4m3fn:
            x_codes = x_codes.view(torch.uint8)
        if x_codes.dtype != torch.uint8:
            raise L.NQError(L.NQ_ERR_INVALID, "FP8Linear.forward: x must be e4m3fn codes")
        return self._forward(x_codes, L.DT_FP8_E4M3, x_scale, out, out_dtype, bias, epilogue, "FP8Linear.forward")

    def forward_a16(self, x: torch.Tensor, bias=None, epilogue="none", out=None, out_dtype=torch.float32):
        """fp32 or bf16 activations over the e4m3fn weight: y = x @ (decode(W) * scale)^T.  The codes enter the
        bf16 matrix cores as their exact decoded values, fp32 activations as three bf16 terms."""
        if x.dtype not in _TORCH_DT:
            raise L.NQError(L.NQ_ERR_INVALID, "FP8Linear.forward_a16: x must be fp32 or bf16")
        return self._forward(x, _TORCH_DT[x.dtype], None, out, out_dtype, bias, epilogue, "FP8Linear.forward_a16")


class FusedRows:
    """Up to four loaded layers that read the same activations (q|k|v, gate|up
    of a decoder layer: `DecoderLayerWeights.proj_fwd`, layer_weights.mojo:455-508)
    as ONE layer: their [OUT, IN] rows are concatenated on the device and
    `forward` writes one dense [M, OUT_t] output per part, what each part's own
    forward writes, in one launch where the kernel allows it."""

    def device_bytes(self) -> int:
        """Device memory of the fused copy of the parts' weights (nq_device_bytes); the parts keep their own."""
        return int(L.lib().nq_device_bytes(self._h))

    def __init__(self, layers):
        layers = list(layers)
        arr = (C.c_void_p * len(layers))(*[l._h for l in layers])
        h = C.c_void_p()
        L.check(L.lib().nq_fuse_rows(C.byref(h), arr, len(layers), _stream_ptr()))
        self._h = h
        self.IN = layers[0].IN
        self.OUTS = [l.OUT for l in layers]
        self.OUT = sum(self.OUTS)
        self._kind = type(layers[0])

    def __del__(self):
        h = getattr(self, "_h", None)
        if h is not None and h.value:
            try:
                L.lib().nq_destroy(h)
            except Exception:
                pass
            self._h = None

    def parts(self) -> int:
        return int(L.lib().nq_fused_parts(self._h))

    def forward(self, x: torch.Tensor, x_scale: Optional[torch.Tensor] = None, outs=None, bias=None,
                epilogue: str = "none", out_dtype: torch.dtype = torch.float32):
        """Returns the list of per-part outputs.  x: fp32/bf16 [M, IN], or e4m3fn
        codes with `x_scale` for fused FP8Linear layers."""
        if x.dtype == torch.float8_e4m3fn:
            x = x.view(torch.uint8)
        if x.dtype == torch.uint8:
            x_dt = L.DT_FP8_E4M3
        elif x.dtype in _TORCH_DT:
            x_dt = _TORCH_DT[x.dtype]
        else:
            raise L.NQError(L.NQ_ERR_INVALID, "FusedRows.forward: x must be fp32, bf16 or e4m3fn codes")
        M = _check_x(x, self.IN, "FusedRows.forward")
        if outs is None:
            outs = [torch.empty((M, n), dtype=out_dtype, device=x.device) for n in self.OUTS]
        y_dt = {torch.float32: L.DT_F32, torch.bfloat16: L.DT_BF16}[out_dtype]
        b_dt = L.DT_F32
        if bias is not None:
            if bias.dtype not in _TORCH_DT or bias.numel() != self.OUT or not bias.is_cuda:
                raise L.NQError(L.NQ_ERR_INVALID, "FusedRows.forward: bias must be a device fp32/bf16 tensor of "
                                                  "sum(OUT) values")
            b_dt = _TORCH_DT[bias.dtype]
        epi = {"none": L.EPI_NONE, "relu": L.EPI_RELU}[epilogue]
        ys = (C.c_void_p * len(outs))(*[_dev_ptr(o) for o in outs])
        L.check(L.lib().nq_forward_fused(self._h, _dev_ptr(x), x_dt, _dev_ptr(x_scale), ys, len(outs), y_dt, M,
                                         _dev_ptr(bias), b_dt, epi, _stream_ptr()))
        return outs


    def forward_lora(self, x: torch.Tensor, adapters, outs=None, bias=None, glu_out: Optional[torch.Tensor] = None,
                     glu_dtype: Optional[torch.dtype] = None):
        """`forward` with one frozen adapter per part (`nq_forward_fused_lora`): the caller's per-projection
        `proj_fwd` = base linear + `LoRAAdapter.forward_add` (layer_weights.mojo:455-508) for a whole group in two
        launches.  `adapters`: one `LoRAAdapter` (or None, or a merged one: no share) per part.  Returns the list of
        fp32 per-part outputs; with `glu_dtype` (or `glu_out`) the two parts are gate and up of one MLP and the
        call returns up * silu(gate) instead ([M, OUT]; the per-part outputs are then scratch holding the base
        projections)."""
        if x.dtype not in _TORCH_DT:
            raise L.NQError(L.NQ_ERR_INVALID, "FusedRows.forward_lora: x must be fp32 or bf16")
        M = _check_x(x, self.IN, "FusedRows.forward_lora")
        adapters = list(adapters)
        if len(adapters) != len(self.OUTS):
            raise L.NQError(L.NQ_ERR_INVALID, "FusedRows.forward_lora: one adapter (or None) per part")
        if outs is None:
            outs = [torch.empty((M, n), dtype=torch.float32, device=x.device) for n in self.OUTS]
        if any(o.dtype != torch.float32 or not o.is_cuda for o in outs):
            raise L.NQError(L.NQ_ERR_INVALID, "FusedRows.forward_lora: the per-part outputs are fp32 device tensors")
        table = (L.LoraPart * len(adapters))()
        for t, ad in enumerate(adapters):
            if ad is None or ad.merged:
                table[t] = L.LoraPart(None, None, 0, 0.0)
                continue
            if ad.IN != self.IN or ad.OUT != self.OUTS[t]:
                raise L.NQError(L.NQ_ERR_INVALID, "FusedRows.forward_lora: adapter %d does not fit its part" % t)
            table[t] = L.LoraPart(ad.lora_A.data_ptr(), ad.lora_B.data_ptr(), ad.R_PAD, ad.scale())
        b_dt = L.DT_F32
        if bias is not None:
            if bias.dtype not in _TORCH_DT or bias.numel() != self.OUT or not bias.is_cuda:
                raise L.NQError(L.NQ_ERR_INVALID, "FusedRows.forward_lora: bias must be a device fp32/bf16 tensor of "
                                                  "sum(OUT) values")
            b_dt = _TORCH_DT[bias.dtype]
        want_glu = glu_out is not None or glu_dtype is not None
        if want_glu:
            if glu_out is None:
                glu_out = torch.empty((M, self.OUTS[0]), dtype=glu_dtype, device=x.device)
            if glu_out.dtype not in _TORCH_DT or glu_out.numel() < M * self.OUTS[0]:
                raise L.NQError(L.NQ_ERR_INVALID, "FusedRows.forward_lora: glu_out must be an fp32/bf16 [M, OUT] tensor")
        ys = (C.c_void_p * len(outs))(*[_dev_ptr(o) for o in outs])
        L.check(L.lib().nq_forward_fused_lora(self._h, _dev_ptr(x), _TORCH_DT[x.dtype], ys, len(outs), M, _dev_ptr(bias),
                                              b_dt, table, _dev_ptr(glu_out) if want_glu else C.c_void_p(0),
                                              _TORCH_DT[glu_out.dtype] if want_glu else L.DT_F32, _stream_ptr()))
        return glu_out if want_glu else outs


class FusedGLU:
    """gate | up of a decoder MLP with the SwiGLU between them and `down` in ONE launch (nq_fuse_glu): the
    reference's caller runs two projections, a concatenation and `SwiGLU.forward`
    (noeira/deep_agents/smolvla/fused.mojo:337-353).  `forward` returns up(x) * silu(gate(x)) as [M, OUT];
    with bf16 in and `out_dtype=torch.bfloat16` nothing of the MLP's first half leaves the GPU's registers in
    fp32 (the bf16 flow the reference lists as unbuilt, peft-quant.mdx:215-216)."""

    def device_bytes(self) -> int:
        """Device memory of the fused copy of the parts' weights (nq_device_bytes); the parts keep their own."""
        return int(L.lib().nq_device_bytes(self._h))

    def __init__(self, gate, up):
        h = C.c_void_p()
        L.check(L.lib().nq_fuse_glu(C.byref(h), gate._h, up._h, _stream_ptr()))
        self._h = h
        self.IN, self.OUT = gate.IN, gate.OUT

    def __del__(self):
        h = getattr(self, "_h", None)
        if h is not None and h.value:
            try:
                L.lib().nq_destroy(h)
            except Exception:
                pass
            self._h = None

    def forward(self, x: torch.Tensor, out: Optional[torch.Tensor] = None,
                out_dtype: torch.dtype = torch.float32) -> torch.Tensor:
        if out is not None:
            out_dtype = out.dtype
        if x.dtype not in _TORCH_DT or out_dtype not in _TORCH_DT:
            raise L.NQError(L.NQ_ERR_INVALID, "FusedGLU.forward: x and y must be fp32 or bf16")
        M = _check_x(x, self.IN, "FusedGLU.forward")
        if out is None or out.numel() < M * self.OUT:
            out = torch.empty((M, self.OUT), dtype=out_dtype, device=x.device)
        L.check(L.lib().nq_forward(self._h, _dev_ptr(x), _TORCH_DT[x.dtype], C.c_void_p(0), _dev_ptr(out),
                                   _TORCH_DT[out_dtype], M, C.c_void_p(0), L.DT_F32, L.EPI_SWIGLU, _stream_ptr()))
        return out

    def forward_lora(self, x: torch.Tensor, gate_adapter, up_adapter, out: Optional[torch.Tensor] = None,
                     out_dtype: torch.dtype = torch.float32) -> torch.Tensor:
        """`forward` with the gate and the up projection's frozen adapters added ahead of the activation, in the same
        single launch (`nq_forward_fused_lora` on a layer made by nq_fuse_glu): up'(x) * silu(gate'(x)) with
        p'(x) = p(x) + scale_p * (x A_p) B_p, i.e. `proj_fwd` on both projections (layer_weights.mojo:455-508) and
        `SwiGLU.forward`.  Both adapters (one padded rank) or neither; raises NQ_ERR_UNSUPPORTED where no kernel can
        add them ahead of SwiGLU (then: `FusedRows.forward_lora(..., glu_dtype=...)`)."""
        if out is not None:
            out_dtype = out.dtype
        if x.dtype not in _TORCH_DT or out_dtype not in _TORCH_DT:
            raise L.NQError(L.NQ_ERR_INVALID, "FusedGLU.forward_lora: x and y must be fp32 or bf16")
        M = _check_x(x, self.IN, "FusedGLU.forward_lora")
        if out is None or out.numel() < M * self.OUT:
            out = torch.empty((M, self.OUT), dtype=out_dtype, device=x.device)
        table = (L.LoraPart * 2)()
        for t, ad in enumerate((gate_adapter, up_adapter)):
            if ad is None or ad.merged:
                table[t] = L.LoraPart(None, None, 0, 0.0)
                continue
            if ad.IN != self.IN or ad.OUT != self.OUT:
                raise L.NQError(L.NQ_ERR_INVALID, "FusedGLU.forward_lora: adapter %d does not fit its projection" % t)
            table[t] = L.LoraPart(ad.lora_A.data_ptr(), ad.lora_B.data_ptr(), ad.R_PAD, ad.scale())
        L.check(L.lib().nq_forward_fused_lora(self._h, _dev_ptr(x), _TORCH_DT[x.dtype], None, 0, M, C.c_void_p(0), L.DT_F32,
                                              table, _dev_ptr(out), _TORCH_DT[out_dtype], _stream_ptr()))
        return out


def quantize_rows_i8(x: torch.Tensor, q: Optional[torch.Tensor] = None, scales: Optional[torch.Tensor] = None):
    """Per-token absmax int8 quantisation on the device: (q int8 [M, K], s fp32 [M])."""
    if x.dtype not in _TORCH_DT or x.dim() != 2 or not x.is_contiguous():
        raise L.NQError(L.NQ_ERR_INVALID, "quantize_rows_i8: x must be a contiguous fp32/bf16 [M, K] device tensor")
    M, K = x.shape
    if q is None:
        q = torch.empty((M, K), dtype=torch.int8, device=x.device)
    if scales is None:
        scales = torch.empty((M,), dtype=torch.float32, device=x.device)
    L.check(L.lib().nq_quantize_rows_i8(_dev_ptr(x), _TORCH_DT[x.dtype], _dev_ptr(q), _dev_ptr(scales), M, K,
                                        _stream_ptr()))
    return q, scales


def cast_pad_bf16(x: torch.Tensor, cols_pad: int) -> torch.Tensor:
    """fp32 [rows, cols] -> bf16 [rows, cols_pad], zero tail (qlinear.mojo:152-172)."""
    rows, cols = x.shape
    out = torch.empty((rows, cols_pad), dtype=torch.bfloat16, device=x.device)
    L.check(L.lib().nq_cast_pad_bf16(_dev_ptr(x), _dev_ptr(out), rows, cols, cols_pad, _stream_ptr()))
    return out


def slice_cast_f32(xb: torch.Tensor, cols: int) -> torch.Tensor:
    """bf16 [rows, cols_pad] -> fp32 [rows, cols] (qlinear.mojo:175-192)."""
    rows, cols_pad = xb.shape
    out = torch.empty((rows, cols), dtype=torch.float32, device=xb.device)
    L.check(L.lib().nq_slice_cast_f32(_dev_ptr(xb), _dev_ptr(out), rows, cols, cols_pad, _stream_ptr()))
    return out


def mlp3_w8a8_forward(l1: W8Linear, l2: W8Linear, l3: W8Linear, x: torch.Tensor, b1=None, b2=None, b3=None,
                      final_relu: bool = False, out: Optional[torch.Tensor] = None) -> torch.Tensor:
    """The three-layer W8A8 actor MLP as one launch (per-token int8 requantisation
    between layers, int32 accumulation, fused ReLU)."""
    M = _check_x(x, l1.IN, "mlp3_w8a8_forward")
    if out is None:
        out = torch.empty((M, l3.OUT), dtype=torch.float32, device=x.device)
    L.check(L.lib().nq_mlp3_w8a8_forward(l1._h, l2._h, l3._h, _dev_ptr(x), _dev_ptr(out), M, _dev_ptr(b1),
                                         _dev_ptr(b2), _dev_ptr(b3), int(final_relu), _stream_ptr()))
    return out
