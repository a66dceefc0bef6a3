"""dlopen of libnoeira_qlinear.so and its C prototypes.

Resolution order mirrors the reference's native-shim loaders
(noeira/io/serial/native.mojo:57-71): ``$NOEIRA_QLINEAR_LIB`` -> the package
directory -> the bare name.  A missing library is an error, never a fallback:
there is no CPU path behind this package.
"""
from __future__ import annotations

import ctypes as C
import os

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_NAME = "libnoeira_qlinear.so"

# status codes / enums of include/noeira_qlinear.h
NQ_OK, NQ_ERR_INVALID, NQ_ERR_NOT_LOADED, NQ_ERR_NO_BLOCKS, NQ_ERR_SIZE, NQ_ERR_HIP, NQ_ERR_UNSUPPORTED = range(7)
FMT_Q4_0, FMT_W8_CHANNEL, FMT_W4_GROUP, FMT_FP8_E4M3 = range(4)
DT_F32, DT_BF16, DT_I8, DT_FP8_E4M3, DT_I32 = range(5)
EPI_NONE, EPI_RELU, EPI_SWIGLU = 0, 1, 2
ABI_VERSION = 7

FLAG_NO_TILE_COPY = 1
FLAG_PREFER_TILE = 2


class LoraPart(C.Structure):
    """`nq_lora_part`: one adapter of nq_forward_fused_lora (a = b = NULL: the part has none)."""
    _fields_ = [("a", C.c_void_p), ("b", C.c_void_p), ("r_pad", C.c_int32), ("scale", C.c_float)]


EXPORTS = [
    "nq_abi_version", "nq_last_error", "nq_create", "nq_destroy", "nq_set_blocks", "nq_set_weight_f32",
    "nq_set_weight_i8", "nq_set_weight_w4g", "nq_set_weight_fp8", "nq_blocks_bytes", "nq_get_blocks",
    "nq_keep_only_repacked", "nq_device_bytes", "nq_workspace_bytes", "nq_set_workspace", "nq_forward", "nq_dequantize", "nq_grad_input", "nq_quantize_rows_i8",
    "nq_cast_pad_bf16", "nq_slice_cast_f32", "nq_mlp3_w8a8_forward", "nq_fuse_rows", "nq_fused_parts",
    "nq_forward_fused", "nq_fuse_glu", "nq_hessian_create", "nq_hessian_destroy", "nq_hessian_add", "nq_hessian_rows",
    "nq_hessian_get", "nq_hessian_set", "nq_hinv_upper_f64", "nq_hinv_upper_f64_dev", "nq_set_weight_gptq", "nq_q4_0_objective", "nq_lora_forward_add", "nq_forward_lora", "nq_forward_fused_lora", "nq_diag_mfma_rate", "nq_diag_stream_read", "nq_diag_gemm8_timeline", "nq_diag_forward_a16", "nq_diag_forward_gemm8",
]


class NQError(RuntimeError):
    """A non-zero status from the library, carrying its sentence (the Mojo
    wrapper raises ``Error(msg)`` from the same text)."""

    def __init__(self, code: int, msg: str):
        super().__init__(msg)
        self.code = code


def candidates():
    out = []
    override = os.environ.get("NOEIRA_QLINEAR_LIB", "")
    if override:
        out.append(override)
    out.append(os.path.join(_HERE, LIB_NAME))
    out.append(LIB_NAME)
    return out


_lib = None


def lib() -> C.CDLL:
    global _lib
    if _lib is not None:
        return _lib
    # torch first: the device pointers and streams this package hands to the library come from
    # torch, so both must run on the one HIP runtime torch ships (same SONAME; the first one
    # loaded into the process wins).
    import torch  # noqa: F401

    last = None
    for path in candidates():
        if os.sep in path and not os.path.exists(path):
            continue
        try:
            L = C.CDLL(path)
            break
        except OSError as e:  # keep looking, report all at the end
            last = e
    else:
        raise OSError(
            "libnoeira_qlinear.so not found. Tried:\n  - " + "\n  - ".join(candidates())
            + "\nBuild it with `python -m noeira_amd.build`, or set NOEIRA_QLINEAR_LIB=/path/to/"
            + LIB_NAME + (f"\n(last loader error: {last})" if last else ""))
    i32, i64, p, f32 = C.c_int32, C.c_int64, C.c_void_p, C.c_float
    L.nq_abi_version.restype = i32
    L.nq_abi_version.argtypes = []
    L.nq_last_error.restype = i64
    L.nq_last_error.argtypes = [C.c_char_p, i64]
    L.nq_create.restype = i32
    L.nq_create.argtypes = [C.POINTER(p), i32, i32, i32, i32, i32]
    L.nq_destroy.restype = i32
    L.nq_destroy.argtypes = [p]
    L.nq_set_blocks.restype = i32
    L.nq_set_blocks.argtypes = [p, p, i64, p]
    L.nq_set_weight_f32.restype = i32
    L.nq_set_weight_f32.argtypes = [p, p, i64, p]
    L.nq_set_weight_i8.restype = i32
    L.nq_set_weight_i8.argtypes = [p, p, p, p]
    L.nq_set_weight_w4g.restype = i32
    L.nq_set_weight_w4g.argtypes = [p, p, p, p, p]
    L.nq_set_weight_fp8.restype = i32
    L.nq_set_weight_fp8.argtypes = [p, p, f32, p]
    L.nq_blocks_bytes.restype = i64
    L.nq_blocks_bytes.argtypes = [p]
    L.nq_get_blocks.restype = i32
    L.nq_get_blocks.argtypes = [p, p, i64]
    L.nq_keep_only_repacked.restype = i32
    L.nq_keep_only_repacked.argtypes = [p]
    L.nq_forward.restype = i32
    L.nq_forward.argtypes = [p, p, i32, p, p, i32, i32, p, i32, i32, p]
    L.nq_dequantize.restype = i32
    L.nq_dequantize.argtypes = [p, p, i64, p]
    L.nq_grad_input.restype = i32
    L.nq_grad_input.argtypes = [p, p, p, i32, p]
    L.nq_quantize_rows_i8.restype = i32
    L.nq_quantize_rows_i8.argtypes = [p, i32, p, p, i32, i32, p]
    L.nq_cast_pad_bf16.restype = i32
    L.nq_cast_pad_bf16.argtypes = [p, p, i32, i32, i32, p]
    L.nq_slice_cast_f32.restype = i32
    L.nq_slice_cast_f32.argtypes = [p, p, i32, i32, i32, p]
    L.nq_mlp3_w8a8_forward.restype = i32
    L.nq_mlp3_w8a8_forward.argtypes = [p, p, p, p, p, i32, p, p, p, i32, p]
    L.nq_fuse_rows.restype = i32
    L.nq_fuse_rows.argtypes = [C.POINTER(p), C.POINTER(p), i32, p]
    L.nq_fuse_glu.restype = i32
    L.nq_fuse_glu.argtypes = [C.POINTER(p), p, p, p]
    L.nq_fused_parts.restype = i32
    L.nq_fused_parts.argtypes = [p]
    L.nq_forward_fused.restype = i32
    L.nq_forward_fused.argtypes = [p, p, i32, p, C.POINTER(p), i32, i32, i32, p, i32, i32, p]
    f64 = C.c_double
    L.nq_hessian_create.restype = i32
    L.nq_hessian_create.argtypes = [C.POINTER(p), i32]
    L.nq_hessian_destroy.restype = i32
    L.nq_hessian_destroy.argtypes = [p]
    L.nq_hessian_add.restype = i32
    L.nq_hessian_add.argtypes = [p, p, i32, i32, p]
    L.nq_hessian_rows.restype = i64
    L.nq_hessian_rows.argtypes = [p]
    L.nq_hessian_get.restype = i32
    L.nq_hessian_get.argtypes = [p, p, i64]
    L.nq_hessian_set.restype = i32
    L.nq_hessian_set.argtypes = [p, p, i64, i64]
    L.nq_hinv_upper_f64.restype = i32
    L.nq_hinv_upper_f64.argtypes = [p, i32, p, p]
    L.nq_hinv_upper_f64_dev.restype = i32
    L.nq_hinv_upper_f64_dev.argtypes = [p, i32, p, p, p]
    L.nq_set_weight_gptq.restype = i32
    L.nq_set_weight_gptq.argtypes = [p, p, i64, p, f64, C.POINTER(i64), C.POINTER(f64), p]
    L.nq_q4_0_objective.restype = i32
    L.nq_q4_0_objective.argtypes = [p, p, i64, p, C.POINTER(f64), p]
    L.nq_lora_forward_add.restype = i32
    L.nq_lora_forward_add.argtypes = [p, p, i32, i32, i32, f32, p, i32, p, i32, p]
    L.nq_diag_mfma_rate.restype = i32
    L.nq_diag_mfma_rate.argtypes = [p, p, i64, i32, i32, p, p]
    L.nq_diag_stream_read.restype = i32
    L.nq_diag_stream_read.argtypes = [p, i64, p]
    L.nq_forward_fused_lora.restype = i32
    L.nq_forward_fused_lora.argtypes = [p, p, i32, C.POINTER(p), i32, i32, p, i32, C.POINTER(LoraPart), p, i32, p]
    L.nq_forward_lora.restype = i32
    L.nq_forward_lora.argtypes = [p, p, i32, p, i32, i32, p, i32, p, p, i32, C.c_float, p]
    L.nq_diag_forward_gemm8.restype = i32
    L.nq_diag_forward_gemm8.argtypes = [p, p, i32, p, p, i32, i32, p, i32, i32, i32, p]
    L.nq_diag_gemm8_timeline.restype = i32
    L.nq_diag_gemm8_timeline.argtypes = [p, p, i32, p, p, i32, i32, p, i64, p]
    L.nq_device_bytes.restype = i64
    L.nq_device_bytes.argtypes = [p]
    L.nq_workspace_bytes.restype = i64
    L.nq_workspace_bytes.argtypes = [p, i32]
    L.nq_set_workspace.restype = i32
    L.nq_set_workspace.argtypes = [p, p, i64]
    L.nq_diag_forward_a16.restype = i32
    L.nq_diag_forward_a16.argtypes = [p, p, i32, p, i32, i32, i32, i32, p]
    got = L.nq_abi_version()
    if got != ABI_VERSION:
        raise OSError(f"{LIB_NAME}: ABI version {got}, this package binds version {ABI_VERSION}")
    _lib = L
    return L


def last_error() -> str:
    L = lib()
    n = L.nq_last_error(None, 0)
    buf = C.create_string_buffer(int(n) + 1)
    L.nq_last_error(buf, n + 1)
    return buf.value.decode("utf-8", "replace")


def check(rc: int):
    if rc != NQ_OK:
        raise NQError(rc, last_error())
