"""ctypes/numpy front end of the CPU oracle (oracle/nq_oracle.c).

TEST INFRASTRUCTURE ONLY: imported by tests/, by __graft_entry__.smoke() and
by bench.py's cpu_baseline leg, never by the noeira_amd package.  Every
function here is a thin wrapper that hands numpy buffers to the C restatement;
the citations of the reference live beside the C functions.
"""
from __future__ import annotations

import ctypes as C
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_SO = os.path.join(_HERE, "libnq_oracle.so")

Q4_GROUP = 32
Q4_BLOCK = 18


def build(force: bool = False) -> str:
    """Compile oracle/nq_oracle.c with gcc (oracle/Makefile)."""
    src = os.path.join(_HERE, "nq_oracle.c")
    if force or not os.path.exists(_SO) or os.path.getmtime(_SO) < os.path.getmtime(src):
        subprocess.check_call(["make", "-C", _HERE, "-B", "libnq_oracle.so"],
                              stdout=subprocess.DEVNULL)
    return _SO


_lib = None


def lib() -> C.CDLL:
    global _lib
    if _lib is None:
        if not os.path.exists(_SO):
            build()
        L = C.CDLL(_SO)
        i64, f32, p = C.c_int64, C.c_float, C.c_void_p
        L.nqo_q4_0_row_bytes.restype = i64
        L.nqo_q4_0_row_bytes.argtypes = [i64]
        L.nqo_f32_to_bf16_bits.restype = C.c_uint16
        L.nqo_f32_to_bf16_bits.argtypes = [f32]
        L.nqo_bf16_round.restype = f32
        L.nqo_bf16_round.argtypes = [f32]
        L.nqo_round_half_even.restype = f32
        L.nqo_round_half_even.argtypes = [f32]
        L.nqo_f16_value.restype = f32
        L.nqo_f16_value.argtypes = [C.c_uint16]
        L.nqo_f16_bits.restype = C.c_uint16
        L.nqo_f16_bits.argtypes = [f32]
        L.nqo_q4_0_group_scale.restype = f32
        L.nqo_q4_0_group_scale.argtypes = [p]
        L.nqo_q4_0_code.restype = C.c_uint8
        L.nqo_q4_0_code.argtypes = [f32, f32]
        for name in ("nqo_quantize_rtn_q4_0", "nqo_pack_q4_0", "nqo_unpack_q4_0"):
            getattr(L, name).restype = C.c_int
        L.nqo_quantize_rtn_q4_0.argtypes = [p, i64, i64, p, p]
        L.nqo_pack_q4_0.argtypes = [p, p, i64, i64, p]
        L.nqo_unpack_q4_0.argtypes = [p, i64, i64, p, p]
        L.nqo_rtn_q4_0_blocks.restype = C.c_int
        L.nqo_rtn_q4_0_blocks.argtypes = [p, i64, i64, p]
        L.nqo_dequantize_q4_0.restype = C.c_int
        L.nqo_dequantize_q4_0.argtypes = [p, i64, i64, p]
        L.nqo_gemm_cpu.restype = None
        L.nqo_gemm_cpu.argtypes = [C.c_int, C.c_int, i64, i64, i64, f32, p, i64, p, i64, f32, p, i64]
        L.nqo_qlinear_forward_cpu.restype = C.c_int
        L.nqo_qlinear_forward_cpu.argtypes = [p, i64, i64, p, i64, p]
        L.nqo_qlinear_vjp_cpu.restype = C.c_int
        L.nqo_qlinear_vjp_cpu.argtypes = [p, i64, i64, p, i64, p]
        L.nqo_dense_forward_f64.restype = None
        L.nqo_dense_forward_f64.argtypes = [p, i64, i64, p, i64, p]
        L.nqo_dense_forward_cpu.restype = None
        L.nqo_dense_forward_cpu.argtypes = [p, i64, i64, p, i64, p]
        L.nqo_rel_max.restype = C.c_double
        L.nqo_rel_max.argtypes = [p, p, i64]
        L.nqo_cast_pad_bf16.restype = None
        L.nqo_cast_pad_bf16.argtypes = [p, i64, i64, i64, p]
        L.nqo_slice_cast_f32.restype = None
        L.nqo_slice_cast_f32.argtypes = [p, i64, i64, i64, p]
        L.nqo_w8_forward_f32.restype = None
        L.nqo_w8_forward_f32.argtypes = [p, p, i64, i64, p, i64, p, C.c_int, p]
        L.nqo_w8_forward_f64.restype = None
        L.nqo_w8_forward_f64.argtypes = [p, p, i64, i64, p, i64, p, C.c_int, p]
        L.nqo_quantize_rows_i8.restype = None
        L.nqo_quantize_rows_i8.argtypes = [p, i64, i64, p, p]
        L.nqo_w8a8_acc_i32.restype = None
        L.nqo_w8a8_acc_i32.argtypes = [p, p, i64, i64, i64, p]
        L.nqo_w8a8_epilogue.restype = None
        L.nqo_w8a8_epilogue.argtypes = [p, p, p, p, C.c_int, i64, i64, p]
        L.nqo_w4g_dequantize.restype = None
        L.nqo_w4g_dequantize.argtypes = [p, p, p, i64, i64, i64, p]
        L.nqo_e4m3_decode.restype = f32
        L.nqo_e4m3_decode.argtypes = [C.c_uint8]
        L.nqo_e4m3_encode.restype = C.c_uint8
        L.nqo_e4m3_encode.argtypes = [f32]
        L.nqo_fp8_forward_f64.restype = None
        L.nqo_fp8_forward_f64.argtypes = [p, p, i64, i64, i64, f32, f32, p, p]
        L.nqo_fp8_qlinear_forward_cpu.restype = C.c_int
        L.nqo_fp8_qlinear_forward_cpu.argtypes = [p, f32, i64, i64, p, f32, i64, p, p]
        L.nqo_e4m3_dequantize.restype = None
        L.nqo_e4m3_dequantize.argtypes = [p, i64, p]
        L.nqo_w8_qlinear_forward_cpu.restype = C.c_int
        L.nqo_w8_qlinear_forward_cpu.argtypes = [p, p, i64, i64, p, i64, p, p]
        for name in ("nqo_e4m3_encode_array", "nqo_f16_bits_array", "nqo_f16_value_array"):
            getattr(L, name).restype = None
            getattr(L, name).argtypes = [p, i64, p]
        L.nqo_lora_forward_add.restype = C.c_int
        L.nqo_lora_forward_add.argtypes = [p, p, p, i64, i64, i64, i64, f32, p]
        L.nqo_swiglu.restype = None
        L.nqo_swiglu.argtypes = [p, p, i64, p]
        L.nqo_cholesky_f64.restype = i64
        L.nqo_cholesky_f64.argtypes = [p, i64]
        L.nqo_tri_inv_lower_f64.restype = None
        L.nqo_tri_inv_lower_f64.argtypes = [p, i64, p]
        L.nqo_hinv_upper_f64.restype = i64
        L.nqo_hinv_upper_f64.argtypes = [p, i64, p]
        L.nqo_gptq_q4_0.restype = C.c_int
        L.nqo_gptq_q4_0.argtypes = [p, i64, i64, p, p, p, C.c_double, p, p]
        L.nqo_q4_0_objective.restype = C.c_double
        L.nqo_q4_0_objective.argtypes = [p, p, p, i64, i64, p]
        L.nqo_hessian_add.restype = None
        L.nqo_hessian_add.argtypes = [p, i64, p, i64]
        _lib = L
    return _lib


def _c(a, dtype):
    a = np.ascontiguousarray(a, dtype=dtype)
    return a


def _ptr(a):
    return a.ctypes.data_as(C.c_void_p) if a is not None else None


# ── scalar helpers ─────────────────────────────────────────────────────────
def bf16_round(x):
    return bf16_value(bf16_bits(x))


def bf16_bits(x):
    """fp32 array -> uint16 bf16 bits (round to nearest even), via the
    cast_pad routine with no padding."""
    x = _c(x, np.float32)
    out = np.empty(x.shape, np.uint16)
    lib().nqo_cast_pad_bf16(_ptr(x), 1, x.size, x.size, _ptr(out))
    return out


def bf16_value(bits):
    bits = _c(bits, np.uint16)
    out = np.empty(bits.shape, np.float32)
    lib().nqo_slice_cast_f32(_ptr(bits), 1, bits.size, bits.size, _ptr(out))
    return out


def f16_value(bits):
    bits = _c(bits, np.uint16)
    out = np.empty(bits.shape, np.float32)
    lib().nqo_f16_value_array(_ptr(bits), bits.size, _ptr(out))
    return out


def f16_bits(x):
    x = _c(x, np.float32)
    out = np.empty(x.shape, np.uint16)
    lib().nqo_f16_bits_array(_ptr(x), x.size, _ptr(out))
    return out


def round_half_even(x: float) -> float:
    return lib().nqo_round_half_even(float(x))


# ── Q4_0 ───────────────────────────────────────────────────────────────────
def q4_0_row_bytes(k: int) -> int:
    return lib().nqo_q4_0_row_bytes(k)


def quantize_rtn_q4_0(w):
    w = _c(w, np.float32)
    n, k = w.shape
    q = np.empty((n, k), np.uint8)
    d = np.empty((n, k // Q4_GROUP), np.float32)
    rc = lib().nqo_quantize_rtn_q4_0(_ptr(w), n, k, _ptr(q), _ptr(d))
    if rc:
        raise ValueError(f"quantize_rtn_q4_0: k = {k} is not a multiple of 32")
    return q, d


def pack_q4_0(q, d_bits):
    q = _c(q, np.uint8)
    d_bits = _c(d_bits, np.uint16)
    n, k = q.shape
    out = np.empty((n, (k // Q4_GROUP) * Q4_BLOCK), np.uint8)
    rc = lib().nqo_pack_q4_0(_ptr(q), _ptr(d_bits), n, k, _ptr(out))
    if rc:
        raise ValueError("pack_q4_0: inconsistent sizes")
    return out


def unpack_q4_0(blocks, n, k):
    blocks = _c(blocks, np.uint8)
    q = np.empty((n, k), np.uint8)
    bits = np.empty((n, k // Q4_GROUP), np.uint16)
    rc = lib().nqo_unpack_q4_0(_ptr(blocks), n, k, _ptr(q), _ptr(bits))
    if rc:
        raise ValueError("unpack_q4_0: inconsistent sizes")
    return q, bits


def rtn_q4_0_blocks(w):
    w = _c(w, np.float32)
    n, k = w.shape
    out = np.empty((n, (k // Q4_GROUP) * Q4_BLOCK), np.uint8)
    rc = lib().nqo_rtn_q4_0_blocks(_ptr(w), n, k, _ptr(out))
    if rc:
        raise ValueError("rtn_q4_0_blocks failed")
    return out


def lora_forward_add(x, a, b, s, y):
    """y[T, OUT] += s * (x[T, IN] @ a[IN, R]) @ b[R, OUT], in place, as lora.mojo:305-318."""
    x, a, b = _c(x, np.float32), _c(a, np.float32), _c(b, np.float32)
    assert y.dtype == np.float32 and y.flags.c_contiguous
    T, IN = x.shape
    R, OUT = b.shape
    assert a.shape == (IN, R) and y.shape == (T, OUT)
    lib().nqo_lora_forward_add(_ptr(x), _ptr(a), _ptr(b), T, IN, OUT, R, float(s), _ptr(y))
    return y


# ── GPTQ (gptq.mojo, dense.mojo, hessian.mojo) ─────────────────────────────
def swiglu(u, v):
    """`SwiGLU.forward` on (u, v) of equal shape: u * (v / (1 + exp(-v))) in fp32 (swiglu.mojo:120-141)."""
    u, v = _c(u, np.float32), _c(v, np.float32)
    out = np.empty_like(u)
    lib().nqo_swiglu(_ptr(u), _ptr(v), u.size, _ptr(out))
    return out


def cholesky_f64(a):
    """L (lower, L L^T = a); raises at a non-positive pivot like dense.mojo:229-236."""
    a = np.array(a, dtype=np.float64, order="C")
    n = a.shape[0]
    rc = lib().nqo_cholesky_f64(_ptr(a), n)
    if rc:
        raise ValueError(f"cholesky_f64: not positive definite (pivot {rc - 1})")
    return a


def tri_inv_lower_f64(l):
    l = _c(l, np.float64)
    x = np.empty_like(l)
    lib().nqo_tri_inv_lower_f64(_ptr(l), l.shape[0], _ptr(x))
    return x


def hinv_upper_f64(h):
    """U upper triangular with U^T U = h^-1 (dense.mojo:355-363)."""
    h = np.array(h, dtype=np.float64, order="C")
    u = np.empty_like(h)
    rc = lib().nqo_hinv_upper_f64(_ptr(h), h.shape[0], _ptr(u))
    if rc:
        raise ValueError(f"hinv_upper_f64: not positive definite (pivot {rc - 1})")
    return u


def gptq_q4_0(w, h, damp_frac=0.01):
    """(codes [n, k] u8, scales [n, k/32] f32, dead, damp) as gptq.mojo:62-150."""
    w = _c(w, np.float32)
    n, k = w.shape
    if k % Q4_GROUP != 0:
        raise ValueError(f"gptq_q4_0: k = {k} is not a multiple of 32")
    h = np.array(h, dtype=np.float64, order="C")
    if h.size < k * k:
        raise ValueError("gptq_q4_0: w or h is smaller than [n, k] / [k, k]")
    q = np.zeros((n, k), np.uint8)
    d = np.zeros((n, k // Q4_GROUP), np.float32)
    dead = C.c_int64(0)
    damp = C.c_double(0)
    rc = lib().nqo_gptq_q4_0(_ptr(w), n, k, _ptr(h), _ptr(q), _ptr(d), damp_frac, C.byref(dead), C.byref(damp))
    if rc:
        raise ValueError("gptq_q4_0: the damped Hessian is not positive definite")
    return q, d, dead.value, damp.value


def q4_0_objective(w, q, d, h) -> float:
    w = _c(w, np.float32)
    q = _c(q, np.uint8)
    d = _c(d, np.float32)
    h = _c(h, np.float64)
    n, k = w.shape
    return float(lib().nqo_q4_0_objective(_ptr(w), _ptr(q), _ptr(d), n, k, _ptr(h)))


def hessian_add(h, x):
    """h [n, n] f64 += x^T x for x [rows, n] f32, in place (hessian.mojo:41-77)."""
    x = _c(x, np.float32)
    assert h.dtype == np.float64 and h.flags.c_contiguous
    lib().nqo_hessian_add(_ptr(h), h.shape[0], _ptr(x), x.shape[0])
    return h


def dequantize_q4_0(blocks, n, k):
    blocks = _c(blocks, np.uint8)
    out = np.empty((n, k), np.float32)
    rc = lib().nqo_dequantize_q4_0(_ptr(blocks), n, k, _ptr(out))
    if rc:
        raise ValueError("dequantize_q4_0: inconsistent sizes")
    return out


def gemm_cpu(ta, tb, M, N, K, alpha, a, lda, b, ldb, beta, c, ldc):
    a = _c(a, np.float32)
    b = _c(b, np.float32)
    assert c.dtype == np.float32 and c.flags.c_contiguous
    lib().nqo_gemm_cpu(int(ta), int(tb), M, N, K, alpha, _ptr(a), lda, _ptr(b), ldb, beta, _ptr(c), ldc)
    return c


def qlinear_forward_cpu(blocks, IN, OUT, x):
    blocks = _c(blocks, np.uint8)
    x = _c(x, np.float32)
    B = x.size // IN
    y = np.empty((B, OUT), np.float32)
    rc = lib().nqo_qlinear_forward_cpu(_ptr(blocks), IN, OUT, _ptr(x), B, _ptr(y))
    if rc:
        raise ValueError("qlinear_forward_cpu failed")
    return y


def qlinear_vjp_cpu(blocks, IN, OUT, gy):
    blocks = _c(blocks, np.uint8)
    gy = _c(gy, np.float32)
    B = gy.size // OUT
    gx = np.empty((B, IN), np.float32)
    rc = lib().nqo_qlinear_vjp_cpu(_ptr(blocks), IN, OUT, _ptr(gy), B, _ptr(gx))
    if rc:
        raise ValueError("qlinear_vjp_cpu failed")
    return gx


def dense_forward_f64(w, x):
    """Exact fp64 product y[M, N] = x[M, K] @ w[N, K]^T over fp32 operands."""
    w = _c(w, np.float32)
    x = _c(x, np.float32)
    N, K = w.shape
    M = x.size // K
    y = np.empty((M, N), np.float64)
    lib().nqo_dense_forward_f64(_ptr(w), N, K, _ptr(x), M, _ptr(y))
    return y


def dense_forward_cpu(w, x):
    w = _c(w, np.float32)
    x = _c(x, np.float32)
    N, K = w.shape
    M = x.size // K
    y = np.empty((M, N), np.float32)
    lib().nqo_dense_forward_cpu(_ptr(w), N, K, _ptr(x), M, _ptr(y))
    return y


def rel_max(a, b) -> float:
    a = _c(a, np.float32)
    b = _c(b, np.float32)
    return lib().nqo_rel_max(_ptr(a), _ptr(b), a.size)


def cast_pad_bf16(x, cols_pad):
    x = _c(x, np.float32)
    rows, cols = x.shape
    out = np.empty((rows, cols_pad), np.uint16)
    lib().nqo_cast_pad_bf16(_ptr(x), rows, cols, cols_pad, _ptr(out))
    return out


def slice_cast_f32(bits, cols):
    bits = _c(bits, np.uint16)
    rows, cols_pad = bits.shape
    out = np.empty((rows, cols), np.float32)
    lib().nqo_slice_cast_f32(_ptr(bits), rows, cols, cols_pad, _ptr(out))
    return out


# ── extension formats ──────────────────────────────────────────────────────
def w8_forward_f32(w, s, x, bias=None, relu=False):
    w = _c(w, np.int8)
    s = _c(s, np.float32)
    x = _c(x, np.float32)
    N, K = w.shape
    M = x.size // K
    b = _c(bias, np.float32) if bias is not None else None
    y = np.empty((M, N), np.float32)
    lib().nqo_w8_forward_f32(_ptr(w), _ptr(s), N, K, _ptr(x), M, _ptr(b), int(relu), _ptr(y))
    return y


def w8_forward_f64(w, s, x, bias=None, relu=False):
    w = _c(w, np.int8)
    s = _c(s, np.float32)
    x = _c(x, np.float32)
    N, K = w.shape
    M = x.size // K
    b = _c(bias, np.float32) if bias is not None else None
    y = np.empty((M, N), np.float64)
    lib().nqo_w8_forward_f64(_ptr(w), _ptr(s), N, K, _ptr(x), M, _ptr(b), int(relu), _ptr(y))
    return y


def w8_qlinear_forward_cpu(w, s, x, bias=None, out=None):
    """Dequantize-to-scratch then serial GEMM, as QLinear.forward["cpu"] does."""
    w = _c(w, np.int8)
    s = _c(s, np.float32)
    x = _c(x, np.float32)
    N, K = w.shape
    M = x.size // K
    b = _c(bias, np.float32) if bias is not None else None
    y = out if out is not None else np.empty((M, N), np.float32)
    rc = lib().nqo_w8_qlinear_forward_cpu(_ptr(w), _ptr(s), N, K, _ptr(x), M, _ptr(b), _ptr(y))
    if rc:
        raise MemoryError("w8_qlinear_forward_cpu")
    return y


def quantize_rows_i8(x):
    x = _c(x, np.float32)
    M, K = x.shape
    q = np.empty((M, K), np.int8)
    s = np.empty((M,), np.float32)
    lib().nqo_quantize_rows_i8(_ptr(x), M, K, _ptr(q), _ptr(s))
    return q, s


def w8a8_acc_i32(xq, w):
    xq = _c(xq, np.int8)
    w = _c(w, np.int8)
    M, K = xq.shape
    N = w.shape[0]
    acc = np.empty((M, N), np.int32)
    lib().nqo_w8a8_acc_i32(_ptr(xq), _ptr(w), M, N, K, _ptr(acc))
    return acc


def w8a8_epilogue(acc, sx, sw, bias=None, relu=False):
    acc = _c(acc, np.int32)
    sx = _c(sx, np.float32)
    sw = _c(sw, np.float32)
    M, N = acc.shape
    b = _c(bias, np.float32) if bias is not None else None
    y = np.empty((M, N), np.float32)
    lib().nqo_w8a8_epilogue(_ptr(acc), _ptr(sx), _ptr(sw), _ptr(b), int(relu), M, N, _ptr(y))
    return y


def w4g_dequantize(codes, scales_f16_bits, zps, N, K, group):
    codes = _c(codes, np.uint8)
    scales = _c(scales_f16_bits, np.uint16)
    zps = _c(zps, np.uint8)
    out = np.empty((N, K), np.float32)
    lib().nqo_w4g_dequantize(_ptr(codes), _ptr(scales), _ptr(zps), N, K, group, _ptr(out))
    return out


def e4m3_decode_table():
    L = lib()
    return np.array([L.nqo_e4m3_decode(i) for i in range(256)], np.float32)


def e4m3_decode(codes):
    codes = _c(codes, np.uint8)
    out = np.empty(codes.shape, np.float32)
    lib().nqo_e4m3_dequantize(_ptr(codes), codes.size, _ptr(out))
    return out


def e4m3_encode(x):
    x = _c(x, np.float32)
    out = np.empty(x.shape, np.uint8)
    lib().nqo_e4m3_encode_array(_ptr(x), x.size, _ptr(out))
    return out


def fp8_forward_f64(a, b, sa, sb, want_bf16=True):
    a = _c(a, np.uint8)
    b = _c(b, np.uint8)
    M, K = a.shape
    N = b.shape[0]
    y64 = np.empty((M, N), np.float64)
    ob = np.empty((M, N), np.uint16) if want_bf16 else None
    lib().nqo_fp8_forward_f64(_ptr(a), _ptr(b), M, N, K, sa, sb, _ptr(y64), _ptr(ob))
    return y64, ob


def fp8_qlinear_forward_cpu(w, sb, a, sa, want_bf16=False):
    """Dequantize-to-scratch then serial GEMM, as QLinear.forward["cpu"] does, for e4m3 weights and activations."""
    w = _c(w, np.uint8)
    a = _c(a, np.uint8)
    N, K = w.shape
    M = a.size // K
    y = np.empty((M, N), np.float32)
    ob = np.empty((M, N), np.uint16) if want_bf16 else None
    rc = lib().nqo_fp8_qlinear_forward_cpu(_ptr(w), sb, N, K, _ptr(a), sa, M, _ptr(y), _ptr(ob))
    if rc:
        raise MemoryError("fp8_qlinear_forward_cpu")
    return (y, ob) if want_bf16 else y
