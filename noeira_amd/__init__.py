"""noeira_amd — noeira's quantized-linear inference path on AMD MI355X (gfx950).

Hand-written HIP kernels behind a C ABI (include/noeira_qlinear.h) and a thin
host mirror of the reference's ``QLinear`` operator.  Importing this package
does not load the library; the first use does, and fails loudly when
libnoeira_qlinear.so is missing (there is no CPU path).
"""
from ._lib import NQError  # noqa: F401

__all__ = ["NQError", "QLinear", "W8Linear", "W4GroupLinear", "FP8Linear", "FusedRows"]


def __getattr__(name):
    if name in ("QLinear", "W8Linear", "W4GroupLinear", "FP8Linear", "quantize_rows_i8",
                "cast_pad_bf16", "slice_cast_f32", "mlp3_w8a8_forward", "FusedRows"):
        from . import qlinear

        return getattr(qlinear, name)
    raise AttributeError(name)
