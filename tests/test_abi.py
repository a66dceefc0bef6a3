"""The C-ABI shared library on a machine without a GPU: it loads through the
same dlopen/dlsym mechanics the reference's `OwnedDLHandle.get_function` uses,
exports every symbol include/noeira_qlinear.h and include/noeira_qlinear_diag.h declare, and its host-side
argument checks raise the reference's sentences.  No compute call is made."""
import ctypes as C
import os
import re

import numpy as np
import pytest

from noeira_amd import _lib as L

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def declared_symbols():
    text = "".join(open(os.path.join(ROOT, "include", f)).read() for f in ("noeira_qlinear.h", "noeira_qlinear_diag.h"))
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(nq_[a-z0-9_]+)\s*\(", text)))


def test_library_loads_and_exports_every_declared_symbol():
    lib = L.lib()
    names = declared_symbols()
    assert len(names) >= 19
    for n in names:
        assert hasattr(lib, n), f"{n} is declared in include/ but not exported"
    assert sorted(L.EXPORTS) == names
    assert lib.nq_abi_version() == L.ABI_VERSION


def test_header_is_plain_c(tmp_path):
    """The header compiles as C99 on its own (no C++ or torch types in it)."""
    import subprocess
    src = tmp_path / "t.c"
    src.write_text('#include "noeira_qlinear.h"\n#include "noeira_qlinear_diag.h"\nint main(void){return NQ_ABI_VERSION - 1;}\n')
    subprocess.check_call(["gcc", "-std=c99", "-Wall", "-Werror", "-I", os.path.join(ROOT, "include"),
                           "-c", str(src), "-o", str(tmp_path / "t.o")])


def _create(fmt, IN, OUT, group=0):
    h = C.c_void_p()
    rc = L.lib().nq_create(C.byref(h), fmt, IN, OUT, group, 0)
    return rc, h


def test_create_validation_sentences():
    rc, _ = _create(L.FMT_Q4_0, 100, 8, 32)
    assert rc == L.NQ_ERR_INVALID and "IN must be a multiple of 32" in L.last_error()  # qlinear.mojo:243-245
    rc, _ = _create(7, 64, 8)
    assert rc == L.NQ_ERR_INVALID and "unknown format" in L.last_error()
    rc, _ = _create(L.FMT_W4_GROUP, 960, 8, 100)
    assert rc == L.NQ_ERR_INVALID
    rc, h = _create(L.FMT_Q4_0, 960, 320, 32)
    assert rc == L.NQ_OK and h.value
    assert L.lib().nq_blocks_bytes(h) == 320 * 30 * 18
    assert L.lib().nq_destroy(h) == L.NQ_OK
    assert L.lib().nq_destroy(None) == L.NQ_OK


def test_lifecycle_errors_before_load():
    """forward / blocks / dequantized before a load raise `no weights (set_weight
    or set_blocks first)` (qlinear.mojo:358-369); a wrong block count raises
    `<n> bytes, expected <BYTES>` (qlinear.mojo:276-281)."""
    lib = L.lib()
    rc, h = _create(L.FMT_Q4_0, 64, 4, 32)
    assert rc == 0
    buf = np.zeros(4 * 2 * 18, np.uint8)
    assert lib.nq_get_blocks(h, buf.ctypes.data_as(C.c_void_p), buf.size) == L.NQ_ERR_NOT_LOADED
    assert "QLinear.blocks: no weights (set_weight or set_blocks first)" == L.last_error()
    assert lib.nq_forward(h, None, 0, None, None, 0, 1, None, 0, 0, None) == L.NQ_ERR_NOT_LOADED
    assert "QLinear.forward: no weights" in L.last_error()
    assert lib.nq_dequantize(h, None, 0, None) == L.NQ_ERR_NOT_LOADED
    assert lib.nq_grad_input(h, None, None, 1, None) == L.NQ_ERR_NOT_LOADED
    assert lib.nq_keep_only_repacked(h) == L.NQ_ERR_NOT_LOADED
    assert lib.nq_set_blocks(h, buf.ctypes.data_as(C.c_void_p), buf.size - 1, None) == L.NQ_ERR_SIZE
    assert L.last_error() == "QLinear[64, 4].set_blocks: 143 bytes, expected 144"
    w = np.zeros(10, np.float32)
    assert lib.nq_set_weight_f32(h, w.ctypes.data_as(C.c_void_p), 10, None) == L.NQ_ERR_SIZE
    assert "10 values for a [4, 64] weight" in L.last_error()
    # a layer of one format refuses another format's loader
    assert lib.nq_set_weight_fp8(h, buf.ctypes.data_as(C.c_void_p), C.c_float(1.0), None) == L.NQ_ERR_INVALID
    # the shared dequantize scratch (`share_scratch`, qlinear.mojo:330-340): its size, and the reference's sentence
    # for a buffer that is too small; no buffer is touched by either call
    assert lib.nq_workspace_bytes(h, 1) == lib.nq_workspace_bytes(h, 4096) == 4 * 4 * 64
    assert lib.nq_workspace_bytes(None, 1) == 0
    assert lib.nq_set_workspace(h, C.c_void_p(4096), 4 * 4 * 64 - 4) == L.NQ_ERR_SIZE
    assert L.last_error() == "QLinear.share_scratch: 255 values for a [4, 64] weight"
    assert lib.nq_set_workspace(h, C.c_void_p(4104), 4 * 4 * 64) == L.NQ_ERR_INVALID   # not 16-byte aligned
    assert lib.nq_set_workspace(h, None, 4 * 4 * 64) == L.NQ_ERR_INVALID
    assert lib.nq_set_workspace(h, C.c_void_p(4096), 4 * 4 * 64) == 0
    assert lib.nq_set_workspace(h, None, 0) == 0
    lib.nq_destroy(h)


def test_last_error_truncates():
    _create(7, 64, 8)
    full = L.last_error()
    b = C.create_string_buffer(8)
    n = L.lib().nq_last_error(b, 8)
    assert n == len(full.encode()) and b.value == full.encode()[:7]


def test_missing_library_is_loud(monkeypatch, tmp_path):
    """No library, no fallback: the loader names what it tried."""
    import importlib
    import noeira_amd._lib as mod
    monkeypatch.setattr(mod, "_lib", None)
    monkeypatch.setattr(mod, "candidates", lambda: [str(tmp_path / "nope.so")])
    with pytest.raises(OSError, match="not found"):
        mod.lib()
    monkeypatch.undo()
    importlib.reload(mod)


def test_mirror_refuses_cpu_target():
    from noeira_amd.qlinear import QLinear
    with pytest.raises(L.NQError, match="no CPU path"):
        QLinear.make(64, 4, target="cpu")


def test_bench_refuses_more_than_one_gpu():
    """The path runs on one GPU: `bench.py --gpus N` with N > 1 exits with a message saying so."""
    import subprocess
    import sys

    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    r = subprocess.run([sys.executable, os.path.join(root, "bench.py"), "--gpus", "2"], capture_output=True, text=True,
                       timeout=120)
    assert r.returncode != 0
    assert "one GPU" in r.stderr
