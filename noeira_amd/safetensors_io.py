"""Minimal safetensors reader/writer for the quantized-weight files.

A deployed Q4_0 layer is not part of the fp32 checkpoint: its blocks live as a
U8 tensor ``[OUT, IN/32*18]`` named ``<torch weight name>.q4_0`` in a
safetensors file (reference: noeira/deep_agents/smolvla/layer_weights.mojo:136-142
for the key, :853-863 for the shape check; reader noeira/io/safetensors.mojo:446
``read_raw``, writer :769 ``add_u8`` / :827 ``save``).

The format is an 8-byte little-endian header length, a JSON header
``{name: {"dtype", "shape", "data_offsets"}}`` padded with spaces to 8 bytes,
then the raw tensor bytes.  Nothing in a file is executed.
"""
from __future__ import annotations

import json
import struct

import numpy as np

_DTYPES = {
    "F32": np.float32, "F64": np.float64, "F16": np.float16, "BF16": np.uint16,
    "U8": np.uint8, "I8": np.int8, "I32": np.int32, "I64": np.int64, "U16": np.uint16,
    "F8_E4M3": np.uint8,
}
_NAMES = {np.dtype(np.float32): "F32", np.dtype(np.uint8): "U8", np.dtype(np.int8): "I8",
          np.dtype(np.float16): "F16", np.dtype(np.int32): "I32", np.dtype(np.float64): "F64",
          np.dtype(np.int64): "I64", np.dtype(np.uint16): "U16"}

Q4_GROUP = 32
Q4_BLOCK = 18


class SafeTensors:
    """Read-only view of one file (mirrors the reference's ``SafeTensors``)."""

    def __init__(self, path: str):
        self.path = path
        with open(path, "rb") as f:
            (hlen,) = struct.unpack("<Q", f.read(8))
            self._header = json.loads(f.read(hlen).decode("utf-8"))
            self._base = 8 + hlen
        self._header.pop("__metadata__", None)

    def names(self):
        return list(self._header.keys())

    def _entry(self, name: str):
        if name not in self._header:
            raise KeyError(f"safetensors: '{self.path}' has no tensor '{name}'")
        return self._header[name]

    def dtype_of(self, name: str) -> str:
        return self._entry(name)["dtype"]

    def shape(self, name: str):
        return list(self._entry(name)["shape"])

    def shape_str(self, name: str) -> str:
        return "[" + ", ".join(str(s) for s in self.shape(name)) + "]"

    def read_raw(self, name: str) -> np.ndarray:
        """The tensor's bytes, as a flat uint8 array."""
        e = self._entry(name)
        a, b = e["data_offsets"]
        with open(self.path, "rb") as f:
            f.seek(self._base + a)
            return np.frombuffer(f.read(b - a), np.uint8).copy()

    def read(self, name: str) -> np.ndarray:
        e = self._entry(name)
        if e["dtype"] not in _DTYPES:
            raise ValueError(f"safetensors: dtype {e['dtype']} of '{name}' is not supported")
        return self.read_raw(name).view(_DTYPES[e["dtype"]]).reshape(e["shape"])

    def read_f32(self, name: str) -> np.ndarray:
        if self.dtype_of(name) != "F32":
            raise ValueError(f"safetensors: '{name}' is {self.dtype_of(name)}, not F32")
        return self.read(name)


class SafeTensorsWriter:
    def __init__(self):
        self._tensors = {}

    def add(self, name: str, array: np.ndarray):
        a = np.ascontiguousarray(array)
        if a.dtype not in _NAMES:
            raise ValueError(f"safetensors: cannot write dtype {a.dtype}")
        if name in self._tensors:
            raise ValueError(f"safetensors: '{name}' added twice")
        self._tensors[name] = a

    def add_u8(self, name: str, shape, data):
        a = np.ascontiguousarray(data, dtype=np.uint8).reshape(shape)
        self.add(name, a)

    def save(self, path: str):
        header, off = {}, 0
        for name, a in self._tensors.items():
            n = a.nbytes
            header[name] = {"dtype": _NAMES[a.dtype], "shape": list(a.shape),
                            "data_offsets": [off, off + n]}
            off += n
        h = json.dumps(header, separators=(",", ":")).encode()
        h += b" " * ((8 - len(h) % 8) % 8)
        with open(path, "wb") as f:
            f.write(struct.pack("<Q", len(h)))
            f.write(h)
            for a in self._tensors.values():
                f.write(a.tobytes())


def q4_blocks_key(torch_weight_name: str) -> str:
    """``<name>.q4_0`` (layer_weights.mojo:136-142)."""
    return torch_weight_name + ".q4_0"


def load_q4_blocks(blocks_file: SafeTensors, torch_weight_name: str, IN: int, OUT: int) -> np.ndarray:
    """The Q4_0 blocks of one projection, shape-checked as the reference's
    loader does (layer_weights.mojo:853-863)."""
    key = q4_blocks_key(torch_weight_name)
    row = (IN // Q4_GROUP) * Q4_BLOCK
    shape = blocks_file.shape(key)
    if len(shape) != 2 or shape[0] != OUT or shape[1] != row:
        raise ValueError(
            f"load_q4_blocks: '{key}' is {blocks_file.shape_str(key)}, expected [{OUT}, {row}]")
    if blocks_file.dtype_of(key) != "U8":
        raise ValueError(f"load_q4_blocks: '{key}' is {blocks_file.dtype_of(key)}, expected U8")
    return blocks_file.read_raw(key)
