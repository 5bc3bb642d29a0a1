"""Writers for the checkpoint containers, used by the tests only (the reference has none either:
its tests assemble the bytes by hand, src/gguf.rs:1055-1097, src/hf/safetensors.rs:244-262).
They emit the formats as specified, so that the library's readers are exercised on real files."""
from __future__ import annotations

import json
import struct

import numpy as np

GGUF_MAGIC = 0x46554747
# GGUF metadata value type codes (reference GgufMetaType, src/gguf.rs:262-277)
U8, I8, U16, I16, U32, I32, F32, BOOL, STRING, ARRAY, U64, I64, F64 = range(13)
_FMT = {U8: "<B", I8: "<b", U16: "<H", I16: "<h", U32: "<I", I32: "<i", F32: "<f", BOOL: "<B",
        U64: "<Q", I64: "<q", F64: "<d"}


def _gguf_string(s: str) -> bytes:
    b = s.encode()
    return struct.pack("<Q", len(b)) + b


def _gguf_value(ty, v) -> bytes:
    if ty == STRING:
        return _gguf_string(v)
    if ty == ARRAY:
        et, items = v
        return struct.pack("<IQ", et, len(items)) + b"".join(_gguf_value(et, x) for x in items)
    return struct.pack(_FMT[ty], v)


def gguf_bytes(metadata, tensors, version=3, alignment=32) -> bytes:
    """metadata: [(key, type_code, value)] (ARRAY value = (elem_type, [items]));
    tensors: [(name, logical_shape_outermost_first, ggml_type_code, raw_bytes)]."""
    out = bytearray()
    out += struct.pack("<II", GGUF_MAGIC, version)
    out += struct.pack("<QQ" if version >= 3 else "<II", len(tensors), len(metadata))
    for key, ty, v in metadata:
        out += _gguf_string(key) + struct.pack("<I", ty) + _gguf_value(ty, v)
    offset = 0
    for name, shape, code, raw in tensors:
        out += _gguf_string(name) + struct.pack("<I", len(shape))
        for d in reversed(shape):          # the file stores dimensions innermost first
            out += struct.pack("<Q", d)
        out += struct.pack("<IQ", code, offset)
        offset = (offset + len(raw) + alignment - 1) // alignment * alignment
    out += b"\0" * ((-len(out)) % alignment)
    for _name, _shape, _code, raw in tensors:
        out += bytes(raw)
        out += b"\0" * ((-len(raw)) % alignment)
    return bytes(out)


def safetensors_bytes(tensors, metadata=None) -> bytes:
    """tensors: {name: (dtype_string, shape, raw_bytes)}"""
    header, data = {}, bytearray()
    if metadata is not None:
        header["__metadata__"] = metadata
    for name, (dtype, shape, raw) in tensors.items():
        header[name] = {"dtype": dtype, "shape": list(shape), "data_offsets": [len(data), len(data) + len(raw)]}
        data += bytes(raw)
    h = json.dumps(header, separators=(",", ":")).encode()
    return struct.pack("<Q", len(h)) + h + bytes(data)


def f32_to_bf16_trunc(a: np.ndarray) -> np.ndarray:
    return (np.ascontiguousarray(a, np.float32).view(np.uint32) >> 16).astype(np.uint16)
