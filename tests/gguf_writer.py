"""A small GGUF (v3) writer for tests: typed metadata, tensor infos, aligned tensor data."""
import struct

import numpy as np

T_U32, T_I32, T_F32, T_BOOL, T_STRING, T_ARRAY, T_U64 = 4, 5, 6, 7, 8, 9, 10


def _s(x: str) -> bytes:
    b = x.encode()
    return struct.pack("<Q", len(b)) + b


def _value(v) -> bytes:
    if isinstance(v, bool):
        return struct.pack("<IB", T_BOOL, int(v))
    if isinstance(v, int):
        return struct.pack("<II", T_U32, v)
    if isinstance(v, float):
        return struct.pack("<If", T_F32, v)
    if isinstance(v, str):
        return struct.pack("<I", T_STRING) + _s(v)
    if isinstance(v, list):   # array of strings
        return struct.pack("<IIQ", T_ARRAY, T_STRING, len(v)) + b"".join(_s(x) for x in v)
    raise TypeError(type(v))


def write_gguf(path, metadata: dict, tensors: list, alignment: int = 32, version: int = 3):
    """tensors: [(name, ggml_type, (rows, cols) or (n,), raw_bytes)]"""
    out = bytearray(struct.pack("<IIQQ", 0x46554747, version, len(tensors), len(metadata)))
    for k, v in metadata.items():
        out += _s(k) + _value(v)
    offset = 0
    for name, gtype, shape, raw in tensors:
        dims = list(reversed(shape))                      # ne[0] is the innermost dimension
        out += _s(name) + struct.pack("<I", len(dims)) + b"".join(struct.pack("<Q", d) for d in dims)
        out += struct.pack("<IQ", gtype, offset)
        offset += (len(raw) + alignment - 1) // alignment * alignment
    out += b"\0" * ((-len(out)) % alignment)
    for _, _, _, raw in tensors:
        out += bytes(raw) + b"\0" * ((-len(raw)) % alignment)
    open(path, "wb").write(bytes(out))
