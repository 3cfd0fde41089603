"""Writes GGUF version 3 files for the loader's tests: the layout of llama.cpp's gguf.h (header, metadata
key-values, tensor infos, aligned tensor data), little-endian."""
import struct

import numpy as np

U8, I8, U16, I16, U32, I32, F32, BOOL, STRING, ARRAY, U64, I64, F64 = range(13)
GGML_F32, GGML_F16, GGML_Q8_0, GGML_Q4_K, GGML_Q5_K, GGML_Q6_K, GGML_IQ4_NL, GGML_IQ4_XS, GGML_BF16 = 0, 1, 8, 12, 13, 14, 20, 23, 30
GGML_Q4_0, GGML_Q5_0, GGML_Q3_K = 2, 6, 11


def _string(text):
    raw = text.encode()
    return struct.pack("<Q", len(raw)) + raw


def _value(kind, value):
    if kind == STRING:
        return _string(value)
    if kind == ARRAY:
        inner, items = value
        return struct.pack("<IQ", inner, len(items)) + b"".join(_value(inner, v) for v in items)
    return struct.pack("<" + "BbHhIifBxxQqd"[kind] if kind not in (8, 9) else "", value)


def write_gguf(path, metadata, tensors, alignment=32, version=3, magic=b"GGUF"):
    """metadata: [(key, kind, value)]; tensors: [(name, ggml type, dims (fastest first), bytes array)]."""
    out = bytearray(magic + struct.pack("<IQQ", version, len(tensors), len(metadata)))
    for key, kind, value in metadata:
        out += _string(key) + struct.pack("<I", kind) + _value(kind, value)
    offset, offsets = 0, []
    for _, _, _, data in tensors:
        offsets.append(offset)
        offset += (np.asarray(data).nbytes + alignment - 1) // alignment * alignment
    for (name, kind, dims, _), at in zip(tensors, offsets):
        out += _string(name) + struct.pack("<I", len(dims)) + b"".join(struct.pack("<Q", d) for d in dims) + struct.pack("<IQ", kind, at)
    out += b"\0" * ((-len(out)) % alignment)
    for _, _, _, data in tensors:
        raw = np.ascontiguousarray(data).tobytes()
        out += raw + b"\0" * ((-len(raw)) % alignment)
    with open(path, "wb") as f:
        f.write(out)
    return len(out)
