"""Minimal GGUF v3 writer for the tests, written from the container layout
(magic, version, counts, key/value pairs, tensor directory, aligned data blob)."""
import struct

import numpy as np

U8, I8, U16, I16, U32, I32, F32, BOOL, STR, ARR, U64, I64, F64 = range(13)
_FMT = {U8: "<B", I8: "<b", U16: "<H", I16: "<h", U32: "<I", I32: "<i", F32: "<f", BOOL: "<?", U64: "<Q", I64: "<q", F64: "<d"}


def _s(x):
    b = x.encode()
    return struct.pack("<Q", len(b)) + b


def _val(t, v):
    if t == STR:
        return _s(v)
    if t == ARR:
        inner, items = v
        return struct.pack("<IQ", inner, len(items)) + b"".join(_val(inner, i) for i in items)
    return struct.pack(_FMT[t], v)


def write_gguf(path, kvs, tensors, alignment=32, version=3):
    """kvs: [(key, type, value)] (arrays: value = (inner_type, items)); tensors: [(name, ggml_type, shape, bytes)],
    shape[0] = contiguous dimension.  Returns {name: offset_in_data}."""
    head = struct.pack("<IIQQ", 0x46554747, version, len(tensors), len(kvs))
    body = b"".join(_s(k) + struct.pack("<I", t) + _val(t, v) for k, t, v in kvs)
    offs, off, directory = {}, 0, b""
    tensors = [(n, g, sh, np.ascontiguousarray(d).view(np.uint8).tobytes()) for n, g, sh, d in tensors]
    for name, gtype, shape, data in tensors:
        offs[name] = off
        directory += _s(name) + struct.pack("<I", len(shape)) + b"".join(struct.pack("<Q", d) for d in shape) + struct.pack("<IQ", gtype, off)
        off += (len(data) + alignment - 1) // alignment * alignment
    meta = head + body + directory
    pad = (-len(meta)) % alignment
    with open(path, "wb") as f:
        f.write(meta + b"\0" * pad)
        for name, _, _, data in tensors:
            f.write(data + b"\0" * ((-len(data)) % alignment))
    return offs
