"""Writer of synthetic GGUF files (v2 / v3, little endian), for tests and the benchmark's load measurement:

    "GGUF" | u32 version | u64 n_tensors | u64 n_kv
    n_kv x  ( string key | u32 value type | value )
    n_tensors x ( string name | u32 n_dims | u64 dims[n_dims] | u32 ggml type | u64 offset from the data start )
    padding to a multiple of the alignment (general.alignment, default 32), then the tensor data

string = u64 length + bytes. Value types: 0 u8, 1 i8, 2 u16, 3 i16, 4 u32, 5 i32, 6 f32, 7 bool, 8 string,
9 array (u32 element type, u64 count, elements), 10 u64, 11 i64, 12 f64.
"""
import struct

import numpy as np

# ggml type -> (values per block, bytes per block)
BLOCKS = {0: (1, 4), 1: (1, 2), 30: (1, 2), 2: (32, 18), 3: (32, 20), 6: (32, 22), 7: (32, 24), 8: (32, 34), 10: (256, 84),
          11: (256, 110), 12: (256, 144), 13: (256, 176), 14: (256, 210), 16: (256, 66), 17: (256, 74), 18: (256, 98),
          19: (256, 50), 20: (32, 18), 21: (256, 110), 22: (256, 82), 23: (256, 136), 29: (256, 56), 42: (64, 18)}
_SCALAR = {0: "<B", 1: "<b", 2: "<H", 3: "<h", 4: "<I", 5: "<i", 6: "<f", 7: "<B", 10: "<Q", 11: "<q", 12: "<d"}


def _s(text):
    b = text.encode() if isinstance(text, str) else bytes(text)
    return struct.pack("<Q", len(b)) + b


def _value(vtype, v):
    if vtype == 8:
        return _s(v)
    if vtype == 9:
        etype, items = v
        return struct.pack("<IQ", etype, len(items)) + b"".join(_value(etype, i) for i in items)
    return struct.pack(_SCALAR[vtype], v)


def tensor_bytes(ftype, dims):
    qb, bb = BLOCKS[ftype]
    rows = 1
    for d in dims[1:]:
        rows *= d
    return rows * (dims[0] // qb) * bb


def write_gguf(path, tensors, meta=(), alignment=None, version=3):
    """tensors: list of (name, ggml type, dims innermost first, uint8 array of the tensor's bytes).
    meta: list of (key, value type, value); arrays as (9, (element type, [items])).
    alignment: written as general.alignment (u32) when given; tensor offsets are multiples of it (32 when absent).
    Returns {name: absolute file offset}."""
    meta = list(meta)
    if alignment is not None:
        meta.append(("general.alignment", 4, alignment))
    al = alignment or 32
    head = b"GGUF" + struct.pack("<IQQ", version, len(tensors), len(meta))
    for k, t, v in meta:
        head += _s(k) + struct.pack("<I", t) + _value(t, v)
    offs, o = [], 0
    for name, ftype, dims, data in tensors:
        data = np.ascontiguousarray(data).view(np.uint8).ravel()
        assert data.size == tensor_bytes(ftype, dims), (name, data.size, tensor_bytes(ftype, dims))
        offs.append(o)
        o = (o + data.size + al - 1) // al * al
    for (name, ftype, dims, _), off in zip(tensors, offs):
        head += _s(name) + struct.pack("<I", len(dims)) + b"".join(struct.pack("<Q", d) for d in dims) + struct.pack("<IQ", ftype, off)
    data0 = (len(head) + al - 1) // al * al
    where = {}
    with open(path, "wb") as f:
        f.write(head)
        f.write(b"\0" * (data0 - len(head)))
        pos = 0
        for (name, _, _, data), off in zip(tensors, offs):
            f.write(b"\0" * (off - pos))
            raw = np.ascontiguousarray(data).view(np.uint8).ravel()
            f.write(raw.tobytes())
            pos = off + raw.size
            where[name] = data0 + off
    return where


