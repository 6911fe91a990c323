"""TEST INFRASTRUCTURE — a GGUF reader in plain Python that restates the reference's parser (src/gguf.c:73-173:
header, metadata skipped except general.alignment, tensor table, data start rounded up to the alignment), to check
the C reader of the library against. Layout as published with ggml (GGUF v2/v3, little endian):

    "GGUF" | u32 version | u64 n_tensors | u64 n_kv
    n_kv x  ( string key | u32 value type | value )
    n_tensors x ( string name | u32 n_dims | u64 dims[n_dims] | u32 ggml type | u64 offset from the data start )
    padding to a multiple of the alignment (general.alignment, default 32), then the tensor data

string = u64 length + bytes. Value types: 0 u8, 1 i8, 2 u16, 3 i16, 4 u32, 5 i32, 6 f32, 7 bool, 8 string,
9 array (u32 element type, u64 count, elements), 10 u64, 11 i64, 12 f64.

Only tests import this module; the product library never does.
"""
import struct

import numpy as np

# ggml type -> (values per block, bytes per block): src/gguf.c:15-25
BLOCKS = {0: (1, 4), 1: (1, 2), 30: (1, 2), 2: (32, 18), 3: (32, 20), 6: (32, 22), 7: (32, 24), 8: (32, 34), 10: (256, 84),
          11: (256, 110), 12: (256, 144), 13: (256, 176), 14: (256, 210), 16: (256, 66), 17: (256, 74), 18: (256, 98),
          19: (256, 50), 20: (32, 18), 21: (256, 110), 22: (256, 82), 23: (256, 136), 29: (256, 56), 42: (64, 18)}


def tensor_bytes(ftype, dims):
    qb, bb = BLOCKS[ftype]
    rows = 1
    for d in dims[1:]:
        rows *= d
    return rows * (dims[0] // qb) * bb


class _Cur:
    def __init__(self, b):
        self.b, self.o = b, 0

    def take(self, n):
        if self.o + n > len(self.b):
            raise ValueError("truncated")
        v = self.b[self.o:self.o + n]
        self.o += n
        return v

    def u32(self):
        return struct.unpack("<I", self.take(4))[0]

    def u64(self):
        return struct.unpack("<Q", self.take(8))[0]

    def string(self):
        n = self.u64()
        if n > 1 << 24:  # src/gguf.c:77
            raise ValueError("string too long")
        return self.take(n).decode()


def read_gguf(path):
    """{'version', 'alignment', 'data_start', 'tensors': [{'name', 'type', 'dims', 'offset' (absolute), 'nbytes'}]}.
    Raises ValueError where the reference's parser returns false."""
    b = open(path, "rb").read()
    c = _Cur(b)
    if c.take(4) != b"GGUF":
        raise ValueError("not GGUF")
    ver, nt, nkv = c.u32(), c.u64(), c.u64()
    if ver < 2:
        raise ValueError("version")
    align = 32
    size = {0: 1, 1: 1, 2: 2, 3: 2, 4: 4, 5: 4, 6: 4, 7: 1, 10: 8, 11: 8, 12: 8}

    def skip(t, key):
        nonlocal align
        if t == 8:
            c.string()
        elif t == 9:
            at, n = c.u32(), c.u64()
            if at == 8:
                for _ in range(n):
                    c.string()
            elif at in size:
                c.take(n * size[at])
            else:
                raise ValueError("array element type")
        elif t in size:
            raw = c.take(size[t])
            if key == "general.alignment":
                align = int.from_bytes(raw, "little") & 0xffffffff
        else:
            raise ValueError("value type")

    for _ in range(nkv):
        k = c.string()
        skip(c.u32(), k)
    tensors = []
    for _ in range(nt):
        name = c.string()
        nd = c.u32()
        if nd > 4:
            raise ValueError("dimensions")
        dims = [c.u64() for _ in range(nd)]
        ftype, off = c.u32(), c.u64()
        tensors.append(dict(name=name, type=ftype, dims=dims, offset=off))
    data0 = (c.o + align - 1) // align * align
    for t in tensors:
        t["offset"] += data0
        t["nbytes"] = tensor_bytes(t["type"], t["dims"]) if t["type"] in BLOCKS else 0
    return dict(version=ver, alignment=align, data_start=data0, tensors=tensors, size=len(b))
