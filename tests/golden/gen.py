"""Counter-based input generator of the golden fixtures: every byte is a function of (seed, index) alone
(splitmix64 finaliser), so the inputs are rebuilt identically anywhere and only expected outputs are stored."""
import numpy as np

M64 = (1 << 64) - 1


def hash64(seed, n):
    """n 64-bit words: splitmix64 of seed * 2^32 + index."""
    with np.errstate(over="ignore"):
        z = (np.arange(n, dtype=np.uint64) + np.uint64((seed << 32) & M64)) * np.uint64(0x9E3779B97F4A7C15)
        z = (z ^ (z >> np.uint64(30))) * np.uint64(0xBF58476D1CE4E5B9)
        z = (z ^ (z >> np.uint64(27))) * np.uint64(0x94D049BB133111EB)
        return z ^ (z >> np.uint64(31))


def raw_bytes(seed, n):
    return hash64(seed, (n + 7) // 8).view(np.uint8)[:n].copy()


def blocks(seed, ftype, n):
    """n quantized blocks, uint8 [n, block bytes]: hashed payload bytes; the binary16 scale d has exponent field
    5..6 and hashed mantissa (d in [6.1e-5 * 2^5 ..], about 0.001 .. 0.004), always finite and positive."""
    bb = 110 if ftype == 21 else 34
    out = raw_bytes(seed, n * bb).reshape(n, bb)
    h = hash64(seed ^ 0x5bd1, n)
    d = (np.uint16(5 << 10) + (h & np.uint64(0x7FF)).astype(np.uint16)).astype(np.uint16)
    out[:, 0] = (d & 0xFF).astype(np.uint8)
    out[:, 1] = (d >> 8).astype(np.uint8)
    if ftype == 8:  # int8 -128 does not occur in Q8_0 files (quantizer clamps to +-127)
        q = out[:, 2:]
        q[q == 0x80] = 0x81
    return out


# ggml type -> (values per block, bytes per block, byte offsets of the binary16 scale fields)
FORMATS = {8: (32, 34, (0,)), 21: (256, 110, (0,)), 12: (256, 144, (0, 2)), 13: (256, 176, (0, 2)), 14: (256, 210, (208,)),
           20: (32, 18, (0,)), 23: (256, 136, (0,)), 1: (1, 2, ()), 30: (1, 2, ())}


def blocks_fmt(seed, ftype, n):
    """n blocks of any format of FORMATS, uint8 [n, block bytes]: hashed payload, every binary16 scale field finite
    and positive as in blocks(). Types 1 and 30 (plain binary16 / bfloat16 values): finite values of magnitude
    up to about 4."""
    if ftype in (8, 21):
        return blocks(seed, ftype, n)
    _, bb, scales = FORMATS[ftype]
    if ftype == 1:
        return halves(seed, n, 4.0).view(np.uint8).reshape(n, 2).copy()
    if ftype == 30:
        f = halves(seed, n, 4.0).astype(np.float32) * np.float32(1.0 + 2.0 ** -9)  # not all representable in binary16
        return (f.view(np.uint32) >> 16).astype(np.uint16).view(np.uint8).reshape(n, 2).copy()
    out = raw_bytes(seed, n * bb).reshape(n, bb)
    for k, off in enumerate(scales):
        h = hash64(seed ^ (0x5bd1 + 77 * k), n)
        d = (np.uint16(5 << 10) + (h & np.uint64(0x7FF)).astype(np.uint16)).astype(np.uint16)
        out[:, off] = (d & 0xFF).astype(np.uint8)
        out[:, off + 1] = (d >> 8).astype(np.uint8)
    return out


def halves(seed, n, scale):
    """n binary16 values, roughly uniform in (-scale, scale)."""
    h = hash64(seed, n)
    u = (h >> np.uint64(11)).astype(np.float64) / float(1 << 53)
    return ((2.0 * u - 1.0) * scale).astype(np.float16)


def moe_layer(seed, D, I, E, fgu, fd, fsh):
    qb = {21: 256, 8: 32}
    rb = lambda f, K: K // qb[f] * (110 if f == 21 else 34)
    mat = lambda s, f, rows, K: blocks(s, f, rows * (K // qb[f])).reshape(-1)
    return dict(D=D, I=I, E=E, fgu=fgu, fd=fd, fsg=fsh, fsu=fsh, fsd=fsh,
                Wr=halves(seed + 1, E * D, 0.05).reshape(E, D), wsg=halves(seed + 2, D, 0.05),
                Wg=mat(seed + 3, fgu, E * I, D), Wu=mat(seed + 4, fgu, E * I, D), Wd=mat(seed + 5, fd, E * D, I),
                Wsg=mat(seed + 6, fsh, I, D), Wsu=mat(seed + 7, fsh, I, D), Wsd=mat(seed + 8, fsh, D, I))
