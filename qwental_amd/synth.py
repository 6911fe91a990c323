"""Seeded synthetic inputs of the benchmark configurations (weights as raw GGUF blocks, activations, routing).

IQ3_S block, 110 bytes: d = binary16(|N(0, 0.02)|), qs[64] / qh[8] / signs[32] uniform random bytes, scales[4]
uniform random bytes (eight 4-bit scales). Q8_0 block, 34 bytes: d = binary16(|N(0, 0.01)|), qs uniform int8 in
[-127, 127]. Activations binary16 N(0, 1). Router weights binary16 N(0, 0.02).

One deviation, for the MoE layer only: with block scales |N(0, 0.02)| the layer's output reaches about 5e5, beyond
binary16 (65504), and the binary16 output the interface prescribes becomes +-inf. moe_layer() therefore draws the
block scales ten times smaller (MOE_D_SCALE); every byte other than the two scale bytes per block is unchanged, and
so is the work the kernels do.
"""
import numpy as np

BLOCK = {8: (32, 34), 21: (256, 110), 12: (256, 144), 13: (256, 176), 14: (256, 210), 20: (32, 18), 23: (256, 136),
         1: (1, 2), 30: (1, 2)}  # ggml type -> (values, bytes) per block
D_SIGMA = {21: 0.02, 8: 0.01}
# byte offsets of the binary16 scale fields of the other block formats and the sigma their |N(0, sigma)| is drawn with
SCALE_FIELDS = {12: ((0, 2), 0.002), 13: ((0, 2), 0.001), 14: ((208,), 0.0005), 20: ((0,), 0.0005), 23: ((0,), 0.00005)}
MOE_D_SCALE = 0.1


def row_bytes(ftype, K):
    qb, bb = BLOCK[ftype]
    assert K % qb == 0
    return K // qb * bb


def blocks(rng, ftype, n, d_scale=1.0):
    """n raw blocks of the given type as uint8 [n, block_bytes]."""
    qb, bb = BLOCK[ftype]
    if ftype in (1, 30):  # plain rows: N(0, 0.02) values as binary16 / bfloat16 (truncated)
        v = rng.normal(0.0, 0.02 * d_scale, n).astype(np.float32)
        if ftype == 1:
            return v.astype(np.float16).view(np.uint8).reshape(n, 2)
        return (v.view(np.uint32) >> 16).astype(np.uint16).view(np.uint8).reshape(n, 2)
    if ftype in SCALE_FIELDS:  # every byte uniform, then the scale fields
        out = rng.integers(0, 256, (n, bb), dtype=np.uint8)
        offs, sigma = SCALE_FIELDS[ftype]
        for off in offs:
            out[:, off:off + 2] = np.abs(rng.normal(0.0, sigma * d_scale, n)).astype(np.float16).view(np.uint8).reshape(n, 2)
        return out
    out = np.empty((n, bb), np.uint8)
    d = np.abs(rng.normal(0.0, D_SIGMA[ftype] * d_scale, n)).astype(np.float16)
    if ftype == 21:
        out[:, 2:] = rng.integers(0, 256, (n, bb - 2), dtype=np.uint8)
    else:
        out[:, 2:] = rng.integers(-127, 128, (n, 32), dtype=np.int8).view(np.uint8)
    out[:, :2] = d.view(np.uint8).reshape(n, 2)
    return out


def matrix(rng, ftype, rows, K, d_scale=1.0):
    """rows x K quantized matrix as flat uint8 [rows * row_bytes]."""
    qb, _ = BLOCK[ftype]
    return blocks(rng, ftype, rows * (K // qb), d_scale).reshape(-1)


def activations(rng, nb, K):
    return rng.normal(0.0, 1.0, (nb, K)).astype(np.float16)


def router(rng, E, D):
    """(Wr [E, D], shared gate vector [D]) as binary16."""
    return rng.normal(0.0, 0.02, (E, D)).astype(np.float16), rng.normal(0.0, 0.02, D).astype(np.float16)


def moe_layer(rng, D, I, E, fgu=21, fd=21, fsh=21, fshd=None, experts=None, d_scale=MOE_D_SCALE, fshu=None):
    """One MoE layer as a dict of numpy arrays (the field names of qwo_moe_weights / MoeLayer).
    experts: generate only this many routed experts' bytes (the others are never read when ids are < experts)."""
    ne = E if experts is None else experts
    fshd = fsh if fshd is None else fshd
    fshu = fsh if fshu is None else fshu  # the shared expert's up rows may have a format of their own
    Wr, wsg = router(rng, E, D)
    return dict(D=D, I=I, E=E, fgu=fgu, fd=fd, fsg=fsh, fsu=fshu, fsd=fshd, Wr=Wr, wsg=wsg,
                Wg=matrix(rng, fgu, ne * I, D, d_scale), Wu=matrix(rng, fgu, ne * I, D, d_scale), Wd=matrix(rng, fd, ne * D, I, d_scale),
                Wsg=matrix(rng, fsh, I, D, d_scale), Wsu=matrix(rng, fshu, I, D, d_scale), Wsd=matrix(rng, fshd, D, I, d_scale))


def expert_bytes(D, I, fgu=21, fd=21):
    return 2 * I * row_bytes(fgu, D) + D * row_bytes(fd, I)


def zipf_ids(rng, rows, E, topk, s=1.1):
    """Per row, topk distinct expert ids drawn without replacement with P(rank r) ~ 1 / (r + 1)^s over a seeded
    permutation of the experts."""
    p = 1.0 / np.arange(1, E + 1) ** s
    p /= p.sum()
    perm = rng.permutation(E)
    return np.stack([perm[rng.choice(E, topk, replace=False, p=p)] for _ in range(rows)]).astype(np.uint32)


def logits_for_ids(rng, ids, E):
    """Router logits [rows, E + 1] whose top-k (in rank order) are exactly ids: distinct descending values on the
    chosen experts, noise well below them elsewhere."""
    rows, topk = ids.shape
    lg = rng.normal(0.0, 0.1, (rows, E + 1)).astype(np.float32)
    for t in range(rows):
        lg[t, ids[t]] = 4.0 - 0.25 * np.arange(topk, dtype=np.float32)
    return lg


def to_bf16(a):
    """float -> bfloat16 bit patterns (uint16), round to nearest even."""
    u = np.ascontiguousarray(a, np.float32).view(np.uint32)
    return ((u + 0x7FFF + ((u >> 16) & 1)) >> 16).astype(np.uint16)


def hyper_weights(rng, D, hc=4, lr=320, inject=True):
    """Weights of one hyper-connection of the GGUF profile: norm weights float32 [hc * D] around 1, mix_down [lr, hc * D],
    mix_up [hc * D, lr] and (inject) [hc, hc * D] as bfloat16 bit patterns, scaled so that their products are O(1)."""
    return {"hc_norm": (1 + 0.1 * rng.standard_normal(hc * D)).astype(np.float32),
            "mix_down": to_bf16(rng.standard_normal((lr, hc * D)) / np.sqrt(hc * D) * 2),
            "mix_up": to_bf16(rng.standard_normal((hc * D, lr)) / np.sqrt(lr) * 2),
            "inject": to_bf16(rng.standard_normal((hc, hc * D)) / np.sqrt(D)) if inject else None}


def hyper_state(rng, nb, D, hc=4):
    """Streams h float32 [nb, hc, D] (a different scale per stream), a sublayer output binary16 [nb, D] and inject sums
    float32 [nb, hc, hc]."""
    h = (rng.standard_normal((nb, hc, D)) * (0.5 + np.arange(hc))[None, :, None]).astype(np.float32)
    return h, (0.5 * rng.standard_normal((nb, D))).astype(np.float16), rng.standard_normal((nb, hc, hc)).astype(np.float32)
