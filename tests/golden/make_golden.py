#!/usr/bin/env python3
"""Writes the golden fixtures of tests/golden/ (run from the repository root: python tests/golden/make_golden.py).

The reference stores no vectors for this path (its comparators recompute from model files), so the fixtures are:
  dq_iq3s.npz   hand known-answer blocks and hashed blocks with the values a numpy restatement of
                kernels/moe_iq.metal:102-118 gives (written here, independent of the C oracle; both must agree)
  dq_q8_0.npz   hashed blocks with the values of the closed form int8 * d, checked against the reference's own
                src/ggml_dq.c (oracle/_ref) when that is built
  dq_formats.npz  hashed blocks of Q4_K, Q5_K, Q6_K, IQ4_NL, IQ4_XS, binary16 and bfloat16 rows (inputs rebuilt from
                gen.py) with the values the reference's own src/ggml_dq.c gives (oracle/_ref, built from where
                the reference lies: this file can only be remade where the reference tree is present), plus hand
                known-answer blocks per format
  qmv.npz       y = W x in float64 for small IQ3_S and Q8_0 matrices (inputs rebuilt from gen.py)
  select.npz    logits with ties and duplicates -> ids, weights and the selection record
  moe.npz       two small layers (inputs rebuilt from gen.py) -> logits, ids, float64 outputs
Inputs that gen.py can rebuild are not stored."""
import os
import sys
import zlib

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(os.path.dirname(HERE)))
sys.path.insert(0, HERE)
import gen  # noqa: E402
from oracle import oracle as o  # noqa: E402


def np_dq_iq3s(raw, grid):
    """uint8 [n, 110] -> float32 [n, 256], block layout of kernels/moe_iq.metal:102-118, vectorised over blocks."""
    n = raw.shape[0]
    d = raw[:, 0:2].copy().view(np.float16).astype(np.float32).reshape(n)
    qs, qh, sg, sc = raw[:, 2:66].astype(np.uint32), raw[:, 66:74].astype(np.uint32), raw[:, 74:106], raw[:, 106:110]
    out = np.empty((n, 256), np.float32)
    gb = grid.view(np.uint8).reshape(512, 4).astype(np.float32)
    for ib in range(8):
        s = (sc[:, ib // 2] >> (4 * (ib % 2))) & 15
        db = d * (1 + 2 * s).astype(np.float32)
        for l in range(4):
            i1 = qs[:, 8 * ib + 2 * l] | ((qh[:, ib] << (8 - 2 * l)) & 256)
            i2 = qs[:, 8 * ib + 2 * l + 1] | ((qh[:, ib] << (7 - 2 * l)) & 256)
            sb = sg[:, 4 * ib + l]
            for j in range(4):
                s1 = np.where(sb & (1 << j), -1.0, 1.0).astype(np.float32)
                s2 = np.where(sb & (1 << (j + 4)), -1.0, 1.0).astype(np.float32)
                out[:, 32 * ib + 8 * l + j] = db * gb[i1, j] * s1
                out[:, 32 * ib + 8 * l + 4 + j] = db * gb[i2, j] * s2
    return out


def kat_blocks():
    """Hand cases; expected values follow from the codebook entries 0 = (1,1,1,1) and 256 = (7,5,9,5)."""
    def blk(d=0x3C00, qs=0, qh=0, sg=0, sc=0):
        b = np.zeros(110, np.uint8)
        b[0], b[1] = d & 255, d >> 8
        b[2:66], b[66:74], b[74:106], b[106:110] = qs, qh, sg, sc
        return b
    cases = [blk(), blk(sg=0xFF), blk(sc=0xFF), blk(qh=0xFF), blk(d=0x0001), blk(d=0x7BFF, sc=0xFF), blk(d=0xBC00), blk(d=0), blk(sg=0x0F, sc=0x21)]
    exp = np.empty((len(cases), 256), np.float32)
    exp[0], exp[1], exp[2] = 1.0, -1.0, 31.0
    exp[3] = np.tile(np.array([7, 5, 9, 5], np.float32), 64)
    exp[4] = np.float32(2.0 ** -24)
    exp[5] = np.float32(65504.0 * 31.0)
    exp[6], exp[7] = -1.0, 0.0
    e8 = np.tile(np.concatenate([-np.ones(4), np.ones(4)]), 32).astype(np.float32)  # low nibble of signs flips values 0..3 of each 8
    sc8 = np.repeat(np.array([3, 5] * 4, np.float32), 32)                          # scales byte 0x21: low nibble 1 -> 3, high nibble 2 -> 5
    exp[8] = e8 * sc8
    return np.stack(cases), exp


def kat_formats():
    """One hand block per format whose values can be read off the layout (scale fields 1.0 = 0x3C00)."""
    one = [0x00, 0x3C]
    raw, exp = {}, {}
    # Q4_K: d = 1, dmin = 1; sub-block 0: scale 2, min 3 (bytes 4 and 8); others zero. qs[l] = l & 15 | 0xF0.
    b = np.zeros(144, np.uint8)
    b[0:2], b[2:4], b[4], b[8] = one, one, 2, 3
    b[16:144] = np.tile((np.arange(32) & 15) | 0xF0, 4)
    e = np.zeros(256, np.float32)
    e[:32] = 2.0 * (np.arange(32) & 15) - 3.0  # every other sub-block: 0 * q - 0
    raw[12], exp[12] = b.reshape(1, -1), e.reshape(1, -1)
    # Q5_K: as above with the fifth bit of sub-block 0 set for odd l (bit 0 of qh[l]).
    b = np.zeros(176, np.uint8)
    b[0:2], b[2:4], b[4], b[8] = one, one, 2, 3
    b[16:48] = np.arange(32) & 1
    b[48:176] = np.tile(np.arange(32) & 15, 4)
    e = np.zeros(256, np.float32)
    e[:32] = 2.0 * ((np.arange(32) & 15) + 16 * (np.arange(32) & 1)) - 3.0
    raw[13], exp[13] = b.reshape(1, -1), e.reshape(1, -1)
    # Q6_K: d = 1, scales 1..16, every six-bit value 33 (ql nibbles 1, qh pairs 2) -> q = 1: value = scale of its group.
    b = np.zeros(210, np.uint8)
    b[0:128], b[128:192], b[192:208], b[208:210] = 0x11, 0xAA, np.arange(1, 17), one
    e = np.empty(256, np.float32)
    for i in range(256):
        e[i] = 1 + 8 * (i >> 7) + 2 * ((i >> 5) & 3) + (i & 31) // 16
    raw[14], exp[14] = b.reshape(1, -1), e.reshape(1, -1)
    # IQ4_NL: d = 1, qs[j] = j | (15 - j) << 4 -> codebook in order, then reversed.
    kv = np.array([-127, -104, -83, -65, -49, -35, -22, -10, 1, 13, 25, 38, 53, 69, 89, 113], np.float32)
    b = np.zeros(18, np.uint8)
    b[0:2], b[2:18] = one, np.arange(16) | ((15 - np.arange(16)) << 4)
    raw[20], exp[20] = b.reshape(1, -1), np.concatenate([kv, kv[::-1]]).reshape(1, -1)
    # IQ4_XS: d = 1; six-bit scales 33, 34, ... 40 (low nibbles 1..8, high bits 2) -> factors 1..8; nibbles as IQ4_NL.
    b = np.zeros(136, np.uint8)
    b[0:2] = one
    b[2:4] = np.array([0xAAAA], np.uint16).view(np.uint8)
    b[4:8] = [0x21, 0x43, 0x65, 0x87]
    b[8:136] = np.tile(np.arange(16) | ((15 - np.arange(16)) << 4), 8)
    raw[23] = b.reshape(1, -1)
    exp[23] = np.concatenate([np.concatenate([kv, kv[::-1]]) * (s + 1) for s in range(8)]).astype(np.float32).reshape(1, -1)
    # bfloat16: 1.0, -2.0, 2^-126, the largest finite value
    b = np.array([0x3F80, 0xC000, 0x0080, 0x7F7F], np.uint16)
    raw[30] = b.view(np.uint8).reshape(1, -1)
    exp[30] = (b.astype(np.uint32) << 16).view(np.float32).reshape(1, -1)
    return raw, exp


def main():
    grid = o.iq3s_table()
    assert zlib.crc32(grid.astype("<u4").tobytes()) == 0xF576E4F3
    # ---- IQ3_S
    kraw, kexp = kat_blocks()
    hraw = gen.blocks(101, 21, 48)
    raw = np.concatenate([kraw, hraw])
    exp = np_dq_iq3s(raw, grid)
    assert np.array_equal(exp[:len(kraw)].view(np.uint32), kexp.view(np.uint32)), "numpy restatement disagrees with the hand values"
    for tab in (False, True):
        assert np.array_equal(o.dq_rows(21, raw, 256, tab=tab).view(np.uint32), exp.view(np.uint32)), "C oracle disagrees with the numpy restatement"
    np.savez_compressed(os.path.join(HERE, "dq_iq3s.npz"), raw=raw, expect=exp, n_hand=len(kraw))
    # ---- Q8_0
    raw8 = gen.blocks(102, 8, 96)
    raw8[0, 2:] = np.arange(32, dtype=np.uint8)
    raw8[0, :2] = np.array([0x3C00], np.uint16).view(np.uint8)  # d = 1: values 0..31
    raw8[1, 2:] = np.array([-127] * 16 + [127] * 16, np.int8).view(np.uint8)
    d8 = raw8[:, :2].copy().view(np.float16).astype(np.float32)
    exp8 = raw8[:, 2:].view(np.int8).astype(np.float32) * d8
    assert np.array_equal(exp8[0], np.arange(32, dtype=np.float32))
    assert np.array_equal(o.dq_rows(8, raw8, 32).view(np.uint32), exp8.view(np.uint32))
    try:
        ref = o.ref_dq_rows(8, raw8, 32)
        assert np.array_equal(ref.view(np.uint32), exp8.view(np.uint32)), "reference ggml_dq.c disagrees"
        print("Q8_0: checked against the reference's src/ggml_dq.c")
    except (OSError, FileNotFoundError) as e:
        print("Q8_0: oracle/_ref not built (%s)" % e)
    np.savez_compressed(os.path.join(HERE, "dq_q8_0.npz"), raw=raw8, expect=exp8)
    # ---- the other formats: expected values from the reference's compiled src/ggml_dq.c
    fm = {}
    for ft in (12, 13, 14, 20, 23, 1, 30):
        qb, bb, _ = gen.FORMATS[ft]
        K = 512 if qb > 1 else 384
        raw = gen.blocks_fmt(500 + ft, ft, 6 * (K // qb)).reshape(6, -1)
        ref = o.ref_dq_rows(ft, raw, K)
        if ref is None:
            raise SystemExit("oracle/_ref is not built: dq_formats.npz needs the reference tree (the other files were written)")
        assert np.array_equal(o.dq_rows(ft, raw, K).view(np.uint32), ref.view(np.uint32)), "oracle disagrees with the reference for type %d" % ft
        fm["expect_f%d_k%d" % (ft, K)] = ref
    kraw, kexp = kat_formats()
    for ft in kraw:
        assert np.array_equal(o.dq_rows(ft, kraw[ft], kraw[ft].shape[1] // gen.FORMATS[ft][1] * gen.FORMATS[ft][0]), kexp[ft]), "hand case, type %d" % ft
        assert np.array_equal(o.ref_dq_rows(ft, kraw[ft], kexp[ft].shape[1]), kexp[ft]), "hand case against the reference, type %d" % ft
        fm["hand_raw_f%d" % ft], fm["hand_expect_f%d" % ft] = kraw[ft], kexp[ft]
    np.savez_compressed(os.path.join(HERE, "dq_formats.npz"), **fm)
    # ---- matvec (inputs from gen.py)
    qm = {}
    for ft, K, N, seed in ((21, 512, 48, 201), (21, 2048, 19, 202), (8, 512, 48, 203), (8, 96, 7, 204)):
        qb = 256 if ft == 21 else 32
        W = gen.blocks(seed, ft, N * (K // qb)).reshape(-1)
        x = gen.halves(seed + 50, 5 * K, 2.0).reshape(5, K)
        qm["y_f%d_k%d_n%d_s%d" % (ft, K, N, seed)] = o.qmv(ft, W, N, K, x, f64=True)
    np.savez_compressed(os.path.join(HERE, "qmv.npz"), **qm)
    # ---- selection: ties, duplicates, descending runs
    E, K = 32, 4
    lg = (gen.halves(301, 8 * (E + 1), 4.0).astype(np.float32)).reshape(8, E + 1)
    lg[1] = lg[0]                      # duplicate token
    lg[2, :E] = 1.0                    # all tied -> ids 0, 1, 2, 3
    lg[3, :E] = np.float32(-3.0)
    lg[3, [31, 7, 19]] = 2.5           # three tied above a tied floor -> 7, 19, 31, 0
    lg[4, :E] = np.arange(E, dtype=np.float32)          # ascending -> 31, 30, 29, 28
    lg[5, :E] = -np.arange(E, dtype=np.float32)         # descending -> 0, 1, 2, 3
    lg[6, :E] = np.where(np.arange(E) % 2 == 0, np.float32(1.0), np.float32(np.nextafter(np.float32(1.0), np.float32(2.0))))  # 1-ulp gaps -> 1, 3, 5, 7
    ids = o.topk_ids(lg, K)
    assert ids[2].tolist() == [0, 1, 2, 3] and ids[3].tolist() == [7, 19, 31, 0] and ids[4].tolist() == [31, 30, 29, 28]
    assert ids[5].tolist() == [0, 1, 2, 3] and ids[6].tolist() == [1, 3, 5, 7]
    sel = o.select(lg, K, 8)
    assert np.allclose(sel.w[2, :K], 0.25) and sel.U == len(set(ids.ravel().tolist()))
    np.savez_compressed(os.path.join(HERE, "select.npz"), logits=lg, ids=ids, record=sel.raw, topk=K)
    # ---- two small layers
    mo = {}
    for tag, (D, I, E, K, nb, f, seed) in {"a": (512, 256, 16, 4, 5, 21, 401), "b": (256, 256, 12, 3, 12, 8, 402)}.items():
        m = gen.moe_layer(seed, D, I, E, f, f, f)
        m["topk"] = K
        x = gen.halves(seed + 20, nb * D, 1.5).reshape(nb, D)
        lgm = o.router(m["Wr"], m["wsg"], x)
        out = o.moe_layer_f64(m, lgm, x)
        assert np.isfinite(out).all() and np.abs(out).max() < 6e4
        mo.update({tag + "_shape": np.array([D, I, E, K, nb, f, seed]), tag + "_logits": lgm, tag + "_ids": o.topk_ids(lgm, K), tag + "_out": out})
    np.savez_compressed(os.path.join(HERE, "moe.npz"), **mo)
    for f in sorted(os.listdir(HERE)):
        if f.endswith(".npz"):
            print("%-14s %7d bytes" % (f, os.path.getsize(os.path.join(HERE, f))))


if __name__ == "__main__":
    main()
