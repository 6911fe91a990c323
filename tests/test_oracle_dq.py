"""Pins the CPU oracle's dequantisers (oracle/qw_oracle.c) without the GPU: known answers, the codebook checksum,
closed forms, agreement of the two formulations the reference carries, and the reference's own Q8_0 code."""
import struct
import zlib

import os

import numpy as np
import pytest


def iq3s_block(d=1.0, qs=0, qh=0, signs=0, scales=0):
    b = np.zeros(110, np.uint8)
    b[0:2] = np.frombuffer(np.float16(d).tobytes(), np.uint8) if not isinstance(d, int) else np.frombuffer(struct.pack("<H", d), np.uint8)
    b[2:66] = qs
    b[66:74] = qh
    b[74:106] = signs
    b[106:110] = scales
    return b


def test_half_conversions_match_numpy(oracle):
    L = oracle.load()
    bits = np.arange(65536, dtype=np.uint16)
    ref = bits.view(np.float16).astype(np.float32)
    got = np.array([L.qwo_h2f(int(b)) for b in bits], np.float32)
    ok = np.isnan(ref) | (got.view(np.uint32) == ref.view(np.uint32))
    assert ok.all()
    rng = np.random.default_rng(0)
    f = np.concatenate([rng.normal(0, 1, 20000), rng.normal(0, 1e-5, 20000), rng.normal(0, 3e4, 5000),
                        np.array([0.0, -0.0, 65504.0, 65519.9, 65520.0, 1e9, 5.96e-8, 2.98e-8, 2.9803e-8, 6.1e-5, 6.0975e-5])]).astype(np.float32)
    # every half-way point between adjacent binary16 values (ties must go to even)
    h = np.arange(0, 0x7bff, dtype=np.uint16).view(np.float16).astype(np.float64)
    mid = ((h[:-1] + h[1:]) / 2).astype(np.float32)
    f = np.concatenate([f, mid, -mid])
    with np.errstate(over="ignore"):
        want = f.astype(np.float16).view(np.uint16)
    got = np.array([L.qwo_f2h(float(v)) for v in f], np.uint16)
    assert (got == want).all()


def test_codebook_checksum_and_range(oracle):
    t = oracle.iq3s_table()
    assert zlib.crc32(t.astype("<u4").tobytes()) == 0xF576E4F3  # CRC of the table the reference carries
    by = t.view(np.uint8)
    assert set(np.unique(by)) == {1, 3, 5, 7, 9, 11, 13, 15}
    assert t[0] == 0x01010101 and t[256] == 0x05090507
    assert len(np.unique(t)) == 512


def test_iq3s_known_answers(oracle):
    dq = lambda b: oracle.dq_rows(21, b.reshape(1, 110), 256)[0]
    assert (dq(iq3s_block()) == 1.0).all()                       # entry 0 = (1,1,1,1), scale 1, d 1
    assert (dq(iq3s_block(signs=0xFF)) == -1.0).all()            # all sign bits set
    assert (dq(iq3s_block(scales=0xFF)) == 31.0).all()           # 1 + 2 * 15
    y = dq(iq3s_block(scales=0x21))                              # low nibble = even sub-block, high nibble = odd one
    assert (y.reshape(8, 32)[0::2] == 3.0).all() and (y.reshape(8, 32)[1::2] == 5.0).all()
    y = dq(iq3s_block(qh=0xFF))                                  # every lookup gets bit 8: entry 256 = bytes (7,5,9,5)
    assert (y.reshape(64, 4) == np.array([7, 5, 9, 5], np.float32)).all()
    y = dq(iq3s_block(qh=0x01)).reshape(8, 32)                   # only the first lookup of each sub-block
    assert (y[:, :4] == np.array([7, 5, 9, 5], np.float32)).all() and (y[:, 4:] == 1.0).all()
    y = dq(iq3s_block(qh=0x02)).reshape(8, 32)                   # bit 1 -> second lookup (values 4..7)
    assert (y[:, 4:8] == np.array([7, 5, 9, 5], np.float32)).all() and (y[:, :4] == 1.0).all() and (y[:, 8:] == 1.0).all()
    y = dq(iq3s_block(qh=0x80)).reshape(8, 32)                   # bit 7 -> lookup 7 (values 28..31)
    assert (y[:, 28:] == np.array([7, 5, 9, 5], np.float32)).all() and (y[:, :28] == 1.0).all()
    y = dq(iq3s_block(signs=0x01)).reshape(8, 4, 8)              # bit j of a sign byte -> value j of its group of 8
    assert (y[:, :, 0] == -1.0).all() and (y[:, :, 1:] == 1.0).all()
    y = dq(iq3s_block(signs=0x90)).reshape(8, 4, 8)
    assert (y[:, :, [4, 7]] == -1.0).all() and (y[:, :, [0, 1, 2, 3, 5, 6]] == 1.0).all()
    qs = np.zeros(64, np.uint8); qs[5] = 3                       # one codebook index -> entry 3 = 0x0101010b at values 20..23
    y = dq(iq3s_block(qs=qs))
    assert (y[20:24] == np.array([11, 1, 1, 1], np.float32)).all() and y.sum() == 256 + 10
    assert (dq(iq3s_block(d=1)) == np.float32(2.0 ** -24)).all()                 # smallest subnormal scale
    assert (dq(iq3s_block(d=0x7BFF, scales=0xFF, qh=0xFF))[2] == np.float32(65504.0 * 31 * 9)).all()  # largest finite scale


def test_iq3s_closed_form_and_two_formulations(oracle):
    rng = np.random.default_rng(7)
    raw = rng.integers(0, 256, (64, 8 * 110), dtype=np.uint8)
    blk = raw.reshape(-1, 110)
    blk[:, :2] = np.abs(rng.normal(0, 0.02, len(blk))).astype(np.float16).view(np.uint8).reshape(-1, 2)
    y = oracle.dq_rows(21, raw, 2048)
    assert np.array_equal(y, oracle.dq_rows(21, raw, 2048, tab=True))        # per-32 decoder == 16-value table decoder
    # independent numpy restatement of the block layout: value = sign * d * (2 s + 1) * magnitude
    t = oracle.iq3s_table().view(np.uint8).reshape(512, 4).astype(np.float32)
    d = blk[:, :2].copy().view(np.float16).astype(np.float32)                 # [n, 1]
    qs = blk[:, 2:66].astype(np.int32).reshape(-1, 8, 8)                      # [n, ib, 8 lookups]
    qh = blk[:, 66:74].astype(np.int32)
    hi = ((qh[:, :, None] >> np.arange(8)) & 1) << 8
    mag = t[qs | hi]                                                          # [n, ib, 8, 4]
    sg = blk[:, 74:106].reshape(-1, 8, 4)
    sbits = ((sg[..., None] >> np.arange(8)) & 1).reshape(-1, 8, 8, 4)        # sign byte l covers lookups 2l, 2l+1
    sc = blk[:, 106:110]
    s = np.stack([sc & 15, sc >> 4], -1).reshape(-1, 8).astype(np.float32)
    want = (d[:, :, None, None] * (2 * s + 1)[:, :, None, None]) * mag * np.where(sbits == 1, -1.0, 1.0)
    assert np.array_equal(y.reshape(-1, 8, 8, 4), want.astype(np.float32))
    # every value is +-d * odd(<=31) * odd(<=15): exact in float
    q = np.abs(y.reshape(-1, 256)) / d
    ok = d[:, 0] > 0
    assert np.all(q[ok] == np.round(q[ok])) and q[ok].max() <= 31 * 15


def test_presigned_table(oracle):
    tab = oracle.tab_iq3ss().astype(np.float32)
    t = oracle.iq3s_table().view(np.uint8).reshape(512, 4).astype(np.float32)
    i = np.arange(8192)
    sign = np.where((i[:, None] >> (9 + np.arange(4))) & 1, -1.0, 1.0)
    assert np.array_equal(tab, t[i & 511] * sign)


def test_q8_0_known_answer_closed_form_and_reference(oracle):
    b = np.zeros(34, np.uint8)
    b[:2] = np.frombuffer(np.float16(1.0).tobytes(), np.uint8)
    b[2:] = np.arange(32)
    assert np.array_equal(oracle.dq_rows(8, b.reshape(1, 34), 32)[0], np.arange(32, dtype=np.float32))
    rng = np.random.default_rng(3)
    raw = rng.integers(0, 256, (32, 64 * 34), dtype=np.uint8)
    blk = raw.reshape(-1, 34)
    blk[:, :2] = np.abs(rng.normal(0, 0.01, len(blk))).astype(np.float16).view(np.uint8).reshape(-1, 2)
    y = oracle.dq_rows(8, raw, 2048)
    want = blk[:, 2:].view(np.int8).astype(np.float32) * blk[:, :2].copy().view(np.float16).astype(np.float32)
    assert np.array_equal(y.reshape(-1, 32), want)
    assert np.array_equal(y, oracle.dq_rows(8, raw, 2048, tab=True))
    ref = oracle.ref_dq_rows(8, raw, 2048)  # the reference's src/ggml_dq.c, compiled from where it lies
    if ref is None:
        pytest.skip("oracle/_ref is not built here (reference tree absent); closed form checked above")
    assert np.array_equal(y, ref)


@pytest.mark.parametrize("ftype", [12, 13, 14, 20, 23, 1, 30, 0])
def test_other_formats_against_the_reference(oracle, ftype):
    """Random bytes in every field but the binary16 scales (finite): the per-position formulation of the oracle
    against the reference's block walkers (src/ggml_dq.c:39-143), bit for bit."""
    import sys
    sys.path.insert(0, os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden"))
    import gen
    K = 2048
    if ftype == 0:
        raw = np.random.default_rng(5).normal(0, 1, (9, K)).astype(np.float32).view(np.uint8).reshape(9, -1)
    else:
        raw = gen.blocks_fmt(900 + ftype, ftype, 9 * (K // gen.FORMATS[ftype][0])).reshape(9, -1)
    assert raw.shape[1] == oracle.row_bytes(ftype, K)
    y = oracle.dq_rows(ftype, raw, K)
    ref = oracle.ref_dq_rows(ftype, raw, K)
    if ref is None:
        pytest.skip("oracle/_ref is not built here (reference tree absent); the committed fixture covers this format")
    assert np.array_equal(y.view(np.uint32), ref.view(np.uint32))


def test_unsupported_type_is_rejected(oracle):
    with pytest.raises(ValueError):
        oracle.dq_rows(10, np.zeros((1, 84), np.uint8), 256)
    import os
    if os.path.exists(os.path.join(os.path.dirname(oracle.__file__), "_ref", "libggml_dq_ref.so")):
        assert oracle.ref_dq_rows(21, np.zeros((1, 110), np.uint8), 256) is None  # the reference has no IQ3_S on the CPU
