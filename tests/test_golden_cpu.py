"""The CPU oracle against the committed golden fixtures of tests/golden/ (made by tests/golden/make_golden.py;
hand known-answer blocks, a numpy restatement of the IQ3_S decode, the reference's own Q8_0 C code)."""
import os
import sys
import zlib

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.join(HERE, "golden"))
import gen  # noqa: E402


def load(name):
    return np.load(os.path.join(HERE, "golden", name), allow_pickle=False)


def test_generator_is_stable():
    """The inputs that are rebuilt rather than stored: a checksum guards the generator itself."""
    assert zlib.crc32(gen.raw_bytes(7, 1000).tobytes()) == 0xEDA4C8AB
    a = gen.blocks(101, 21, 48)
    assert a.shape == (48, 110) and np.array_equal(a, load("dq_iq3s.npz")["raw"][-48:])
    b = gen.blocks(102, 8, 96)
    assert np.array_equal(b[2:], load("dq_q8_0.npz")["raw"][2:])
    assert np.isfinite(gen.halves(1, 4096, 2.0).astype(np.float32)).all()


def test_iq3s_fixture(oracle):
    g = load("dq_iq3s.npz")
    raw, exp, nh = g["raw"], g["expect"], int(g["n_hand"])
    assert np.array_equal(exp[0], np.ones(256, np.float32)) and np.array_equal(exp[1], -np.ones(256, np.float32))  # the hand cases are in the file
    assert np.array_equal(exp[3, :4], np.array([7, 5, 9, 5], np.float32)) and nh == 9
    for tab in (False, True):
        assert np.array_equal(oracle.dq_rows(21, raw, 256, tab=tab).view(np.uint32), exp.view(np.uint32))
    # rows of several blocks decode block by block
    assert np.array_equal(oracle.dq_rows(21, raw[:56].reshape(7, 880), 2048).reshape(56, 256).view(np.uint32), exp[:56].view(np.uint32))


def test_q8_0_fixture(oracle):
    g = load("dq_q8_0.npz")
    assert np.array_equal(g["expect"][0], np.arange(32, dtype=np.float32))
    assert np.array_equal(oracle.dq_rows(8, g["raw"], 32).view(np.uint32), g["expect"].view(np.uint32))


def test_formats_fixture(oracle):
    """Q4_K, Q5_K, Q6_K, IQ4_NL, IQ4_XS, binary16, bfloat16: the oracle against the values the reference's own
    src/ggml_dq.c gave for hashed blocks, and against the hand blocks."""
    g = load("dq_formats.npz")
    seen = set()
    for key in g.files:
        if key.startswith("expect_f"):
            ft, K = int(key.split("_")[1][1:]), int(key.split("_")[2][1:])
            qb = gen.FORMATS[ft][0]
            raw = gen.blocks_fmt(500 + ft, ft, 6 * (K // qb)).reshape(6, -1)
            got = oracle.dq_rows(ft, raw, K)
            assert np.array_equal(got.view(np.uint32), g[key].view(np.uint32)), ft
            assert np.isfinite(got).all() and np.abs(got).max() > 0
            seen.add(ft)
        elif key.startswith("hand_raw_f"):
            ft = int(key[len("hand_raw_f"):])
            exp = g["hand_expect_f%d" % ft]
            assert np.array_equal(oracle.dq_rows(ft, g[key], exp.shape[1]).view(np.uint32), exp.view(np.uint32)), ft
    assert seen == {12, 13, 14, 20, 23, 1, 30}
    assert g["hand_expect_f14"][0, 0] == 1.0 and g["hand_expect_f14"][0, 255] == 16.0  # the hand cases are in the file
    assert g["hand_expect_f20"][0, 0] == -127.0 and g["hand_expect_f12"][0, 5] == 7.0


def qmv_cases():
    g = load("qmv.npz")
    for key in g.files:
        _, f, k, n, s = key.split("_")
        ft, K, N, seed = int(f[1:]), int(k[1:]), int(n[1:]), int(s[1:])
        qb = 256 if ft == 21 else 32
        W = gen.blocks(seed, ft, N * (K // qb)).reshape(-1)
        x = gen.halves(seed + 50, 5 * K, 2.0).reshape(5, K)
        yield ft, K, N, W, x, g[key]


def test_qmv_fixture(oracle):
    n = 0
    for ft, K, N, W, x, y in qmv_cases():
        assert np.array_equal(oracle.qmv(ft, W, N, K, x, f64=True), y)
        assert np.abs(oracle.qmv(ft, W, N, K, x) - y).max() <= 2e-3 * np.abs(y).max()
        # and against a dot product over the dequantized rows written here
        rb = oracle.row_bytes(ft, K)
        Wf = oracle.dq_rows(ft, W.reshape(N, rb), K).astype(np.float64)
        assert np.allclose(x.astype(np.float64) @ Wf.T, y, rtol=1e-12, atol=1e-12 * np.abs(y).max())
        n += 1
    assert n == 4


def test_select_fixture(oracle):
    g = load("select.npz")
    lg, K = g["logits"], int(g["topk"])
    ids = oracle.topk_ids(lg, K)
    assert np.array_equal(ids, g["ids"])
    assert np.array_equal(ids, np.argsort(-lg[:, :-1], axis=1, kind="stable")[:, :K])  # the reference's comparator (tools/moe_ref.py:75)
    sel = oracle.select(lg, K, 8)
    assert np.array_equal(sel.raw, g["record"])


def moe_cases():
    g = load("moe.npz")
    for tag in ("a", "b"):
        D, I, E, K, nb, f, seed = (int(v) for v in g[tag + "_shape"])
        m = gen.moe_layer(seed, D, I, E, f, f, f)
        m["topk"] = K
        x = gen.halves(seed + 20, nb * D, 1.5).reshape(nb, D)
        yield tag, m, x, nb, g[tag + "_logits"], g[tag + "_ids"], g[tag + "_out"]


def test_moe_fixture(oracle):
    for tag, m, x, nb, lg, ids, out in moe_cases():
        got = oracle.router(m["Wr"], m["wsg"], x)
        assert np.array_equal(got, lg)
        assert np.array_equal(oracle.topk_ids(got, m["topk"]), ids)
        assert np.array_equal(oracle.moe_layer_f64(m, lg, x), out)
        o32, _, _ = oracle.moe_layer_f32(m, lg, x, 8 if nb <= 8 else 16)
        assert np.abs(o32 - out).max() <= 2e-3 * np.abs(out).max()
