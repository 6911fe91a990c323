"""Pins the oracle's matvec, router, selection, MoE layer and packing with independent numpy restatements,
closed forms and invariants (no GPU)."""
import numpy as np
import pytest

from qwental_amd import synth


@pytest.mark.parametrize("ftype", [21, 8])
def test_qmv_against_numpy_float64(oracle, ftype):
    N, K, nb = 96, 512, 5
    rng = np.random.default_rng(1)
    W = synth.matrix(rng, ftype, N, K)
    x = synth.activations(rng, nb, K)
    Wf = oracle.dq_rows(ftype, W.reshape(N, -1), K).astype(np.float64)
    want = x.astype(np.float64) @ Wf.T                      # the method of tools/ggmtest.py:44
    y64 = oracle.qmv(ftype, W, N, K, x, f64=True)
    assert np.allclose(y64, want, rtol=1e-12, atol=1e-12)
    y32 = oracle.qmv(ftype, W, N, K, x)
    assert np.abs(y32 - want).max() / np.abs(want).max() < 1e-5
    # linearity in x and independence of rows from the batch they are computed in
    y1 = oracle.qmv(ftype, W, N, K, x[2:3], f64=True)
    assert np.array_equal(y1[0], y64[2])
    assert np.array_equal(oracle.qmv(ftype, W, N, K, x, threads=1), y32)


def test_router_against_numpy(oracle):
    rng = np.random.default_rng(2)
    Wr, wsg = synth.router(rng, 32, 256)
    x = synth.activations(rng, 3, 256)
    lg = oracle.router(Wr, wsg, x)
    want = np.concatenate([x.astype(np.float64) @ Wr.astype(np.float64).T, (x.astype(np.float64) @ wsg.astype(np.float64))[:, None]], 1)
    assert np.array_equal(lg, want.astype(np.float32))
    # bfloat16 weights: the same bit patterns read as bfloat16
    lgb = oracle.router(Wr, wsg, x, wfmt=30)
    wb = (Wr.view(np.uint16).astype(np.uint32) << 16).view(np.float32).astype(np.float64)
    sb = (wsg.view(np.uint16).astype(np.uint32) << 16).view(np.float32).astype(np.float64)
    with np.errstate(over="ignore", invalid="ignore"):
        wantb = np.concatenate([x.astype(np.float64) @ wb.T, (x.astype(np.float64) @ sb)[:, None]], 1).astype(np.float32)
    assert np.array_equal(lgb, wantb, equal_nan=True)


def _numpy_select(logits, K, gnb):
    nb, E1 = logits.shape
    E = E1 - 1
    ids = np.argsort(-logits[:, :E].astype(np.float64), axis=1, kind="stable")[:, :K]   # tools/moe_ref.py:75
    ue, mask, slot = [], [], []
    for p, e in enumerate(ids.ravel()):
        if e not in ue:
            ue.append(e); mask.append(0); slot.append([0] * gnb)
        u = ue.index(e)
        mask[u] |= 1 << (p // K)
        slot[u][p // K] = p % K
    pk = np.take_along_axis(logits[:, :E], ids, 1).astype(np.float64)
    w = np.exp(pk - pk[:, :1]); w /= w.sum(1, keepdims=True)
    sh = 1 / (1 + np.exp(-logits[:, E].astype(np.float64)))
    return ids, ue, mask, slot, np.concatenate([w, sh[:, None]], 1)


@pytest.mark.parametrize("nb,gnb", [(1, 8), (8, 8), (5, 16), (16, 16)])
def test_select_against_numpy(oracle, nb, gnb):
    E, K = 512, 10
    rng = np.random.default_rng(nb)
    logits = np.round(rng.normal(0, 1, (nb, E + 1)) * 8).astype(np.float32) / 8     # many exact ties
    if nb > 3:
        logits[3] = logits[0]
    s = oracle.select(logits, K, gnb)
    ids, ue, mask, slot, w = _numpy_select(logits, K, gnb)
    assert np.array_equal(oracle.topk_ids(logits, K), ids)
    assert s.U == len(ue) == len(set(ids.ravel()))
    assert list(s.ue[:s.U]) == ue and list(s.mask[:s.U]) == mask
    assert np.array_equal(s.slot[:s.U], np.array(slot, np.uint8))
    assert not s.ue[s.U:].any() and not s.mask[s.U:].any() and not s.slot[s.U:].any()
    assert np.allclose(s.w[:nb], w, rtol=1e-6)
    assert sum(bin(int(v)).count("1") for v in s.mask) == nb * K
    assert len(s.raw) == 4 + 8 * gnb * K + gnb * K * gnb + 4 * gnb * (K + 1)
    if gnb == 8:
        assert len(s.raw) == 1636   # sizeof(gg_sel), kernels/moe_gg.metal:110-116


def test_select_one_ulp_gap(oracle):
    E, K = 64, 10
    l = np.zeros((1, E + 1), np.float32)
    l[0, 20:31] = 1.0
    l[0, 30] = np.nextafter(np.float32(1), np.float32(2))
    assert list(oracle.topk_ids(l, K)[0]) == [30] + list(range(20, 29))


def _numpy_layer(m, logits, x, oracle):
    D, I, E, K = m["D"], m["I"], m["E"], m["topk"]
    dq = lambda W, f, rows, cols: oracle.dq_rows(f, np.asarray(W).reshape(rows, -1), cols).astype(np.float64)
    ids, _, _, _, w = _numpy_select(logits, K, 16)
    silu = lambda v: v / (1 + np.exp(-v))
    xs = x.astype(np.float64)
    SG, SU, SD = dq(m["Wsg"], m["fsg"], I, D), dq(m["Wsu"], m["fsu"], I, D), dq(m["Wsd"], m["fsd"], D, I)
    rgu, rd = synth.row_bytes(m["fgu"], D), synth.row_bytes(m["fd"], I)
    out = np.zeros((len(x), D))
    for t in range(len(x)):
        for k, e in enumerate(ids[t]):
            G = dq(m["Wg"][e * I * rgu:(e + 1) * I * rgu], m["fgu"], I, D)
            U = dq(m["Wu"][e * I * rgu:(e + 1) * I * rgu], m["fgu"], I, D)
            Dn = dq(m["Wd"][e * D * rd:(e + 1) * D * rd], m["fd"], D, I)
            out[t] += w[t, k] * (Dn @ (silu(G @ xs[t]) * (U @ xs[t])))          # tools/moe_ref.py:78-81
        out[t] += w[t, K] * (SD @ (silu(SG @ xs[t]) * (SU @ xs[t])))
    return out


@pytest.mark.parametrize("fmt", [21, 8])
def test_moe_layer_against_numpy(oracle, fmt):
    D, I, E, K, nb = 256, 256, 16, 4, 5
    rng = np.random.default_rng(5)
    m = synth.moe_layer(rng, D, I, E, fgu=fmt, fd=fmt, fsh=fmt)
    m["topk"] = K
    x = synth.activations(rng, nb, D)
    x[4] = x[1]
    logits = oracle.router(m["Wr"], m["wsg"], x)
    want = _numpy_layer(m, logits, x, oracle)
    got64 = oracle.moe_layer_f64(m, logits, x)
    assert np.allclose(got64, want, rtol=1e-10, atol=1e-12)
    out32, H, sel = oracle.moe_layer_f32(m, logits, x, 8)
    assert np.abs(out32.astype(np.float64) - want).max() / np.abs(want).max() < 2e-3
    assert np.array_equal(out32[4], out32[1])
    assert sel.U == len(set(oracle.topk_ids(logits, K).ravel()))


def test_pack_invariants(oracle):
    E, K, rows, tm = 512, 10, 64, 16
    rng = np.random.default_rng(8)
    ids = synth.zipf_ids(rng, rows, E, K)
    counts, offs, pos, tiles, nt = oracle.moe_pack(ids, E, tm, 1024)
    flat = ids.ravel()
    assert np.array_equal(counts, np.bincount(flat, minlength=E))
    assert np.array_equal(offs, np.concatenate([[0], np.cumsum(counts)[:-1]]))
    assert sorted(pos) == list(range(rows * K))                          # a permutation
    assert np.all(pos >= offs[flat]) and np.all(pos < offs[flat] + counts[flat])
    order = np.argsort(flat, kind="stable")
    assert np.array_equal(pos[order], np.arange(rows * K))              # stable within each expert
    assert nt == int(np.sum((counts + tm - 1) // tm))
    t = tiles[:nt]
    assert np.all(t[:, 2] - t[:, 1] <= tm) and np.all(t[:, 2] > t[:, 1])
    assert np.array_equal(np.sort(np.concatenate([np.arange(a, b) for _, a, b, _ in t])), np.arange(rows * K))
    assert not tiles[nt:].any()
    assert np.all(offs[t[:, 0]] <= t[:, 1]) and np.all(t[:, 2] <= offs[t[:, 0]] + counts[t[:, 0]])
