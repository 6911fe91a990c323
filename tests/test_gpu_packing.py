"""Ragged batches through the packing path (count -> plan -> scatter -> grouped product -> combine): integer stages
bit-exact against the oracle, outputs against a float64 recompute."""
import os

import numpy as np
import pytest

import qwental_amd as q
from helpers import DeviceLayer, maxrel
from qwental_amd import synth

pytestmark = pytest.mark.gpu
TOL = 2e-3


def expert_ref(o, m, e, x):
    """float64 down(SiLU(gate x) * up x) of expert e for one row x (float16)."""
    D, I = m["D"], m["I"]
    rg, rd = synth.row_bytes(m["fgu"], D), synth.row_bytes(m["fd"], I)
    Wg = m["Wg"].reshape(m["E"], I * rg)[e]
    Wu = m["Wu"].reshape(m["E"], I * rg)[e]
    Wd = m["Wd"].reshape(m["E"], D * rd)[e]
    g = o.qmv(m["fgu"], Wg, I, D, x[None, :], f64=True)[0]
    u = o.qmv(m["fgu"], Wu, I, D, x[None, :], f64=True)[0]
    h = (g / (1.0 + np.exp(-g)) * u)
    return h, Wd


def run_case(gpu, oracle, T, ids, E, K, D, I, fmt, tm, seed, device_only=False, fd=None):
    rng = np.random.default_rng(seed)
    m = synth.moe_layer(rng, D, I, E, fgu=fmt, fd=fmt if fd is None else fd, fsh=fmt)
    x = synth.activations(rng, T, D)
    w = rng.uniform(0.05, 1.0, (T, K)).astype(np.float32)
    w /= w.sum(axis=1, keepdims=True)
    path = q.Path(gpu, D, I, E, K, 16)
    path.pf_reserve(T, tm)
    dl = DeviceLayer(gpu, m, device_only=device_only)
    xb, ib, wb, ob = gpu.buf_from(x), gpu.buf_from(ids.astype(np.uint32).ravel()), gpu.buf_from(w.ravel()), gpu.buf(T * D * 2)
    packed0 = gpu.L.qw_hip_packed_bytes(gpu.g)
    b = gpu.batch()
    path.pf_moe(b, dl.layer, T, xb, ib, wb, ob)
    assert b.end() >= 0, gpu.last_error()
    if device_only and fmt == 21 and fd is None:  # weights that live in HBM only get the tile-major copies: gate + up as one, down
        assert gpu.L.qw_hip_packed_bytes(gpu.g) - packed0 == (2 * E * I * (D // 256) + E * D * (I // 256)) // 16 * 1792
    P = T * K
    # integer stages against the oracle (kernels/moe_prefill.metal:15-93)
    mt = path.pf_max_tiles()
    counts, offs, pos_ref, tiles, nt = oracle.moe_pack(ids.ravel(), E, tm, mt)
    assert np.array_equal(path.pf_scratch(0, np.uint32)[:E], counts)
    assert np.array_equal(path.pf_scratch(1, np.uint32)[:E], offs)
    assert np.array_equal(path.pf_scratch(2, np.uint32)[:4 * mt].reshape(mt, 4), tiles.reshape(mt, 4))
    pos = path.pf_scratch(3, np.uint32)[:P]
    assert sorted(pos.tolist()) == list(range(P))  # a permutation of the packed rows
    flat = ids.ravel()
    assert all(offs[flat[p]] <= pos[p] < offs[flat[p]] + counts[flat[p]] for p in range(P))  # inside the pair's expert range
    Xs = path.pf_scratch(4, np.float16)[:P * D].reshape(P, D)
    assert all(np.array_equal(Xs[pos[p]].view(np.uint16), x[p // K].view(np.uint16)) for p in range(P))  # scatter copied the right rows
    # outputs: float64 recompute with the reference's binary16 roundings of H and of the down output (kernels/prefill.metal:485-499)
    out = ob.view(np.float16)[:T * D].reshape(T, D).astype(np.float64)
    ref = np.zeros((T, D))
    for t in range(T):
        for s in range(K):
            h, Wd = expert_ref(oracle, m, int(ids[t, s]), x[t])
            d = oracle.qmv(m["fd"], Wd, D, I, h.astype(np.float16)[None, :], f64=True)[0]
            ref[t] += w[t, s] * d
    assert maxrel(out, ref) <= TOL, maxrel(out, ref)
    for bb in (xb, ib, wb, ob):
        bb.free()
    dl.free()
    path.close()


@pytest.mark.parametrize("fmt,tm", [(21, 16), (21, 64), (8, 32)])
def test_packing_uniform_routing(gpu, oracle, fmt, tm):
    T, E, K, D, I = 24, 32, 4, 512, 512
    rng = np.random.default_rng(7 + tm)
    ids = np.stack([rng.choice(E, K, replace=False) for _ in range(T)])
    run_case(gpu, oracle, T, ids, E, K, D, I, fmt, tm, 70 + tm)


@pytest.mark.parametrize("dev", [False, True])
def test_packing_iq4_nl_down_rows(gpu, oracle, dev):
    """The reference model's formats on the packing path: IQ3_S gate/up, IQ4_NL down rows of 640 values."""
    T, E, K, D, I = 40, 32, 4, 512, 640
    rng = np.random.default_rng(19)
    ids = synth.zipf_ids(rng, T, E, K)
    run_case(gpu, oracle, T, ids, E, K, D, I, 21, 16, 190, device_only=dev, fd=20)


@pytest.mark.parametrize("tm", [16, 64])
def test_packing_tile_major_weights(gpu, oracle, tm):
    """The same through the tile-major copies (weights resident in HBM only): gate and up of a tile entry in one
    launch, results as with the GGUF rows."""
    if os.environ.get("QW_HIP_REPACK") == "0":
        pytest.skip("tile-major copies are switched off in this environment")
    T, E, K, D, I = 40, 32, 4, 512, 512
    rng = np.random.default_rng(17 + tm)
    ids = synth.zipf_ids(rng, T, E, K)
    run_case(gpu, oracle, T, ids, E, K, D, I, 21, tm, 170 + tm, device_only=True)


def test_packing_zipf_hot_experts(gpu, oracle):
    """Continuous-batching shape in small: 16 slots with 1..16 rows each (64 rows here), Zipf(1.1) routing: a few
    experts collect far more than one tile of rows, most none."""
    T, E, K, D, I = 64, 64, 4, 512, 256
    rng = np.random.default_rng(4)
    ids = synth.zipf_ids(rng, T, E, K)
    counts = np.bincount(ids.ravel(), minlength=E)
    assert counts.max() > 16 and (counts == 0).sum() > 0
    run_case(gpu, oracle, T, ids, E, K, D, I, 21, 16, 44)


def test_packing_all_pairs_one_expert(gpu, oracle):
    """Every token's first pick is expert 3: its rows span several tile entries; the other picks are distinct."""
    T, E, K, D, I = 40, 16, 2, 256, 256
    ids = np.stack([np.array([3, (5 + t) % E if (5 + t) % E != 3 else 4]) for t in range(T)])
    run_case(gpu, oracle, T, ids, E, K, D, I, 21, 32, 9)


def test_ragged_step_decode_groups_equal_packing_path(gpu, oracle):
    """A continuous-batching step in small (BASELINE configs[3] shape: 16 slots, n[i] ~ U{1..16} rows each, Zipf(1.1)
    routing forced through the logits): the decode path in groups of at most 16 rows and the packing path in one pass
    give the same routed sums. The shared expert's block scales are zero here, so that the decode path's output is
    the routed part alone."""
    E, K, D, I = 64, 4, 512, 512
    rng = np.random.default_rng(21)
    n = rng.integers(1, 17, 16)
    T = int(n.sum())
    m = synth.moe_layer(rng, D, I, E)
    for key in ("Wsg", "Wsu", "Wsd"):
        m[key].reshape(-1, 110)[:, :2] = 0  # d = 0: the shared expert contributes nothing
    m["topk"] = K
    x = synth.activations(rng, T, D)
    ids = synth.zipf_ids(rng, T, E, K)
    lg = synth.logits_for_ids(rng, ids, E)
    path = q.Path(gpu, D, I, E, K, 16)
    dl = DeviceLayer(gpu, m)
    out_dec = np.zeros((T, D), np.float16)
    wts = np.zeros((T, K), np.float32)
    for g0 in range(0, T, 16):
        nb = min(16, T - g0)
        xb, lb = gpu.buf_from(x[g0:g0 + nb]), gpu.buf_from(lg[g0:g0 + nb])
        sb, ob = gpu.buf(path.sel_bytes(nb)), gpu.buf(nb * D * 2)
        b = gpu.batch()
        path.gg_moe_lg(b, dl.layer, nb, xb, lb, sb, ob)
        assert b.end() >= 0, gpu.last_error()
        out_dec[g0:g0 + nb] = ob.view(np.float16)[:nb * D].reshape(nb, D)
        gnb = 8 if nb <= 8 else 16
        sel = oracle.Sel(sb.view(np.uint8).copy(), gnb, K)
        ref = oracle.select(lg[g0:g0 + nb], K, gnb)
        assert sel.U == ref.U and np.array_equal(sel.ue[:ref.U], ref.ue[:ref.U])
        assert np.array_equal(oracle.topk_ids(lg[g0:g0 + nb], K), ids[g0:g0 + nb])  # the forced routing took
        wts[g0:g0 + nb] = sel.w[:nb, :K]
        for bb in (xb, lb, sb, ob):
            bb.free()
    path.pf_reserve(T, 16)
    xb, ib, wb, ob = gpu.buf_from(x), gpu.buf_from(ids.astype(np.uint32).ravel()), gpu.buf_from(wts.ravel()), gpu.buf(T * D * 2)
    b = gpu.batch()
    path.pf_moe(b, dl.layer, T, xb, ib, wb, ob)
    assert b.end() >= 0, gpu.last_error()
    out_pk = ob.view(np.float16)[:T * D].reshape(T, D)
    counts = path.pf_scratch(0, np.uint32)[:E]
    assert counts.sum() == T * K and counts.max() > 16  # a hot expert spans several tile entries
    assert maxrel(out_pk, out_dec.astype(np.float64)) <= TOL
    for bb in (xb, ib, wb, ob):
        bb.free()
    dl.free()
    path.close()


@pytest.mark.parametrize("dev,tm,T", [(True, 16, 40), (True, 64, 40), (False, 16, 24), (True, 16, 130)])
def test_packing_fused_launches_equal_one_per_dispatch(gpu, oracle, dev, tm, T):
    """p_zero + moe_count + moe_plan_t + moe_scatter run as one launch (qwk_moe_prep), and p_act2 rides at the end of the
    gate / up launch when that one runs over the tile-major copy. Against one launch per dispatch (QW_HIP_PK_SPLIT):
    counts, offsets and tile table equal, every pair's packed x and H rows equal bit for bit, the output equal bit for
    bit; the packed order inside an expert is the order of the pairs."""
    if dev and os.environ.get("QW_HIP_REPACK") == "0":
        pytest.skip("tile-major copies are switched off in this environment")
    E, K, D, I = 32, 4, 512, 512
    rng = np.random.default_rng(300 + tm + T)
    m = synth.moe_layer(rng, D, I, E, fgu=21, fd=21, fsh=21)
    x = synth.activations(rng, T, D)
    ids = synth.zipf_ids(rng, T, E, K)
    w = rng.uniform(0.05, 1.0, (T, K)).astype(np.float32)
    dl = DeviceLayer(gpu, m, device_only=dev)
    P = T * K
    res = {}
    for split in (True, False):
        with gpu.switches(pk_split="1" if split else None):
            path = q.Path(gpu, D, I, E, K, 16)
            path.pf_reserve(T, tm)
            xb, ib, wb, ob = gpu.buf_from(x), gpu.buf_from(ids.astype(np.uint32).ravel()), gpu.buf_from(w.ravel()), gpu.buf(T * D * 2)
            gpu.profile(True)
            b = gpu.batch()
            path.pf_moe(b, dl.layer, T, xb, ib, wb, ob)
            assert b.end() >= 0, gpu.last_error()
            names = [n for n, _ in gpu.profile_entries()]
            gpu.profile(False)
            mt = path.pf_max_tiles()
            res[split] = dict(names=names, out=ob.view(np.uint16)[:T * D].copy(), cnt=path.pf_scratch(0, np.uint32)[:E].copy(), offs=path.pf_scratch(1, np.uint32)[:E].copy(),
                              tiles=path.pf_scratch(2, np.uint32)[:4 * mt].copy(), pos=path.pf_scratch(3, np.uint32)[:P].copy(),
                              Xs=path.pf_scratch(4, np.uint16)[:P * D].reshape(P, D).copy(), H=path.pf_scratch(5, np.uint16)[:P * I].reshape(P, I).copy())
            for bb in (xb, ib, wb, ob):
                bb.free()
            path.close()
    a, f = res[True], res[False]
    assert "qwk_moe_prep" in f["names"] and not any(n in f["names"] for n in ("qwk_zero", "qwk_moe_count", "qwk_moe_plan", "qwk_moe_scatter")), f["names"]
    assert "qwk_moe_prep" not in a["names"] and "qwk_moe_scatter" in a["names"] and "qwk_moe_act" in a["names"], a["names"]
    assert ("qwk_moe_act" not in f["names"]) == dev, f["names"]  # it rides only in the launch over the tile-major copy of gate and up
    for key in ("cnt", "offs", "tiles", "out"):
        assert np.array_equal(a[key], f[key]), key
    assert sorted(f["pos"].tolist()) == list(range(P))
    flat = ids.ravel()
    for e in range(E):  # inside an expert: the order of the pairs
        pe = f["pos"][flat == e]
        assert np.array_equal(pe, f["offs"][e] + np.arange(len(pe)))
    assert np.array_equal(a["Xs"][a["pos"]], f["Xs"][f["pos"]]) and np.array_equal(a["H"][a["pos"]], f["H"][f["pos"]])
    dl.free()


def _pk_kernels(gpu, tag, E, K, KD, I, tm):
    ks = {}
    for base in ("p_zero", "moe_count", "moe_plan_t", "moe_scatter"):
        name = "%s_%s" % (base, tag)
        ok, err = gpu.compile("#define %s %s\n#define E %d\n#define TOPK %d\n#define KD %d\n#define I %d\n#define TM %d\n" % (base, name, E, K, KD, I, tm))
        assert ok, err
        ks[base] = gpu.kernel(name)
        assert ks[base]
    return ks


def _pk_dispatch(b, ks, which, **a):
    """One dispatch of the packing sequence with the reference's binding indices (src/engine.c:4137-4144, 4201-4227)."""
    b.kernel(ks[which])
    if which == "p_zero":
        b.buf(0, a["x"])
        b.bytes(1, np.uint32([a["n"]]))
        b.dispatch((a["n"] + 255) // 256, tx=256)
    elif which == "moe_count":
        b.buf(0, a["ids"])
        b.buf(1, a["counts"])
        b.bytes(2, np.uint32([a["P"]]))
        b.dispatch((a["P"] + 255) // 256, tx=256)
    elif which == "moe_plan_t":
        for i, key in enumerate(("counts", "offs", "cursor", "tiles")):
            b.buf(i, a[key])
        b.bytes(4, np.uint32([a["max_tiles"]]))
        b.bytes(5, np.uint32([a["tm"]]))
        b.dispatch(1, tx=a["E"])
    else:
        for i, key in enumerate(("X", "ids", "cursor", "Xs", "pos_of")):
            b.buf(i, a[key])
        b.dispatch(a["P"], tx=256)


def test_packing_sequence_that_breaks_the_pattern(gpu, oracle):
    """p_zero, moe_count and moe_plan_t wait for the next dispatch of the sequence; a dispatch that does not continue it
    on the same buffers (or the end of the batch) launches what waited, one kernel per dispatch, in order. Every case
    must leave what the dispatches say, whichever launches carry them."""
    E, K, KD, I, tm, T = 32, 4, 512, 512, 16, 20
    P = T * K
    ks = _pk_kernels(gpu, "brk", E, K, KD, I, tm)
    rng = np.random.default_rng(81)
    ids = synth.zipf_ids(rng, T, E, K).astype(np.uint32).ravel()
    x = synth.activations(rng, T, KD)
    mt = (P + tm - 1) // tm + E
    counts, offs, _, tiles, _ = oracle.moe_pack(ids, E, tm, mt)
    idb, idb2, xb = gpu.buf_from(ids), gpu.buf_from(ids), gpu.buf_from(x)
    mk = lambda n: gpu.buf_from(np.full(n, 7, np.uint32))  # stale contents everywhere
    gpu.profile(True)

    def names():
        return [n for n, _ in gpu.profile_entries()]

    # 1. the counters cleared are not the counters counted into: two launches, both effects
    A, B = mk(E), mk(E)
    b = gpu.batch()
    _pk_dispatch(b, ks, "p_zero", x=A, n=E)
    _pk_dispatch(b, ks, "moe_count", ids=idb, counts=B, P=P)
    b.end()
    assert names() == ["qwk_zero", "qwk_moe_count"]
    assert not A.view(np.uint32)[:E].any() and np.array_equal(B.view(np.uint32)[:E], 7 + counts)
    # 2. the batch ends after the count: the two that waited are launched
    b = gpu.batch()
    _pk_dispatch(b, ks, "p_zero", x=A, n=E)
    _pk_dispatch(b, ks, "moe_count", ids=idb, counts=A, P=P)
    b.end()
    assert names() == ["qwk_zero", "qwk_moe_count"] and np.array_equal(A.view(np.uint32)[:E], counts)
    # 3. fewer dwords cleared than there are counters: no part of the pattern
    b = gpu.batch()
    _pk_dispatch(b, ks, "p_zero", x=B, n=E // 2)
    _pk_dispatch(b, ks, "moe_count", ids=idb, counts=B, P=P)
    b.end()
    assert names() == ["qwk_zero", "qwk_moe_count"]
    assert np.array_equal(B.view(np.uint32)[:E], np.concatenate([counts[:E // 2], 7 + 2 * counts[E // 2:]]))
    # 4. the scatter reads other ids than the count did (the same values at another address): three launches, then the scatter
    offb, curb, tilb, posb, Xs = mk(E), mk(E), mk(4 * mt), mk(P), gpu.buf(P * KD * 2)
    seq = dict(counts=A, offs=offb, cursor=curb, tiles=tilb, max_tiles=mt, tm=tm, E=E, X=xb, Xs=Xs, pos_of=posb, P=P)
    b = gpu.batch()
    _pk_dispatch(b, ks, "p_zero", x=A, n=E)
    _pk_dispatch(b, ks, "moe_count", ids=idb, **seq)
    _pk_dispatch(b, ks, "moe_plan_t", **seq)
    _pk_dispatch(b, ks, "moe_scatter", ids=idb2, **seq)
    b.end()
    assert names() == ["qwk_zero", "qwk_moe_count", "qwk_moe_plan", "qwk_moe_scatter"]

    def check():
        assert np.array_equal(A.view(np.uint32)[:E], counts) and np.array_equal(offb.view(np.uint32)[:E], offs)
        assert np.array_equal(curb.view(np.uint32)[:E], offs + counts) and np.array_equal(tilb.view(np.uint32)[:4 * mt], tiles.ravel())
        pos = posb.view(np.uint32)[:P]
        assert sorted(pos.tolist()) == list(range(P)) and all(offs[ids[p]] <= pos[p] < offs[ids[p]] + counts[ids[p]] for p in range(P))
        rows = Xs.view(np.uint16)[:P * KD].reshape(P, KD)
        assert all(np.array_equal(rows[pos[p]], x[p // K].view(np.uint16)) for p in range(P))

    check()
    # 5. the whole sequence twice in one batch, on the same buffers: one launch each, the same contents
    for bb in (A, offb, curb, posb):
        bb.fill(np.full(bb.view(np.uint32).size, 9, np.uint32))
    b = gpu.batch()
    for _ in range(2):
        _pk_dispatch(b, ks, "p_zero", x=A, n=E)
        _pk_dispatch(b, ks, "moe_count", ids=idb, **seq)
        _pk_dispatch(b, ks, "moe_plan_t", **seq)
        _pk_dispatch(b, ks, "moe_scatter", ids=idb, **seq)
    b.end()
    assert names() == ["qwk_moe_prep", "qwk_moe_prep"]
    check()
    gpu.profile(False)
    for bb in (idb, idb2, xb, A, B, offb, curb, tilb, posb, Xs):
        bb.free()
