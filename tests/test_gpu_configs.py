"""The benchmark configurations at their own shapes (D 2048, I 512, E 512, top-10), through the C interface, against
the CPU oracle: one layer at 8 tokens, the continuous-batching step of 16 slots with about 64 rows and Zipf(1.1)
routing (groups of 16 rows and the packing path), and consecutive layers of the mixed-format stack at 16 tokens with
every layer's output compared. The weights are generated on the device (as the benchmark does) and read back for the
oracle, so both sides see the same bytes."""
import numpy as np
import pytest

from helpers import maxrel
from qwental_amd import synth
from qwental_amd.gpu import SelRecord
from qwental_amd.stack import MoeStack

pytestmark = pytest.mark.gpu
TOL = 2e-3  # max |err| / max |ref| of the layer output (binary16), fp32 accumulation
D, I, E, K = 2048, 512, 512, 10


@pytest.fixture(scope="module")
def stack8(gpu):
    s = MoeStack(gpu, layers=8, D=D, I=I, E=E, topk=K, nbmax=16, q8_every=4, seed=77)
    yield s
    s.free()


def layer_out(stack, nb):
    return stack.out.view(np.float16)[:nb * D].reshape(nb, D).astype(np.float64)


def layer_logits(stack, l, nb):
    return stack.lg[l].read(dtype=np.float32)[:nb * (E + 1)].reshape(nb, E + 1).copy()


def test_config2_one_layer_eight_tokens(gpu, oracle, stack8):
    """BASELINE configs[2]: one MoE decode layer, B = 8, 512 experts, binary16 router, top-10 softmax gating, SwiGLU."""
    nb = 8
    xh = synth.activations(np.random.default_rng(8), nb, D)
    x = gpu.buf_from(xh, device_only=True)
    stack8.step(x, nb, nlayers=1)
    m = stack8.layer_weights_host(0)
    lg = layer_logits(stack8, 0, nb)
    # router: logits and picks against the oracle's own router over the same weights
    lg_ref = oracle.router(m["Wr"], m["wsg"], xh)
    assert maxrel(lg, lg_ref) <= 1e-5
    ids_ref = oracle.topk_ids(lg_ref, K)
    assert np.array_equal(oracle.topk_ids(lg, K), ids_ref)
    sel = SelRecord(stack8.sel[0].read(), 8, K)
    ref = oracle.select(lg, K, 8)
    assert sel.U == ref.U and np.array_equal(sel.ue[:sel.U], ref.ue[:ref.U]) and np.array_equal(sel.mask[:sel.U], ref.mask[:ref.U])
    assert np.array_equal(sel.slot[:sel.U], ref.slot[:ref.U])
    assert np.abs(sel.w[:nb] - ref.w[:nb]).max() <= 1e-6
    assert sorted(sel.ue[:sel.U].tolist()) == sorted(set(ids_ref.ravel().tolist()))
    err = maxrel(layer_out(stack8, nb), oracle.moe_layer_f64(m, lg, xh))
    assert err <= TOL, err
    x.free()


def test_config4_every_layer_of_the_mixed_stack(gpu, oracle, stack8):
    """BASELINE configs[4] over 8 consecutive layers at B = 16 (layers 3 and 7 carry their shared expert in Q8_0):
    the stack call with l + 1 layers leaves layer l's output, which is compared with the oracle for every l; the top-k
    of every layer is the oracle's."""
    nb = 16
    xh = synth.activations(np.random.default_rng(16), nb, D)
    x = gpu.buf_from(xh, device_only=True)
    assert [f[0] for f in stack8.shared_fmt] == [21, 21, 21, 8, 21, 21, 21, 8]
    worst = 0.0
    for l in range(stack8.L):
        stack8.step(x, nb, nlayers=l + 1)
        m = stack8.layer_weights_host(l)
        lg = layer_logits(stack8, l, nb)
        assert np.array_equal(oracle.topk_ids(lg, K), oracle.topk_ids(oracle.router(m["Wr"], m["wsg"], xh), K)), l
        sel = SelRecord(stack8.sel[l].read(), 16, K)
        ref = oracle.select(lg, K, 16)
        assert sel.U == ref.U and np.array_equal(sel.ue[:sel.U], ref.ue[:ref.U]), l
        err = maxrel(layer_out(stack8, nb), oracle.moe_layer_f64(m, lg, xh))
        worst = max(worst, err)
        assert err <= TOL, (l, err)
        del m
    print("worst layer error %.2e" % worst)
    x.free()


def test_config4_all_48_layers_at_full_size(gpu, oracle):
    """BASELINE configs[4] at its full size: the 48-layer stack (about 33 GB resident, every fourth layer's shared expert in
    Q8_0) at B = 16, every one of the 48 layers against the float32 oracle on the layer's own resident bytes, top-k
    identical everywhere. (The benchmark's CPU leg makes the same comparison on the layers its time budget reaches.)"""
    from qwental_amd.stack import MoeStack
    nb = 16
    stack = MoeStack(gpu, layers=48, nbmax=16)
    xh = synth.activations(np.random.default_rng(2024), nb, D)
    x = gpu.buf_from(xh, device_only=True)
    assert [f[0] for f in stack.shared_fmt] == [21, 21, 21, 8] * 12
    worst = 0.0
    for l in range(stack.L):
        stack.step(x, nb, nlayers=l + 1)
        m = stack.layer_weights_host(l)
        lg = layer_logits(stack, l, nb)
        assert np.array_equal(oracle.topk_ids(lg, K), oracle.topk_ids(oracle.router(m["Wr"], m["wsg"], xh), K)), l
        out32, _, _ = oracle.moe_layer_f32(m, lg, xh, 16)
        err = maxrel(layer_out(stack, nb), out32)
        worst = max(worst, err)
        assert err <= TOL, (l, err)
        del m
    print("48 layers, worst layer error %.2e" % worst)
    x.free()
    stack.free()


def test_config3_continuous_batching_step(gpu, oracle, stack8):
    """BASELINE configs[3]: 16 slots with seeded row counts in 1..16 (64 rows), Zipf(1.1) routing forced through the
    logits. The rows go through the decode path in groups of 16 (every group against the float64 layer) and through
    the packing path in one pass: counts, offsets, tile table and packed positions bit-exact against the oracle, the
    routed sums against a float64 recompute per row."""
    rng = np.random.default_rng(1064)
    while True:
        n = rng.integers(1, 17, 16)
        if abs(int(n.sum()) - 64) <= 4:
            break
    T = int(n.sum())
    path, layer = stack8.path, stack8.layers[1]
    m = stack8.layer_weights_host(1)
    xh = synth.activations(rng, T, D)
    ids = synth.zipf_ids(rng, T, E, K)
    lg = synth.logits_for_ids(rng, ids, E)
    counts = np.bincount(ids.ravel(), minlength=E)
    assert counts.max() > 16  # a hot expert spans more than one tile entry
    wts = np.zeros((T, K), np.float32)
    for g0 in range(0, T, 16):
        nb = min(16, T - g0)
        gnb = 8 if nb <= 8 else 16
        xb, lb = gpu.buf_from(xh[g0:g0 + nb]), gpu.buf_from(lg[g0:g0 + nb])
        sb, ob = gpu.buf(path.sel_bytes(nb)), gpu.buf(nb * D * 2)
        b = gpu.batch()
        path.gg_moe_lg(b, layer, nb, xb, lb, sb, ob)
        b.end()
        sel = SelRecord(sb.view(np.uint8).copy(), gnb, K)
        ref = oracle.select(lg[g0:g0 + nb], K, gnb)
        assert sel.U == ref.U and np.array_equal(sel.ue[:ref.U], ref.ue[:ref.U])
        assert np.array_equal(oracle.topk_ids(lg[g0:g0 + nb], K), ids[g0:g0 + nb])
        got = ob.view(np.float16)[:nb * D].reshape(nb, D).astype(np.float64)
        err = maxrel(got, oracle.moe_layer_f64(m, lg[g0:g0 + nb], xh[g0:g0 + nb]))
        assert err <= TOL, (g0, err)
        wts[g0:g0 + nb] = sel.w[:nb, :K]
        for bb in (xb, lb, sb, ob):
            bb.free()
    # the packing path over all rows at once
    tm = 16
    path.pf_reserve(T, tm)
    xb, ib, wb, ob = gpu.buf_from(xh), gpu.buf_from(ids.astype(np.uint32).ravel()), gpu.buf_from(wts.ravel()), gpu.buf(T * D * 2)
    b = gpu.batch()
    path.pf_moe(b, layer, T, xb, ib, wb, ob)
    b.end()
    P, mt = T * K, path.pf_max_tiles()
    c_ref, offs, _, tiles, _ = oracle.moe_pack(ids.ravel(), E, tm, mt)
    assert np.array_equal(path.pf_scratch(0, np.uint32)[:E], c_ref) and np.array_equal(c_ref, counts)
    assert np.array_equal(path.pf_scratch(1, np.uint32)[:E], offs)
    assert np.array_equal(offs, np.concatenate([[0], np.cumsum(counts)[:-1]]))  # exclusive prefix sums
    assert np.array_equal(path.pf_scratch(2, np.uint32)[:4 * mt].reshape(mt, 4), tiles.reshape(mt, 4))
    pos = path.pf_scratch(3, np.uint32)[:P]
    flat = ids.ravel()
    assert sorted(pos.tolist()) == list(range(P))
    assert all(offs[flat[p]] <= pos[p] < offs[flat[p]] + counts[flat[p]] for p in range(P))
    # float64 recompute of the routed sums with the reference's binary16 roundings of H and of the down output
    rg, rd = synth.row_bytes(21, D), synth.row_bytes(21, I)
    Wg, Wu, Wd = m["Wg"].reshape(E, I * rg), m["Wu"].reshape(E, I * rg), m["Wd"].reshape(E, D * rd)
    ref = np.zeros((T, D))
    for t in range(T):
        for s in range(K):
            e = int(ids[t, s])
            g = oracle.qmv(21, Wg[e], I, D, xh[t][None, :], f64=True)[0]
            u = oracle.qmv(21, Wu[e], I, D, xh[t][None, :], f64=True)[0]
            h = (g / (1.0 + np.exp(-g)) * u).astype(np.float16)
            d = oracle.qmv(21, Wd[e], D, I, h[None, :], f64=True)[0]
            ref[t] += wts[t, s] * d.astype(np.float16).astype(np.float64)
    got = ob.view(np.float16)[:T * D].reshape(T, D).astype(np.float64)
    err = maxrel(got, ref)
    assert err <= TOL, err
    for bb in (xb, ib, wb, ob):
        bb.free()


def test_two_packing_passes_in_one_batch(gpu, oracle, stack8):
    """The packing sequence twice in one batch (two layers of a step): the second pass starts from counters cleared on
    the device, so its counts, offsets and outputs are those of a pass on its own."""
    rng = np.random.default_rng(2)
    T = 24
    path = stack8.path
    xh = synth.activations(rng, T, D)
    ids_a, ids_b = synth.zipf_ids(rng, T, E, K), synth.zipf_ids(rng, T, E, K)
    w = np.full((T, K), 1.0 / K, np.float32)
    path.pf_reserve(T, 16)
    xb, wb = gpu.buf_from(xh), gpu.buf_from(w.ravel())
    ia, ib = gpu.buf_from(ids_a.astype(np.uint32).ravel()), gpu.buf_from(ids_b.astype(np.uint32).ravel())
    oa, ob, oc = gpu.buf(T * D * 2), gpu.buf(T * D * 2), gpu.buf(T * D * 2)
    b = gpu.batch()
    path.pf_moe(b, stack8.layers[0], T, xb, ia, wb, oa)
    path.pf_moe(b, stack8.layers[2], T, xb, ib, wb, ob)
    b.end()
    assert np.array_equal(path.pf_scratch(0, np.uint32)[:E], np.bincount(ids_b.ravel(), minlength=E))
    b = gpu.batch()
    path.pf_moe(b, stack8.layers[2], T, xb, ib, wb, oc)
    b.end()
    assert np.array_equal(ob.view(np.uint16), oc.view(np.uint16))
    for bb in (xb, wb, ia, ib, oa, ob, oc):
        bb.free()
