"""Routed gate/up, down and combine of a layer as one launch (qwk_gud_*; kernels/moe_gg.metal:600-663 of the reference in
one pass): everything it leaves in memory must equal, bit for bit, what the separate launches leave, and the output
must meet the float64 layer. Also: the record given instead of made, several layers and several batches over the same
synchronisation words, and the bounded wait giving up (forced from the host, so that every workgroup still exits)."""
import os

import numpy as np
import pytest

import qwental_amd as q
from qwental_amd import synth
from helpers import DeviceLayer, maxrel, run_moe

pytestmark = pytest.mark.gpu
TOL = 2e-3


def layer_state(gpu, path, dl, x, nb, K, D, I):
    gpu.profile(True)
    out, lg, sel, _ = run_moe(gpu, path, dl, x, nb)
    names = [n for n, _ in gpu.profile_entries()]
    gpu.profile(False)
    H = path.scratch(1).view(np.uint16)
    plane = gpu.L.qw_path_nbv(nb) * (K + 1) * I  # the planes lie as far apart as the compiled token count asks
    used = nb * (K + 1) * I
    return dict(out=out, lg=lg, sel=sel[:path.sel_bytes(nb)].copy(), names=names, Hhi=H[:used].copy(), Hlo=H[plane:plane + used].copy(),
                Psh=path.scratch(2).view(np.uint32)[:nb * D].copy(), Pg=path.scratch(3).view(np.uint32)[:nb * K * D].copy())


def same_bits(a, b, nb, K, I, lg):
    assert np.array_equal(a["out"].view(np.uint16), b["out"].view(np.uint16))
    assert np.array_equal(a["lg"].view(np.uint32), b["lg"].view(np.uint32)) and np.array_equal(a["sel"], b["sel"])
    assert np.array_equal(a["Psh"], b["Psh"])
    # H and Pg hold a value only where a token picked an expert in that slot: every slot of every token, here
    assert np.array_equal(a["Hhi"], b["Hhi"]) and np.array_equal(a["Hlo"], b["Hlo"])
    assert np.array_equal(a["Pg"], b["Pg"])


@pytest.mark.parametrize("nb", [1, 2, 3, 4, 6, 7, 8, 12, 13, 16])
@pytest.mark.parametrize("fshd,E,K,D", [(21, 64, 10, 2048), (8, 64, 10, 2048), (21, 512, 10, 2048), (21, 64, 8, 1024), (8, 96, 6, 2048), (21, 32, 4, 512)])
def test_one_launch_equals_the_separate_launches(gpu, oracle, nb, fshd, E, K, D):
    """Every token count's split into shares (one share of one token; two, four or eight shares of up to three), both
    shared-expert formats, an expert count the fast selection does not take (96), smaller D (fewer tile groups than
    workgroups: some workgroups only take part in the gate/up phase)."""
    if os.environ.get("QW_HIP_REPACK") == "0":
        pytest.skip("tile-major copies are switched off in this environment")
    I = 512
    rng = np.random.default_rng(4100 + nb + fshd + E + K + D)
    m = synth.moe_layer(rng, D, I, E, fgu=21, fd=21, fsh=21 if fshd == 21 else 8, fshd=fshd)
    m["topk"] = K
    x = synth.activations(rng, nb, D)
    if nb > 1:
        x[nb - 1] = x[0]  # two tokens of different shares on the same experts
    dl = DeviceLayer(gpu, m, device_only=True)
    res = {}
    for fuse in (0, 1):
        with gpu.switches(fuse=fuse):
            path = q.Path(gpu, D, I, E, K, 16)
            res[fuse] = layer_state(gpu, path, dl, x, nb, K, D, I)
            path.close()
    a, b = res[0], res[1]
    assert any(n.startswith("qwk_gud_") for n in b["names"]) and not any(n.startswith(("qwk_gu_", "qwk_dn", "qwk_cmb")) for n in b["names"]), b["names"]
    assert any(n.startswith("qwk_gu_") for n in a["names"]) and not any(n.startswith("qwk_gud_") for n in a["names"]), a["names"]
    same_bits(a, b, nb, K, I, b["lg"])
    assert maxrel(b["out"], oracle.moe_layer_f64(m, b["lg"], x)) <= TOL
    dl.free()


def test_one_launch_with_the_record_given(gpu, oracle):
    """With the selection as a launch of its own (QW_HIP_SPLIT_SELECT) the fused launch loads the record instead of
    making it; same bits."""
    if os.environ.get("QW_HIP_REPACK") == "0":
        pytest.skip("tile-major copies are switched off in this environment")
    D, I, E, K, nb = 2048, 512, 128, 10, 11
    rng = np.random.default_rng(4242)
    m = synth.moe_layer(rng, D, I, E)
    m["topk"] = K
    x = synth.activations(rng, nb, D)
    dl = DeviceLayer(gpu, m, device_only=True)
    res = []
    for split in (None, "1"):
        with gpu.switches(split_select=split, fuse=1):
            path = q.Path(gpu, D, I, E, K, 16)
            res.append(layer_state(gpu, path, dl, x, nb, K, D, I))
            path.close()
    assert "qwk_select" in res[1]["names"] and "qwk_select" not in res[0]["names"]
    assert all(any(n.startswith("qwk_gud_") for n in r["names"]) for r in res)
    same_bits(res[0], res[1], nb, K, I, res[0]["lg"])
    assert maxrel(res[1]["out"], oracle.moe_layer_f64(m, res[1]["lg"], x)) <= TOL
    dl.free()


def test_chained_layers_and_repeated_batches_over_the_same_barrier_words(gpu, oracle):
    """Four layers in one batch, each one's output the next one's input, run three times, and once with separate
    launches: the synchronisation words go through twelve barriers and every run gives the same bits."""
    if os.environ.get("QW_HIP_REPACK") == "0":
        pytest.skip("tile-major copies are switched off in this environment")
    D, I, E, K, nb, NL = 2048, 512, 64, 10, 16, 4
    rng = np.random.default_rng(4343)
    # a layer's output grows with the cube of its block scales and the square of its input: scales drawn smaller from the
    # second layer on keep every layer's output at a few hundred (binary16 stays finite and far from zero)
    ms = [synth.moe_layer(rng, D, I, E, d_scale=synth.MOE_D_SCALE / (1, 150, 40, 40)[l]) for l in range(NL)]
    for m in ms:
        m["topk"] = K
    x = synth.activations(rng, nb, D)
    dls = [DeviceLayer(gpu, m, device_only=True) for m in ms]
    path = q.Path(gpu, D, I, E, K, 16)
    xb = gpu.buf_from(x)
    acts = [gpu.buf(nb * D * 2) for _ in range(NL)]
    lgs, sels = [gpu.buf(path.logits_bytes(nb)) for _ in range(NL)], [gpu.buf(path.sel_bytes(nb)) for _ in range(NL)]

    def run():
        b = gpu.batch()
        for l in range(NL):
            path.gg_moe(b, dls[l].layer, nb, xb if l == 0 else acts[l - 1], lgs[l], sels[l], acts[l])
        assert b.end() >= 0, gpu.last_error()
        return [a.view(np.uint16)[:nb * D].copy() for a in acts]

    ref = run()
    with gpu.switches(fuse=1):
        for _ in range(3):
            got = run()
            assert all(np.array_equal(r, g) for r, g in zip(ref, got))
    h = x
    for l in range(NL):  # and every layer against the float64 layer on the input it saw
        lg = lgs[l].view(np.float32)[:nb * (E + 1)].reshape(nb, E + 1)
        out = acts[l].view(np.float16)[:nb * D].reshape(nb, D)
        assert np.isfinite(out.astype(np.float64)).all()
        assert maxrel(out, oracle.moe_layer_f64(ms[l], lg, h)) <= TOL, l
        h = out.copy()
    for bb in [xb] + acts + lgs + sels:
        bb.free()
    for d in dls:
        d.free()
    path.close()


def test_a_wait_that_gives_up_fails_the_batch_and_nothing_hangs(gpu, oracle):
    """QW_HIP_SPIN_LIMIT=0: a workgroup that does not find the barrier complete at its first look gives up, so every
    workgroup exits at once. The batch reports failure with a message, later batches run the layer as separate launches
    (and give the right result), and after qw_hip_reload_switches the fused launch is used again."""
    if os.environ.get("QW_HIP_REPACK") == "0":
        pytest.skip("tile-major copies are switched off in this environment")
    D, I, E, K, nb = 2048, 512, 64, 10, 8
    rng = np.random.default_rng(4444)
    m = synth.moe_layer(rng, D, I, E)
    m["topk"] = K
    x = synth.activations(rng, nb, D)
    dl = DeviceLayer(gpu, m, device_only=True)
    path = q.Path(gpu, D, I, E, K, 16)
    with gpu.switches(fuse=1):
        good = layer_state(gpu, path, dl, x, nb, K, D, I)
    assert any(n.startswith("qwk_gud_") for n in good["names"])
    xb, lg, sel, out = gpu.buf_from(x), gpu.buf(path.logits_bytes(nb)), gpu.buf(path.sel_bytes(nb)), gpu.buf(nb * D * 2)
    with gpu.switches(spin_limit=0, quiet=1, fuse=1):
        b = gpu.batch()
        path.gg_moe(b, dl.layer, nb, xb, lg, sel, out)
        assert b.end(check=False) < 0
        assert "timed out" in gpu.last_error()
        later = layer_state(gpu, path, dl, x, nb, K, D, I)  # the device has given fused launches up
        assert not any(n.startswith("qwk_gud_") for n in later["names"])
        same_bits(good, later, nb, K, I, good["lg"])
    with gpu.switches(fuse=1):
        again = layer_state(gpu, path, dl, x, nb, K, D, I)  # switches read again on entering the block
    assert any(n.startswith("qwk_gud_") for n in again["names"])
    same_bits(good, again, nb, K, I, good["lg"])
    for bb in (xb, lg, sel, out):
        bb.free()
    dl.free()
    path.close()
