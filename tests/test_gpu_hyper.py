"""The hyper-connection either side of the MoE layer (the reference's kernels/hyper_gg.metal behind its hyper_gg(),
src/engine.c:1344-1412) against the oracle's float64 statement. Tolerances are the reference's own for this step
(tools/hc_ref.py:84): x 1e-3 of the largest value (it is rounded to binary16), h 1e-6, inject sums 1e-4."""
import numpy as np
import pytest

import qwental_amd as q
from qwental_amd import synth

pytestmark = pytest.mark.gpu
HC, LR = 4, 320
TOL_X, TOL_H, TOL_I = 1e-3, 1e-6, 1e-4


def rel(a, b):
    return float(np.abs(a.astype(np.float64) - b).max() / np.abs(b).max())


class Hyper:
    """One hyper-connection's weights in HBM and the buffers of a call."""

    def __init__(self, gpu, D, nbmax, rng, inject=True):
        self.gpu, self.D = gpu, D
        self.path = q.Path(gpu, D, 512, 64, 4, 16)
        self.w = synth.hyper_weights(rng, D, inject=inject)
        self.bufs = {k: gpu.buf_from(v) for k, v in self.w.items() if v is not None}
        self.H = {"hc_norm": q.Tensor(self.bufs["hc_norm"], 0), "mix_down": q.Tensor(self.bufs["mix_down"], 30), "mix_up": q.Tensor(self.bufs["mix_up"], 30),
                  "inject": q.Tensor(self.bufs["inject"], 30) if inject else None}
        self.pd = gpu.buf(int(gpu.L.qw_path_hyper_pd_bytes(nbmax)))

    def run(self, h, out, inj, apply, three=False):
        gpu, nb = self.gpu, h.shape[0]
        hb, ob, ib = gpu.buf_from(h), gpu.buf_from(out), gpu.buf_from(inj)
        io, x = gpu.buf_from(np.full((nb, HC, HC), 7.0, np.float32)), gpu.buf(nb * self.D * 2)
        b = gpu.batch()
        self.path.hyper_gg(b, self.H, nb, apply, hb, ob, ib, io, self.pd, x, three=three)
        b.end()
        res = (hb.view(np.float32).reshape(nb, HC, self.D).copy(), x.view(np.float16).reshape(nb, self.D).copy(), io.view(np.float32).reshape(nb, HC, HC).copy())
        for bb in (hb, ob, ib, io, x):
            bb.free()
        return res

    def oracle(self, o, h, out, inj, apply):
        return o.hyper_gg(h, out, inj, self.w["hc_norm"], self.w["mix_down"], self.w["inject"], self.w["mix_up"], apply)

    def free(self):
        for b in self.bufs.values():
            b.free()
        self.pd.free()
        self.path.close()


@pytest.fixture(scope="module", params=[2048, 2560])
def hyper(request, gpu):
    hy = Hyper(gpu, request.param, 16, np.random.default_rng(request.param))
    yield hy
    hy.free()


@pytest.mark.parametrize("nb", [1, 2, 5, 8, 16])
@pytest.mark.parametrize("apply", [0, 1])
def test_against_the_oracle(gpu, oracle, hyper, nb, apply):
    h, out, inj = synth.hyper_state(np.random.default_rng(100 * nb + apply), nb, hyper.D)
    gh, gx, gi = hyper.run(h, out, inj, apply)
    rh, rx, ri = hyper.oracle(oracle, h, out, inj, apply)
    assert rel(gx, rx) <= TOL_X and rel(gi, ri) <= TOL_I
    if apply:
        assert rel(gh, rh) <= TOL_H
    else:
        assert np.array_equal(gh, h)  # nothing is written back


def test_three_kernel_sequence_gives_the_same_bits(gpu, oracle, hyper):
    """The reference runs ghc_dsk, ghc_mid, ghc_upv for more than one token (src/engine.c:1347-1386) and promises the
    same bits as its two-kernel form; so do the kernels here (one routine makes sx and rs in both)."""
    for nb, apply in ((1, 1), (7, 1), (16, 0)):
        h, out, inj = synth.hyper_state(np.random.default_rng(7 + nb), nb, hyper.D)
        a, b = hyper.run(h, out, inj, apply), hyper.run(h, out, inj, apply, three=True)
        for u, v in zip(a, b):
            assert np.array_equal(u.view(np.uint8), v.view(np.uint8))
        rh, rx, ri = hyper.oracle(oracle, h, out, inj, apply)
        assert rel(b[1], rx) <= TOL_X and rel(b[2], ri) <= TOL_I


def test_a_token_does_not_depend_on_its_batch(gpu, hyper):
    h, out, inj = synth.hyper_state(np.random.default_rng(11), 16, hyper.D)
    gh, gx, gi = hyper.run(h, out, inj, 1)
    for t in (0, 9, 15):
        h1, x1, i1 = hyper.run(h[t:t + 1], out[t:t + 1], inj[t:t + 1], 1)
        assert np.array_equal(h1[0].view(np.uint32), gh[t].view(np.uint32)) and np.array_equal(x1[0].view(np.uint16), gx[t].view(np.uint16))
        assert np.array_equal(i1[0].view(np.uint32), gi[t].view(np.uint32))


def test_without_inject_rows_nothing_is_written_there(gpu, oracle):
    """The reference's final mixer has no inject matrix (src/model.h:44): the flag is off and inj_out stays as it was."""
    hy = Hyper(gpu, 2048, 4, np.random.default_rng(5), inject=False)
    h, out, inj = synth.hyper_state(np.random.default_rng(6), 3, 2048)
    for three in (False, True):
        gh, gx, gi = hy.run(h, out, inj, 1, three=three)
        rh, rx, _ = hy.oracle(oracle, h, out, inj, 1)
        assert rel(gx, rx) <= TOL_X and rel(gh, rh) <= TOL_H and np.all(gi == 7.0)
    hy.free()


def test_two_in_a_row_carry_the_streams_and_the_inject_sums(gpu, oracle, hyper):
    """hyper_in before a sublayer, the sublayer's output, hyper_in of the next sublayer with the residual applied
    (src/engine.c:1415-1423): the second call reads the h the first left (unchanged: nothing was pending), the output and the
    first call's inject sums; each call is checked against the oracle on the inputs the device had."""
    rng = np.random.default_rng(21)
    nb, D = 4, hyper.D
    h, out, inj = synth.hyper_state(rng, nb, D)
    h1, x1, i1 = hyper.run(h, out, inj, 0)
    sub = (x1.astype(np.float32) * 0.7).astype(np.float16)  # a stand-in for the sublayer
    h2, x2, i2 = hyper.run(h1, sub, i1, 1)
    rh, rx, ri = hyper.oracle(oracle, h1, sub, i1, 1)
    assert rel(x2, rx) <= TOL_X and rel(h2, rh) <= TOL_H and rel(i2, ri) <= TOL_I
    assert not np.array_equal(h2, h1)


def test_refusals(gpu):
    blk = "#define ghc_down ghc_down_t\n#define ghc_up ghc_up_t\n#define D %d\n#define HC %d\n#define NB %d\n#define GH_R 16\n"
    for D, hc, nb in ((2304, 4, 1), (2048, 3, 1), (2048, 4, 17), (8192, 4, 1)):
        ok, err = gpu.compile(blk % (D, hc, nb))
        assert not ok and err
    ok, err = gpu.compile(blk % (2048, 4, 2))
    assert ok, err
    # a stream buffer one float short, an offset that is not a multiple of 16
    nb, D = 2, 2048
    w = synth.hyper_weights(np.random.default_rng(1), D)
    bufs = {k: gpu.buf_from(v) for k, v in w.items()}
    pd, fl = gpu.buf(nb * HC * 328 * 4), np.array([0, 1], np.uint32)
    for hbytes, off in ((nb * HC * D * 4 - 4, 0), (nb * HC * D * 4 + 16, 8)):
        h = gpu.buf(hbytes)
        b = gpu.batch()
        b.kernel(gpu.kernel("ghc_down_t"))
        b.buf(0, h, off)
        b.buf(3, bufs["hc_norm"])
        b.buf(4, bufs["mix_down"])
        b.buf(5, bufs["inject"])
        b.buf(6, pd)
        b.bytes(7, fl)
        b.dispatch(21, 4, 1, D // 8, 1, 1)
        assert b.end(check=False) < 0 and gpu.last_error()
        h.free()
    for bb in list(bufs.values()) + [pd]:
        bb.free()


def test_hyper_then_moe_layer_after_layer(gpu, oracle):
    """The FFN half of the decode loop with a real dependency between layers (hyper_in -> moe, src/engine.c:1415-1423, :2169):
    the stack is run for 1, 2 and 3 layers from the same start, and the last layer of every run is checked stage by stage
    against the oracle on the state the device had before it (so that a near-tie in a router cannot flip the comparison)."""
    from qwental_amd.stack import MoeStack
    stack = MoeStack(gpu, layers=3, nbmax=8, seed=5).add_hyper(seed=6)
    nb, D = 5, stack.D
    h0, _, inj0 = synth.hyper_state(np.random.default_rng(8), nb, D)

    def run(k):
        stack.h.fill(h0)
        stack.inj[0].fill(inj0)
        stack.inj[1].fill(np.zeros_like(inj0))
        stack.step_hyper(nb, nlayers=k)
        return dict(h=stack.h.view(np.float32)[:nb * HC * D].reshape(nb, HC, D).copy(), x=stack.x.view(np.float16)[:nb * D].reshape(nb, D).copy(),
                    out=stack.out.view(np.float16)[:nb * D].reshape(nb, D).copy(), inj=stack.inj[k % 2].view(np.float32)[:nb * 16].reshape(nb, HC, HC).copy(),
                    lg=stack.lg[k - 1].read(dtype=np.float32)[:nb * (stack.E + 1)].reshape(nb, stack.E + 1).copy())

    prev = dict(h=h0, out=np.zeros((nb, D), np.float16), inj=inj0)
    for k in (1, 2, 3):
        cur = run(k)
        w = stack.hyper_host[k - 1]
        rh, rx, ri = oracle.hyper_gg(prev["h"], prev["out"], prev["inj"], w["hc_norm"], w["mix_down"], w["inject"], w["mix_up"], k > 1)
        assert rel(cur["x"], rx) <= TOL_X and rel(cur["inj"], ri) <= TOL_I
        assert rel(cur["h"], rh) <= TOL_H if k > 1 else np.array_equal(cur["h"], h0)
        ref = oracle.moe_layer_f64(stack.layer_weights_host(k - 1), cur["lg"], cur["x"])
        assert np.isfinite(cur["out"]).all() and rel(cur["out"], ref) <= 2e-3
        prev = cur
    again = run(3)  # the same bits on a second run from the same start
    for key in ("h", "x", "out", "inj"):
        assert np.array_equal(again[key].view(np.uint8), prev[key].view(np.uint8))
    stack.free()
