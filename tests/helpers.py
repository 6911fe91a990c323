"""Shared pieces of the GPU parity tests: device-side layer construction and error metrics."""
import numpy as np

import qwental_amd as q


def maxrel(got, ref):
    """max |got - ref| / max |ref| — the metric of the reference's comparators (tools/ggmtest.py:45-53, tools/moe_ref.py:87-91)."""
    got = np.asarray(got, np.float64)
    ref = np.asarray(ref, np.float64)
    return float(np.abs(got - ref).max() / (np.abs(ref).max() + 1e-300))


def dq_define_block(ftype):
    return "#define IQ_DQ_ONLY 1\n#define DQ_TEST %d\n" % ftype  # tools/dqtest.c:27


def gpu_dq_rows(gpu, ftype, raw, K):
    """The flow of tools/dqtest.c:26-48 through the C interface."""
    rows, rb = raw.shape
    ok, err = gpu.compile(dq_define_block(ftype))
    assert ok, err
    k = gpu.kernel("dq_test")
    assert k
    w = gpu.buf_from(raw)
    y = gpu.buf(rows * K * 4)
    b = gpu.batch()
    b.kernel(k)
    b.buf(0, w)
    b.buf(1, y)
    b.bytes(2, np.array([K, rb], np.uint32))
    b.dispatch(rows, 1, 1, 32, 1, 1)
    b.end()
    out = y.view(np.float32).reshape(rows, K).copy()
    w.free()
    y.free()
    return out


class DeviceLayer:
    """A synthetic MoE layer (qwental_amd.synth.moe_layer dict) resident in HBM."""

    def __init__(self, gpu, m, router_type=1, device_only=False):
        self.m = m
        mk = lambda a: gpu.buf_from(a, device_only=device_only)
        self.bufs = {k: mk(m[k]) for k in ("Wg", "Wu", "Wd", "Wsg", "Wsu", "Wsd")}
        self.bufs["Wr"] = mk(m["Wr"].view(np.uint16))
        self.bufs["wsg"] = mk(m["wsg"].view(np.uint16))
        T = q.Tensor
        self.layer = q.MoeLayer(router=T(self.bufs["Wr"], router_type), sh_gate_w=T(self.bufs["wsg"], router_type),
                                gate=T(self.bufs["Wg"], m["fgu"]), up=T(self.bufs["Wu"], m["fgu"]), down=T(self.bufs["Wd"], m["fd"]),
                                sh_gate=T(self.bufs["Wsg"], m["fsg"]), sh_up=T(self.bufs["Wsu"], m["fsu"]), sh_down=T(self.bufs["Wsd"], m["fsd"]))

    def free(self):
        for b in self.bufs.values():
            b.free()


def run_moe(gpu, path, dl, x, nb):
    """One layer through qw_path_gg_moe; returns (out f16 [nb, D], logits f32 [nb, E+1], selection bytes)."""
    D, E = path.D, path.E
    xb = gpu.buf_from(x)
    lg = gpu.buf(path.logits_bytes(nb))
    sel = gpu.buf(path.sel_bytes(nb))
    out = gpu.buf(nb * D * 2)
    b = gpu.batch()
    path.gg_moe(b, dl.layer, nb, xb, lg, sel, out)
    t = b.end()
    res = (out.view(np.float16).reshape(nb, D).copy(), lg.view(np.float32).reshape(nb, E + 1).copy(), sel.view(np.uint8).copy(), t)
    for bb in (xb, lg, sel, out):
        bb.free()
    return res
