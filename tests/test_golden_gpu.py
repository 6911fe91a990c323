"""The HIP path, through the C interface, against the committed golden fixtures of tests/golden/."""
import numpy as np
import pytest

import qwental_amd as q
from helpers import DeviceLayer, gpu_dq_rows, maxrel, run_moe
from test_golden_cpu import load, moe_cases, qmv_cases

pytestmark = pytest.mark.gpu
TOL = 2e-3


def test_gpu_iq3s_fixture(gpu):
    g = load("dq_iq3s.npz")
    assert np.array_equal(gpu_dq_rows(gpu, 21, g["raw"], 256).view(np.uint32), g["expect"].view(np.uint32))


def test_gpu_q8_0_fixture(gpu):
    g = load("dq_q8_0.npz")
    assert np.array_equal(gpu_dq_rows(gpu, 8, g["raw"], 32).view(np.uint32), g["expect"].view(np.uint32))


def test_gpu_qmv_fixture(gpu):
    path = q.Path(gpu, 2048, 512, 512, 10, 16)
    for ft, K, N, W, x, y in qmv_cases():
        print("qmv fixture type %d K %d N %d" % (ft, K, N), flush=True)
        wb, xb, yb = gpu.buf_from(W), gpu.buf_from(x), gpu.buf(5 * N * 4)
        b = gpu.batch()
        path.qmv_gg(b, q.Tensor(wb, ft), N, K, xb, yb, 5, fout=True)
        assert b.end() >= 0, gpu.last_error()
        assert maxrel(yb.view(np.float32)[:5 * N].reshape(5, N), y) <= 1e-5
        for bb in (wb, xb, yb):
            bb.free()
    path.close()


def test_gpu_select_fixture(gpu):
    g = load("select.npz")
    lg, K = g["logits"], int(g["topk"])
    nb, E = lg.shape[0], lg.shape[1] - 1
    ok, err = gpu.compile("#define E %d\n#define TOPK %d\n#define D 256\n#define I 256\n#define NB %d\n#define GG_PART 0\n#define moe_sel_gg sel_fix\n#define gg_tab_init tab_fix\n" % (E, K, nb))
    assert ok, err
    lb, sb = gpu.buf_from(lg), gpu.buf(len(g["record"]))
    b = gpu.batch()
    b.kernel(gpu.kernel("sel_fix"))
    b.buf(0, lb)
    b.buf(1, sb)
    b.bytes(2, np.array([nb], np.uint32))
    b.dispatch(1, 1, 1, 1024, 1, 1)
    assert b.end() >= 0, gpu.last_error()
    rec, ref = sb.view(np.uint8).copy(), g["record"]
    wo = len(ref) - 4 * 8 * (K + 1)  # everything before the float weights is integer work: identical
    assert np.array_equal(rec[:wo], ref[:wo])
    assert np.allclose(rec[wo:].view(np.float32), ref[wo:].view(np.float32), rtol=2e-6, atol=1e-7)
    lb.free()
    sb.free()


def test_gpu_moe_fixture(gpu):
    for tag, m, x, nb, lg, ids, out in moe_cases():
        print("moe fixture", tag, flush=True)
        path = q.Path(gpu, m["D"], m["I"], m["E"], m["topk"], 16)
        dl = DeviceLayer(gpu, m)
        got, glg, _, t = run_moe(gpu, path, dl, x, nb)
        assert t >= 0
        assert maxrel(glg, lg) <= 1e-5
        # identical indices wherever the fixture's own rank K / K + 1 gap is above the logits' rounding noise
        srt = -np.sort(-lg[:, :-1], axis=1)
        clear = (srt[:, m["topk"] - 1] - srt[:, m["topk"]]) > 1e-4 * np.abs(lg).max()
        from oracle import oracle as o
        assert np.array_equal(o.topk_ids(glg, m["topk"])[clear], ids[clear]) and clear.sum() >= nb - 1
        if clear.all():
            assert maxrel(got, out) <= TOL
        dl.free()
        path.close()
