"""The entry point that allocates nothing (qw_path_gg_moe_noalloc, include/qw_path.h) against the entry point it is a
variant of (qw_path_gg_moe): the same layer over the same device memory, two calls in a row, the second with fewer
tokens; outputs bit for bit."""
import ctypes as C

import numpy as np
import pytest

import qwental_amd as q
from helpers import DeviceLayer, maxrel
from qwental_amd import synth
from qwental_amd.gpu import QwMoeWeightsDev

pytestmark = pytest.mark.gpu


def devptr(gpu, buf):
    return gpu.L.qw_hip_buf_devptr(buf.ref())


@pytest.mark.parametrize("shape", [(2048, 512, 64, 10, 21, 21, 21), (2560, 640, 32, 10, 21, 20, 8), (1024, 256, 128, 8, 8, 8, 8)])
def test_no_alloc_layer_equals_the_allocating_entry_point(gpu, oracle, shape):
    D, I, E, K, fgu, fd, fsh = shape
    rng = np.random.default_rng(D + E)
    m = synth.moe_layer(rng, D, I, E, fgu=fgu, fd=fd, fsh=fsh)
    m["topk"] = K
    dl = DeviceLayer(gpu, m, device_only=True)
    path = q.Path(gpu, D, I, E, K, 16, device_scratch=True)
    W = QwMoeWeightsDev(*[devptr(gpu, dl.bufs[k]) for k in ("Wr", "wsg", "Wg", "Wu", "Wd", "Wsg", "Wsu", "Wsd")], 1, fgu, fd, fsh, fsh, fsh)
    for nb in (16, 5):  # two calls in a row, the second with the smaller input
        x = synth.activations(rng, nb, D)
        xb, lg, sel = gpu.buf_from(x, device_only=True), gpu.buf(path.logits_bytes(nb)), gpu.buf(path.sel_bytes(nb))
        ref_out, out = gpu.buf(nb * D * 2, device_only=True), gpu.buf(nb * D * 2, device_only=True)
        b = gpu.batch()
        path.gg_moe(b, dl.layer, nb, xb, lg, sel, ref_out)  # the allocating form first: it makes the tile-major copies both forms then read
        b.end()
        out.fill(np.full(nb * D, 0x7e00, np.uint16))  # NaN everywhere: every element must be written
        ok = gpu.L.qw_path_gg_moe_noalloc(gpu.g, D, I, E, K, C.byref(W), nb, devptr(gpu, xb), devptr(gpu, out), None)
        assert ok, gpu.last_error()
        gpu.L.qw_gpu_empty_commit_latency(gpu.g, None, 1)  # drains the stream the call launched on
        got, ref = out.read(dtype=np.uint16), ref_out.read(dtype=np.uint16)
        assert np.array_equal(got, ref), nb
        lgh = lg.view(np.float32)[:nb * (E + 1)].reshape(nb, E + 1)
        assert maxrel(got.view(np.float16).reshape(nb, D), oracle.moe_layer_f64(m, lgh, x)) <= 2e-3
        for bb in (xb, lg, sel, ref_out, out):
            bb.free()
    dl.free()
    path.close()


def test_no_alloc_refuses_what_the_scratch_cannot_hold(gpu):
    W = QwMoeWeightsDev()
    one = gpu.buf(64, device_only=True)
    p = devptr(gpu, one)
    for args in ((4096, 512, 64, 10, 4), (2048, 1024, 64, 10, 4), (2048, 512, 2048, 10, 4), (2048, 512, 64, 32, 4), (2048, 512, 64, 10, 17), (2048, 512, 64, 10, 0)):
        D, I, E, K, nb = args
        assert not gpu.L.qw_path_gg_moe_noalloc(gpu.g, D, I, E, K, C.byref(W), nb, p, p, None), args
    one.free()
