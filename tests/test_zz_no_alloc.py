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


# (D, I, E, top-k, routed gate/up, routed down, shared gate, shared up, shared down, router type)
@pytest.mark.parametrize("shape", [(2048, 512, 64, 10, 21, 21, 21, 21, 21, 1), (2560, 640, 32, 10, 21, 20, 8, 8, 8, 1), (1024, 256, 128, 8, 8, 8, 8, 8, 8, 1),
                                   (2560, 640, 32, 10, 21, 20, 12, 23, 20, 1),    # shared gate/up in the K-quant / IQ4 family: the front launch that carries them
                                   (2048, 512, 64, 10, 21, 21, 21, 21, 21, 30),   # bfloat16 router
                                   (2560, 640, 32, 6, 21, 20, 12, 23, 20, 30),    # both: the shared gate/up as a launch of its own beside a bfloat16 router
                                   (2048, 512, 32, 8, 23, 14, 8, 8, 12, 1)])      # routed rows of the other types (the kernels whose type is an argument)
def test_no_alloc_layer_equals_the_allocating_entry_point(gpu, oracle, shape):
    D, I, E, K, fgu, fd, fsg, fsu, fsd, rt = shape
    rng = np.random.default_rng(D + E + fsg + rt)
    m = synth.moe_layer(rng, D, I, E, fgu=fgu, fd=fd, fsh=fsg, fshd=fsd, fshu=fsu)
    m["topk"] = K
    if rt == 30:
        m["Wr"], m["wsg"] = synth.to_bf16(m["Wr"]), synth.to_bf16(m["wsg"])
    dl = DeviceLayer(gpu, m, router_type=rt, device_only=True)
    path = q.Path(gpu, D, I, E, K, 16, device_scratch=True)
    W = QwMoeWeightsDev(*[devptr(gpu, dl.bufs[k]) for k in ("Wr", "wsg", "Wg", "Wu", "Wd", "Wsg", "Wsu", "Wsd")], rt, fgu, fd, fsg, fsu, fsd)
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


def test_no_alloc_without_a_tile_major_copy(gpu, oracle):
    """No allocating call before it, copies switched off: the entry point reads the GGUF rows directly (it never makes a
    copy itself) and must meet the float64 layer; the allocating entry point, then also without copies, gives the same bits."""
    D, I, E, K, nb = 2048, 512, 32, 10, 7
    rng = np.random.default_rng(909)
    m = synth.moe_layer(rng, D, I, E)
    m["topk"] = K
    gpu.L.qw_hip_set_repack(gpu.g, False)
    try:
        dl = DeviceLayer(gpu, m, device_only=True)
        W = QwMoeWeightsDev(*[devptr(gpu, dl.bufs[k]) for k in ("Wr", "wsg", "Wg", "Wu", "Wd", "Wsg", "Wsu", "Wsd")], 1, 21, 21, 21, 21, 21)
        x = synth.activations(rng, nb, D)
        xb, out = gpu.buf_from(x, device_only=True), gpu.buf(nb * D * 2, device_only=True)
        before = gpu.L.qw_hip_packed_bytes(gpu.g)
        out.fill(np.full(nb * D, 0x7e00, np.uint16))
        assert gpu.L.qw_path_gg_moe_noalloc(gpu.g, D, I, E, K, C.byref(W), nb, devptr(gpu, xb), devptr(gpu, out), None), gpu.last_error()
        gpu.L.qw_gpu_empty_commit_latency(gpu.g, None, 1)
        assert gpu.L.qw_hip_packed_bytes(gpu.g) == before
        got = out.read(dtype=np.uint16)
        path = q.Path(gpu, D, I, E, K, 16, device_scratch=True)
        lg, sel, ref_out = gpu.buf(path.logits_bytes(nb)), gpu.buf(path.sel_bytes(nb)), gpu.buf(nb * D * 2, device_only=True)
        b = gpu.batch()
        path.gg_moe(b, dl.layer, nb, xb, lg, sel, ref_out)
        b.end()
        assert np.array_equal(got, ref_out.read(dtype=np.uint16))
        lgh = lg.view(np.float32)[:nb * (E + 1)].reshape(nb, E + 1)
        assert maxrel(got.view(np.float16).reshape(nb, D), oracle.moe_layer_f64(m, lgh, x)) <= 2e-3
        for bb in (xb, out, lg, sel, ref_out):
            bb.free()
        dl.free()
        path.close()
    finally:
        gpu.L.qw_hip_set_repack(gpu.g, True)
