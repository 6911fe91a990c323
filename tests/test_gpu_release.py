"""Keeping only the tile-major copies of the routed experts (qw_hip_buf_release_source, include/qw_hip_ext.h): the same
bits from the same dispatches, half the residency, and a clear refusal for anything that would need the freed bytes."""
import ctypes as C

import numpy as np
import pytest

from helpers import dq_define_block
from qwental_amd import synth
from qwental_amd.stack import MoeStack

pytestmark = pytest.mark.gpu


def test_release_keeps_results_and_refuses_the_rest(gpu):
    L = gpu.L
    stack = MoeStack(gpu, layers=2, nbmax=16, seed=9)
    x = gpu.buf_from(synth.activations(np.random.default_rng(3), 16, stack.D), device_only=True)
    w0 = stack.bufs[0]
    assert not L.qw_hip_buf_release_source(w0.ref())  # no tile-major copy yet: nothing is freed
    outs = {}
    for nb in (16, 5, 1):
        stack.step(x, nb)
        outs[nb] = stack.out.view(np.uint16)[:nb * stack.D].copy()
    packed = L.qw_hip_packed_bytes(gpu.g)
    freed = stack.release_sources()
    assert freed == sum(stack.bufs[3 * l].size for l in range(stack.L)) and L.qw_hip_packed_bytes(gpu.g) == packed
    assert 1.0 < packed / freed < 1.03  # the copies are the matrices' bytes plus the slabs' padding
    for nb in (16, 5, 1):  # range-form down and the fused down + combine both read the copies
        stack.step(x, nb)
        assert np.array_equal(stack.out.view(np.uint16)[:nb * stack.D], outs[nb])
    # what needs the freed bytes is refused, with a message, and nothing is launched
    assert not L.qw_hip_buf_release_source(w0.ref())
    assert L.qw_hip_buf_devptr(w0.ref()) is None
    assert not L.qw_hip_buf_upload(w0.ref(), 0, 16)
    tmp = np.zeros(64, np.uint8)
    assert not L.qw_hip_buf_read(w0.ref(), 0, tmp.ctypes.data, 64)
    ok, err = gpu.compile(dq_define_block(21))
    assert ok, err
    y = gpu.buf(2048 * 4)
    b = gpu.batch()
    b.kernel(gpu.kernel("dq_test"))
    b.buf(0, w0)
    b.buf(1, y)
    b.bytes(2, np.array([2048, 880], np.uint32))
    b.dispatch(1, 1, 1, 32, 1, 1)
    assert b.end(check=False) < 0 and "released" in gpu.last_error()
    # another shape over the same bytes has no copy: a matvec that would take the gate rows as one 512-row matrix
    from qwental_amd import Tensor
    yb = gpu.buf(512 * 4)
    b = gpu.batch()
    ok = True
    try:
        stack.path.qmv_gg(b, Tensor(w0, 21), 512, stack.D, x, yb, 1)
    except RuntimeError:
        ok = False
    assert b.end(check=False) < 0 or not ok
    assert "released" in gpu.last_error()
    stack.step(x, 16)  # and the layer still runs
    assert np.array_equal(stack.out.view(np.uint16)[:16 * stack.D], outs[16])
    for bb in (y, yb, x):
        bb.free()
    stack.free()


def test_release_waits_until_every_matrix_of_the_buffer_has_a_copy(gpu, oracle):
    """Two matrices in one buffer: with a tile-major copy of only the first, the release is refused (the second could never
    be dispatched again) and says why; once both have been through a dispatch it goes through and both still compute."""
    import qwental_amd as q
    from qwental_amd import Tensor
    from helpers import maxrel
    L = gpu.L
    N, K, nb = 512, 1024, 3
    rng = np.random.default_rng(31)
    Wa, Wb = synth.matrix(rng, 21, N, K), synth.matrix(rng, 21, N, K)
    x = synth.activations(rng, nb, K)
    wb = gpu.buf_from(np.concatenate([Wa.ravel(), Wb.ravel()]), device_only=True)
    xb, ya, yb = gpu.buf_from(x), gpu.buf(nb * N * 4), gpu.buf(nb * N * 4)
    path = q.Path(gpu, 2048, 512, 8, 2, 16)

    def run(which):
        b = gpu.batch()
        if which in ("a", "both"):
            path.qmv_gg(b, Tensor(wb, 21), N, K, xb, ya, nb)
        if which in ("b", "both"):
            path.qmv_gg(b, Tensor(wb, 21, Wa.size), N, K, xb, yb, nb)
        assert b.end() >= 0, gpu.last_error()

    run("a")
    assert not L.qw_hip_buf_release_source(wb.ref())
    assert "stand in for" in gpu.last_error()
    run("b")
    assert L.qw_hip_buf_release_source(wb.ref()), gpu.last_error()
    run("both")
    for y, W in ((ya, Wa), (yb, Wb)):
        assert maxrel(y.view(np.float32)[:nb * N].reshape(nb, N), oracle.qmv(21, W, N, K, x, f64=True)) <= 1e-5
    for bb in (wb, xb, ya, yb):
        bb.free()
    path.close()
