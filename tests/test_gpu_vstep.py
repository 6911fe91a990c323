"""The ragged step through the C entry point qw_path_par_vstep (the caller contract of src/engine.c:8783-8814, 9138-9161):
slot i brings n[i] rows, the planner cuts the rows into groups of at most 16, every group runs the layer, the measured
times go back into the planner's table."""
import ctypes as C

import numpy as np
import pytest

import qwental_amd as q
from helpers import DeviceLayer, maxrel, run_moe
from qwental_amd import synth

pytestmark = pytest.mark.gpu
TOL = 2e-3
D, I, E, K = 1024, 512, 64, 4


@pytest.fixture(scope="module")
def layer(gpu):
    rng = np.random.default_rng(915)
    m = synth.moe_layer(rng, D, I, E)
    m["topk"] = K
    dl = DeviceLayer(gpu, m, device_only=True)
    path = q.Path(gpu, D, I, E, K, 16, device_scratch=True)
    yield m, dl, path
    dl.free()
    path.close()


def test_ragged_step_rows_against_the_oracle_and_the_one_token_call(gpu, oracle, layer):
    m, dl, path = layer
    rng = np.random.default_rng(7)
    n = rng.integers(1, 5, 16)  # sixteen slots with one to four rows each
    R = int(n.sum())
    x = synth.activations(rng, R, D)
    xb, ob = gpu.buf_from(x), gpu.buf(R * D * 2)
    par = q.Par()
    seen = set()
    for call in range(4):
        info = path.par_vstep(par, dl.layer, n, xb, ob)
        groups = list(info.groups[:info.ngroups])
        assert info.rows == R and sum(groups) == R and max(groups) <= 16 and min(groups) >= 1
        assert list(info.r0[:16]) == np.concatenate([[0], np.cumsum(n)[:-1]]).tolist()  # src/engine.c:9150-9161
        if call == 0:  # nothing measured yet: every size costs nothing and the larger group wins
            assert groups == [16] * (R // 16) + ([R % 16] if R % 16 else [])
        seen.update(groups)  # later cuts try sizes that were never measured (they count as free, src/engine.c:8787)
    out = ob.view(np.float16)[:R * D].reshape(R, D).copy()
    ref = oracle.moe_layer_f64(m, oracle.router(m["Wr"], m["wsg"], x), x)
    assert maxrel(out, ref) <= TOL
    for r in (0, 15, 16, R - 1):  # a row of a group is the one-token call, bit for bit
        one, _, _, _ = run_moe(gpu, path, dl, x[r:r + 1], 1)
        assert np.array_equal(one.view(np.uint16).ravel(), out[r].view(np.uint16)), r
    # the measured times arrived in the table (the first sample of a size is dropped)
    assert par.group_cost(16) > 0 and par.cost(R) > 0 and len(seen) >= 2
    assert info.gpu_ms > 0 and info.wall_ms >= info.gpu_ms * 0.5
    par.free()
    xb.free()
    ob.free()


def test_the_cut_follows_the_table_and_rows_do_not_depend_on_it(gpu, oracle, layer):
    m, dl, path = layer
    rng = np.random.default_rng(8)
    n = [8, 1, 7, 16]  # 32 rows
    R = sum(n)
    x = synth.activations(rng, R, D)
    xb, oa, ob = gpu.buf_from(x), gpu.buf(R * D * 2), gpu.buf(R * D * 2)
    fresh = q.Par()
    a = path.par_vstep(fresh, dl.layer, n, xb, oa)
    assert list(a.groups[:a.ngroups]) == [16, 16]
    table = q.Par()  # groups of 16 measured slow, groups of 8 fast: the cut becomes four groups of 8
    for b_, ms in ((16, 10.0), (8, 1.0), (4, 0.9), (1, 0.8)):
        table.observe(b_, ms)
        table.observe(b_, ms)
    for b_ in range(1, 17):  # every other size measured too, on the expensive side (a size never measured counts as free)
        if b_ not in (16, 8, 4, 1):
            table.observe(b_, 5.0)
            table.observe(b_, 5.0)
    b = path.par_vstep(table, dl.layer, n, xb, ob)
    assert list(b.groups[:b.ngroups]) == [8, 8, 8, 8]
    assert np.array_equal(oa.view(np.uint16), ob.view(np.uint16))  # the same rows, whatever the cut
    fresh.free()
    table.free()
    for bb in (xb, oa, ob):
        bb.free()


def test_ragged_step_refuses_bad_counts(gpu, layer):
    m, dl, path = layer
    par = q.Par()
    xb, ob = gpu.buf(64 * D * 2), gpu.buf(64 * D * 2)
    for n in ([1, 0, 3], [16] * 5, [65]):
        na = (C.c_int * len(n))(*n)
        assert not gpu.L.qw_path_par_vstep(path.p, par.p, C.byref(dl.layer.c), na, len(n), xb.ref(), ob.ref(), None), n
    small = gpu.buf(4 * D * 2)  # fewer rows than the counts ask for
    na = (C.c_int * 2)(3, 3)
    assert not gpu.L.qw_path_par_vstep(path.p, par.p, C.byref(dl.layer.c), na, 2, small.ref(), ob.ref(), None)
    par.free()
    for bb in (xb, ob, small):
        bb.free()
