"""GPU parity of the other GGUF formats (Q4_K, Q5_K, Q6_K, IQ4_NL, IQ4_XS, binary16, bfloat16) through the C interface:
dequantized values bit-exact against the oracle (itself checked against the reference's compiled src/ggml_dq.c), the
dense matvec and the multi-matrix matvec (kernels/qmv_ggm.metal) within max|err| / max|ref| <= 2e-3 of float64."""
import os
import sys

import numpy as np
import pytest

import qwental_amd as q
from qwental_amd import synth
from helpers import gpu_dq_rows, maxrel

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.join(HERE, "golden"))
import gen  # noqa: E402

pytestmark = pytest.mark.gpu
TOL = 2e-3
FORMATS = [12, 13, 14, 20, 23, 1, 30]


def same_values(got, want):
    """Bit-exact, a zero of either sign taken as equal (0 * scale carries the scale's sign)."""
    g, w = got.view(np.uint32), want.view(np.uint32)
    return np.array_equal(np.where((g << 1) == 0, 0, g), np.where((w << 1) == 0, 0, w))


@pytest.mark.parametrize("ftype", FORMATS)
def test_dq_bit_exact(gpu, oracle, ftype):
    for K, rows, seed in ((2048, 8, 1), (256, 5, 2), (4096, 3, 3)):
        rng = np.random.default_rng(300 + ftype + seed)
        raw = synth.matrix(rng, ftype, rows, K).reshape(rows, -1)
        got = gpu_dq_rows(gpu, ftype, raw, K)
        want = oracle.dq_rows(ftype, raw, K)
        assert same_values(got, want), (ftype, K)
        assert np.isfinite(got).all()


def test_dq_fixture_and_hand_blocks(gpu):
    """The committed values of the reference's own ggml_dq.c, and the hand blocks."""
    g = np.load(os.path.join(HERE, "golden", "dq_formats.npz"), allow_pickle=False)
    for key in g.files:
        if key.startswith("expect_f"):
            ft, K = int(key.split("_")[1][1:]), int(key.split("_")[2][1:])
            raw = gen.blocks_fmt(500 + ft, ft, 6 * (K // gen.FORMATS[ft][0])).reshape(6, -1)
            if ft in (1, 30) and K % 32:
                continue
            assert same_values(gpu_dq_rows(gpu, ft, raw, K), g[key]), key
        elif key.startswith("hand_raw_f"):
            ft = int(key[len("hand_raw_f"):])
            exp = g["hand_expect_f%d" % ft]
            if exp.shape[1] % 32:
                continue  # the four-value bfloat16 hand row is shorter than a decoding unit
            assert same_values(gpu_dq_rows(gpu, ft, g[key], exp.shape[1]), exp), key


def test_dq_extreme_fields(gpu, oracle):
    """All-zero / all-ones payloads with the smallest, largest and negative scales."""
    for ft in (12, 13, 14, 20, 23):
        qb, bb, offs = gen.FORMATS[ft]
        blocks = []
        for fill in (0x00, 0xFF, 0x55, 0xAA, 0x80, 0x7F):
            for d in (0x0001, 0x3C00, 0x7BFF, 0x8001, 0xBC00):
                b = np.full(bb, fill, np.uint8)
                for off in offs:
                    b[off], b[off + 1] = d & 255, d >> 8
                blocks.append(b)
        n = len(blocks) // (256 // qb) * (256 // qb)
        raw = np.stack(blocks[:n]).reshape(-1, 256 // qb * bb)
        got = gpu_dq_rows(gpu, ft, raw, 256)
        want = oracle.dq_rows(ft, raw, 256)
        assert same_values(got, want), ft


@pytest.mark.parametrize("ftype", FORMATS)
@pytest.mark.parametrize("nb", [1, 5, 16])
def test_qmv_parity(gpu, oracle, ftype, nb):
    path = q.Path(gpu, 2048, 512, 512, 10, 16)
    # K = 2560 (the reference model's hidden size) and 1536: the K range of a tile is cut into 5 and 6 parts
    for N, K, fout in ((1000 + 7, 2048, True), (64, 4096, True), (48, 256, False), (640, 2560, True), (100, 1536, True)):
        rng = np.random.default_rng(1000 + ftype + N)
        W = synth.matrix(rng, ftype, N, K)
        x = synth.activations(rng, nb, K)
        wb, xb, yb = gpu.buf_from(W), gpu.buf_from(x), gpu.buf(nb * N * 4)
        b = gpu.batch()
        path.qmv_gg(b, q.Tensor(wb, ftype), N, K, xb, yb, nb, fout=fout)
        assert b.end() >= 0, gpu.last_error()
        y = yb.view(np.float32 if fout else np.float16)[:nb * N].reshape(nb, N).astype(np.float64)
        ref = oracle.qmv(ftype, W, N, K, x, f64=True)
        assert maxrel(y, ref) <= (1e-5 if fout else TOL), (ftype, N, K, maxrel(y, ref))
        for bb in (wb, xb, yb):
            bb.free()
    path.close()


@pytest.mark.parametrize("fmts,nb", [((12, 13, 14, 30), 8), ((23, 20, 1), 16), ((14,), 1), ((12, 12), 3)])
def test_multi_matrix_matvec(gpu, oracle, fmts, nb):
    """q / k / v / indexer style: several matrices of different formats and row counts over the same activations."""
    K = 2048
    Ns = [512 + 16 * 3, 256 + 5, 1024, 100][:len(fmts)]
    rng = np.random.default_rng(7 + len(fmts) + nb)
    Ws = [synth.matrix(rng, f, n, K) for f, n in zip(fmts, Ns)]
    x = synth.activations(rng, nb, K)
    path = q.Path(gpu, 2048, 512, 512, 10, 16)
    wbs = [gpu.buf_from(w) for w in Ws]
    ybs = [gpu.buf(nb * n * 4) for n in Ns]
    xb = gpu.buf_from(x)
    b = gpu.batch()
    path.qmv_ggm(b, [q.Tensor(wb, f) for wb, f in zip(wbs, fmts)], Ns, K, xb, ybs, nb)
    assert b.end() >= 0, gpu.last_error()
    for W, f, n, yb in zip(Ws, fmts, Ns, ybs):
        y = yb.view(np.float32)[:nb * n].reshape(nb, n)
        ref = oracle.qmv(f, W, n, K, x, f64=True)
        assert maxrel(y, ref) <= 1e-5, (f, maxrel(y, ref))
    # one matrix at a time gives the same bits: a row's result does not depend on what else the launch holds
    y1 = gpu.buf(nb * Ns[0] * 4)
    b = gpu.batch()
    path.qmv_gg(b, q.Tensor(wbs[0], fmts[0]), Ns[0], K, xb, y1, nb, fout=True)
    assert b.end() >= 0
    assert np.array_equal(y1.view(np.uint32)[:nb * Ns[0]], ybs[0].view(np.uint32)[:nb * Ns[0]])
    for bb in wbs + ybs + [xb, y1]:
        bb.free()
    path.close()


def test_matvec_rows_independent_of_batch(gpu):
    N, K = 256, 2048
    rng = np.random.default_rng(77)
    path = q.Path(gpu, 2048, 512, 512, 10, 16)
    for ftype in (12, 14, 23):
        W = synth.matrix(rng, ftype, N, K)
        x = synth.activations(rng, 16, K)
        wb, xb, yb, y1 = gpu.buf_from(W), gpu.buf_from(x), gpu.buf(16 * N * 4), gpu.buf(N * 4)
        b = gpu.batch()
        path.qmv_gg(b, q.Tensor(wb, ftype), N, K, xb, yb, 16)
        b.end()
        y16 = yb.view(np.float32).reshape(16, N).copy()
        for t in (0, 9, 15):
            b = gpu.batch()
            path.qmv_gg(b, q.Tensor(wb, ftype), N, K, xb, y1, 1, xoff=t * K * 2)
            b.end()
            assert np.array_equal(y1.view(np.uint32)[:N], y16[t].view(np.uint32))
        for bb in (wb, xb, yb, y1):
            bb.free()
    path.close()


@pytest.mark.parametrize("ftype", [20, 1, 30])
def test_matvec_short_rows_and_few_rows(gpu, oracle, ftype):
    """K that is a multiple of 32 but not of 256 (one decoding unit per chunk), fewer rows than a tile, one row."""
    path = q.Path(gpu, 2048, 512, 512, 10, 16)
    for N, K, nb in ((5, 96, 3), (1, 32, 1), (33, 1056, 16), (16, 4064, 2)):
        rng = np.random.default_rng(2000 + ftype + N + K)
        W = synth.matrix(rng, ftype, N, K)
        x = synth.activations(rng, nb, K)
        wb, xb, yb = gpu.buf_from(W), gpu.buf_from(x), gpu.buf(nb * N * 4)
        b = gpu.batch()
        path.qmv_gg(b, q.Tensor(wb, ftype), N, K, xb, yb, nb, fout=True)
        assert b.end() >= 0, gpu.last_error()
        y = yb.view(np.float32)[:nb * N].reshape(nb, N)
        ref = oracle.qmv(ftype, W, N, K, x, f64=True)
        assert maxrel(y, ref) <= 1e-5, (ftype, N, K, maxrel(y, ref))
        for bb in (wb, xb, yb):
            bb.free()
    path.close()


def test_multi_matrix_largest_k_and_bad_calls(gpu, oracle):
    """K = 4096 (the largest staged row), and the host checks of the multi-matrix launch."""
    K, nb = 4096, 4
    fmts, Ns = (14, 23), (48, 272)
    rng = np.random.default_rng(31)
    Ws = [synth.matrix(rng, f, n, K) for f, n in zip(fmts, Ns)]
    x = synth.activations(rng, nb, K)
    path = q.Path(gpu, 2048, 512, 512, 10, 16)
    wbs, ybs, xb = [gpu.buf_from(w) for w in Ws], [gpu.buf(nb * n * 4) for n in Ns], gpu.buf_from(x)
    b = gpu.batch()
    path.qmv_ggm(b, [q.Tensor(wb, f) for wb, f in zip(wbs, fmts)], list(Ns), K, xb, ybs, nb)
    assert b.end() >= 0, gpu.last_error()
    for W, f, n, yb in zip(Ws, fmts, Ns, ybs):
        assert maxrel(yb.view(np.float32)[:nb * n].reshape(nb, n), oracle.qmv(f, W, n, K, x, f64=True)) <= 1e-5
    # an output buffer too small for its matrix fails the batch before anything is launched
    small = gpu.buf(16)
    b = gpu.batch()
    path.qmv_ggm(b, [q.Tensor(wbs[0], fmts[0])], [Ns[0]], K, xb, [small], nb)
    assert b.end(check=False) < 0 and "needs" in gpu.last_error()
    # a weight buffer shorter than its rows
    b = gpu.batch()
    path.qmv_ggm(b, [q.Tensor(small, 14)], [Ns[0]], K, xb, [ybs[0]], nb)
    assert b.end(check=False) < 0
    ok, err = gpu.compile("#define qmv_ggm bad\n#define KD 8192\n#define NB 1\n#define NMAT 1\n#define GF0 12\n")
    assert not ok and "8192" in err
    for bb in wbs + ybs + [xb, small]:
        bb.free()
    path.close()


def test_large_q6k_matrix_from_its_tile_major_copy(gpu, oracle):
    """A Q6_K matrix of vocabulary size (the reference's lm_head, src/engine.c:658-704) is read from a tile-major copy made
    at its first use: the same bits as from the GGUF rows (copies switched off), through qmv_gg and as one of several
    matrices of qmv_ggm, and the copy is exactly the matrix's bytes."""
    N, K = 16384 + 32, 2048
    rng = np.random.default_rng(14)
    W = synth.matrix(rng, 14, N, K)
    path = q.Path(gpu, 2048, 512, 512, 10, 16)
    wb = gpu.buf_from(W, device_only=True)
    small = synth.matrix(rng, 12, 64, K)
    sb = gpu.buf_from(small, device_only=True)
    res = {}
    for copies in (False, True):
        gpu.L.qw_hip_set_repack(gpu.g, copies)
        before = gpu.L.qw_hip_packed_bytes(gpu.g)
        for nb in (1, 7, 16):
            x = synth.activations(np.random.default_rng(nb), nb, K)
            xb, yb, y2, ys = gpu.buf_from(x), gpu.buf(nb * N * 4), gpu.buf(nb * N * 4), gpu.buf(nb * 64 * 4)
            b = gpu.batch()
            path.qmv_gg(b, q.Tensor(wb, 14), N, K, xb, yb, nb)
            path.qmv_ggm(b, [q.Tensor(sb, 12), q.Tensor(wb, 14)], [64, N], K, xb, [ys, y2], nb)
            assert b.end() >= 0, gpu.last_error()
            y = yb.view(np.float32)[:nb * N].copy()
            assert np.array_equal(y.view(np.uint32), y2.view(np.uint32)[:nb * N])
            if copies:
                assert np.array_equal(y.view(np.uint32), res[nb].view(np.uint32))
            else:
                res[nb] = y
                if nb == 7:
                    assert maxrel(y.reshape(nb, N).astype(np.float64), oracle.qmv(14, W, N, K, x, f64=True)) <= 1e-5
            for bb in (xb, yb, y2, ys):
                bb.free()
        assert gpu.L.qw_hip_packed_bytes(gpu.g) - before == (W.nbytes if copies else 0)
    gpu.L.qw_hip_set_repack(gpu.g, True)
    for bb in (wb, sb):
        bb.free()
    path.close()
