"""GPU parity of the quantized decode path against the CPU oracle, through the C interface (include/gpu.h and
include/qw_path.h). Bars: dequantized values bit-exact; matvec and MoE outputs max|err| / max|ref| <= 2e-3 against
the float64 oracle; router top-k indices identical."""
import os

import numpy as np
import pytest

import qwental_amd as q
from qwental_amd import synth
from helpers import DeviceLayer, gpu_dq_rows, maxrel, run_moe

pytestmark = pytest.mark.gpu
TOL = 2e-3  # max-rel-err bound for matvec and MoE outputs (float accumulation), as the benchmark contract states


# ---------------------------------------------------------------- dequantisation: bit-exact
@pytest.mark.parametrize("ftype,K,rows", [(21, 2048, 8), (21, 256, 3), (21, 512, 64), (8, 2048, 8), (8, 32, 5), (8, 512, 64)])
def test_dq_bit_exact(gpu, oracle, ftype, K, rows):
    rng = np.random.default_rng(100 + ftype + K)
    raw = synth.matrix(rng, ftype, rows, K).reshape(rows, -1)
    got = gpu_dq_rows(gpu, ftype, raw, K)
    want = oracle.dq_rows(ftype, raw, K)
    assert np.array_equal(got.view(np.uint32), want.view(np.uint32))


def test_dq_edge_blocks(gpu, oracle):
    """All-zero and all-ones bytes, denormal and largest scales, every scale nibble and high bit."""
    blocks = []
    for fill in (0x00, 0xFF, 0x55, 0xAA):
        for d in (0x0001, 0x3C00, 0x7BFF, 0x8001, 0x0400):
            b = np.full(110, fill, np.uint8)
            b[0], b[1] = d & 255, d >> 8
            blocks.append(b)
    raw = np.stack(blocks).reshape(len(blocks), 110)
    got = gpu_dq_rows(gpu, 21, raw, 256)
    want = oracle.dq_rows(21, raw, 256)
    assert np.array_equal(got.view(np.uint32), want.view(np.uint32))


def test_lookup_table_buffer(gpu, oracle):
    """gg_tab_init fills the callers' table buffer: the IQ3_S section must equal the oracle's pre-signed table."""
    ok, err = gpu.compile("#define IQ_DQ_ONLY\n#define E 512\n#define TOPK 10\n#define D 2048\n#define I 512\n#define NB 1\n#define GG_PART 0\n"
                          "#define moe_sel_gg moe_sel_gg_t\n#define gg_tab_init gg_tab_init_t\n")
    assert ok, err
    tab = gpu.buf(117760)
    b = gpu.batch()
    b.kernel(gpu.kernel("gg_tab_init_t"))
    b.buf(0, tab)
    b.dispatch(32, 1, 1, 256, 1, 1)
    b.end()
    got = tab.view(np.uint16)[49152 // 2:49152 // 2 + 8192 * 4]
    assert np.array_equal(got, oracle.tab_iq3ss().view(np.uint16).ravel())
    tab.free()


# ---------------------------------------------------------------- dense matvec
@pytest.mark.parametrize("ftype", [21, 8])
@pytest.mark.parametrize("nb", [1, 2, 4, 8, 16])
def test_qmv_parity(gpu, oracle, ftype, nb):
    N, K = 4096, 2048
    rng = np.random.default_rng(1)  # the seed of tools/ggmtest.py:42
    W = synth.matrix(rng, ftype, N, K)
    x = synth.activations(rng, nb, K)
    path = q.Path(gpu, 2048, 512, 512, 10, 16)
    wb, xb, yb = gpu.buf_from(W), gpu.buf_from(x), gpu.buf(nb * N * 4)
    b = gpu.batch()
    path.qmv_gg(b, q.Tensor(wb, ftype), N, K, xb, yb, nb, fout=True)
    b.end()
    y = yb.view(np.float32).reshape(nb, N).copy()
    ref = oracle.qmv(ftype, W, N, K, x, f64=True)
    assert maxrel(y, ref) <= TOL
    assert maxrel(y, ref) <= 1e-5  # float accumulation of exact products is far inside the bar
    assert maxrel(oracle.qmv(ftype, W, N, K, x), ref) <= TOL  # the float CPU path meets the same bar
    for bb in (wb, xb, yb):
        bb.free()
    path.close()


def test_qmv_rows_independent_of_batch(gpu):
    """Row i of a 16-wide call equals the single-activation call bit for bit (fixed per-token summation order)."""
    N, K = 512, 2048
    rng = np.random.default_rng(5)
    W = synth.matrix(rng, 21, N, K)
    x = synth.activations(rng, 16, K)
    path = q.Path(gpu, 2048, 512, 512, 10, 16)
    wb, xb, yb, y1 = gpu.buf_from(W), gpu.buf_from(x), gpu.buf(16 * N * 4), gpu.buf(N * 4)
    b = gpu.batch()
    path.qmv_gg(b, q.Tensor(wb, 21), N, K, xb, yb, 16)
    b.end()
    y16 = yb.view(np.float32).reshape(16, N).copy()
    for t in (0, 7, 15):
        b = gpu.batch()
        path.qmv_gg(b, q.Tensor(wb, 21), N, K, xb, y1, 1, xoff=t * K * 2)
        b.end()
        assert np.array_equal(y1.view(np.uint32)[:N], y16[t].view(np.uint32))
    for bb in (wb, xb, yb, y1):
        bb.free()
    path.close()


def test_qmv_ragged_rows_and_half_output(gpu, oracle):
    """N not a multiple of the 16-row tile; binary16 output."""
    N, K, nb = 1000 + 7, 512, 3
    rng = np.random.default_rng(9)
    W = synth.matrix(rng, 8, N, K)
    x = synth.activations(rng, nb, K)
    path = q.Path(gpu, 2048, 512, 512, 10, 16)
    wb, xb, yb = gpu.buf_from(W), gpu.buf_from(x), gpu.buf(nb * N * 2)
    b = gpu.batch()
    path.qmv_gg(b, q.Tensor(wb, 8), N, K, xb, yb, nb, fout=False)
    b.end()
    y = yb.view(np.float16)[:nb * N].reshape(nb, N).astype(np.float64)
    ref = oracle.qmv(8, W, N, K, x, f64=True)
    assert maxrel(y, ref) <= TOL
    for bb in (wb, xb, yb):
        bb.free()
    path.close()


@pytest.mark.parametrize("ftype", [21, 8])
@pytest.mark.parametrize("N,K,dev", [(640, 2560, True), (640, 2560, False), (200, 1536, True), (48, 1280, False)])
def test_qmv_k_cut_into_odd_parts(gpu, oracle, ftype, N, K, dev):
    """Few tiles and a chunk count of 5 or 3 (K = 2560 is the reference model's hidden size): a tile's K range is cut
    over 5, 3 or 6 waves. Against the float64 matvec; every row of the 16-token call equals the 1-token call."""
    nb = 16
    rng = np.random.default_rng(K + N + ftype)
    W = synth.matrix(rng, ftype, N, K)
    x = synth.activations(rng, nb, K)
    path = q.Path(gpu, 2048, 512, 512, 10, 16)
    wb, xb, yb, y1 = gpu.buf_from(W, device_only=dev), gpu.buf_from(x), gpu.buf(nb * N * 4), gpu.buf(N * 4)
    b = gpu.batch()
    path.qmv_gg(b, q.Tensor(wb, ftype), N, K, xb, yb, nb, fout=True)
    assert b.end() >= 0, gpu.last_error()
    y = yb.view(np.float32)[:nb * N].reshape(nb, N).copy()
    assert maxrel(y, oracle.qmv(ftype, W, N, K, x, f64=True)) <= 1e-5
    b = gpu.batch()
    path.qmv_gg(b, q.Tensor(wb, ftype), N, K, xb, y1, 1, xoff=5 * K * 2)
    assert b.end() >= 0, gpu.last_error()
    assert np.array_equal(y1.view(np.uint32)[:N], y[5].view(np.uint32))
    for bb in (wb, xb, yb, y1):
        bb.free()
    path.close()


def test_bad_calls_fail_without_launching(gpu):
    """Undersized buffers, unknown formats and unknown kernels are refused on the host."""
    ok, err = gpu.compile("#define IQ_DQ_ONLY 1\n#define DQ_TEST 10\n")  # Q2_K
    assert not ok and "10" in err
    ok, err = gpu.compile("#define IQ_DQ_ONLY 1\n#define qmv_gg q_bad\n#define GF 21\n#define KD 2048\n#define RB 881\n#define NB 1\n")
    assert not ok
    assert not gpu.kernel("no_such_kernel")
    head = "#define IQ_DQ_ONLY\n#define E 512\n#define TOPK 10\n#define D 2560\n#define I 640\n#define NB 8\n#define GG_PART 3\n#define DSGN 4\n"
    ok, err = gpu.compile(head + "#define FD 21\n#define moe_dn_gg dn_bad\n#define moe_cmb_gg cmb_bad\n")  # IQ3_S rows cannot be 640 long
    assert not ok and "640" in err
    ok, err = gpu.compile(head + "#define FD 20\n#define moe_dn_gg dn_640_nl\n#define moe_cmb_gg cmb_640_nl\n")
    assert ok, err
    path = q.Path(gpu, 2048, 512, 512, 10, 16)
    W = gpu.buf(100)  # far too small for 4096 rows
    x, y = gpu.buf(4096), gpu.buf(4096 * 4)
    b = gpu.batch()
    path.qmv_gg(b, q.Tensor(W, 21), 4096, 2048, x, y, 1)
    assert b.end(check=False) < 0
    assert "needs" in gpu.last_error()
    for bb in (W, x, y):
        bb.free()
    path.close()


# ---------------------------------------------------------------- router and selection
@pytest.mark.parametrize("nb", [1, 3, 8, 16])
def test_router_and_selection(gpu, oracle, nb):
    D, E, K = 2048, 512, 10
    rng = np.random.default_rng(20 + nb)
    m = synth.moe_layer(rng, D, 512, E, experts=1)
    x = synth.activations(rng, nb, D)
    path = q.Path(gpu, D, 512, E, K, 16)
    dl = DeviceLayer(gpu, m)
    xb, lg = gpu.buf_from(x), gpu.buf(path.logits_bytes(nb))
    b = gpu.batch()
    path.gg_router(b, dl.layer, nb, xb, lg)
    b.end()
    got = lg.view(np.float32).reshape(nb, E + 1).copy()
    ref = oracle.router(m["Wr"], m["wsg"], x)
    assert maxrel(got, ref) <= 1e-5
    # identical top-k: the rank-10 / rank-11 gap of this seeded input is far above the float error of the logits
    srt = -np.sort(-ref[:, :E].astype(np.float64), axis=1)
    assert (srt[:, K - 1] - srt[:, K]).min() > 100 * np.abs(got - ref).max()
    assert np.array_equal(oracle.topk_ids(got, K), oracle.topk_ids(ref, K))
    for bb in (xb, lg):
        bb.free()
    dl.free()
    path.close()


def _select_on_gpu(gpu, logits, nb, E, K):
    nbv = 1 if nb <= 1 else 2 if nb <= 2 else 4 if nb <= 4 else 8 if nb <= 8 else 16
    gnb = 8 if nbv <= 8 else 16
    name = "moe_sel_gg_s%d_%d_%d" % (nbv, E, K)
    ok, err = gpu.compile("#define IQ_DQ_ONLY\n#define E %d\n#define TOPK %d\n#define D 2048\n#define I 512\n#define NB %d\n#define GG_PART 0\n"
                          "#define moe_sel_gg %s\n#define gg_tab_init gti_%s\n" % (E, K, nbv, name, name))
    assert ok, err
    lg = gpu.buf_from(logits)
    from oracle import oracle as o
    sel = gpu.buf(o.sel_bytes(gnb, K))
    b = gpu.batch()
    b.kernel(gpu.kernel(name))
    b.buf(0, lg)
    b.buf(1, sel)
    b.bytes(2, np.array([nb], np.uint32))
    b.dispatch(1, 1, 1, 32 * nb, 1, 1)
    b.end()
    raw = sel.view(np.uint8).copy()
    lg.free()
    sel.free()
    return o.Sel(raw, gnb, K)


def _check_sel(got, want, nb, K):
    assert got.U == want.U
    assert np.array_equal(got.ue, want.ue) and np.array_equal(got.mask, want.mask) and np.array_equal(got.slot, want.slot)
    assert np.allclose(got.w[:nb], want.w[:nb], rtol=2e-6, atol=1e-7)
    assert int(sum(bin(int(v)).count("1") for v in got.mask)) == nb * K


@pytest.mark.parametrize("nb", [1, 2, 5, 8, 11, 16])
def test_selection_matches_oracle(gpu, oracle, nb):
    E, K = 512, 10
    rng = np.random.default_rng(40 + nb)
    logits = rng.normal(0, 1, (nb, E + 1)).astype(np.float32)
    got = _select_on_gpu(gpu, logits, nb, E, K)
    _check_sel(got, oracle.select(logits, K, got.gnb), nb, K)


def test_selection_ties_and_duplicates(gpu, oracle):
    """Exact ties go to the lowest expert index; identical tokens share every expert (dedupe), the way the
    reference forces it with duplicated activations (src/engine.c:7958-7961)."""
    E, K, nb = 512, 10, 8
    rng = np.random.default_rng(77)
    logits = np.round(rng.normal(0, 1, (nb, E + 1)) * 4).astype(np.float32) / 4  # heavy ties
    logits[3] = logits[0]
    logits[5] = logits[1]
    logits[6, :E] = 0.0  # all equal: picks 0..9
    got = _select_on_gpu(gpu, logits, nb, E, K)
    want = oracle.select(logits, K, 8)
    _check_sel(got, want, nb, K)
    assert list(want.ue[want.mask == (want.mask | (1 << 6))][:0]) == []  # (readability: token 6 picks experts 0..9)
    ids = oracle.topk_ids(logits, K)
    assert list(ids[6]) == list(range(10))
    gap = np.nextafter(np.float32(1.0), np.float32(2.0))
    l2 = np.zeros((1, E + 1), np.float32)
    l2[0, 100:111] = 1.0
    l2[0, 110] = gap  # one ulp above ten equal values: rank 0 is 110, then 100..108
    got = _select_on_gpu(gpu, l2, 1, E, K)
    assert list(got.ue[:10]) == [110] + list(range(100, 109))


@pytest.mark.parametrize("E", [64, 128, 256, 512, 1024])
def test_selection_close_values_and_every_expert_count(gpu, oracle, E):
    """Hundreds of logits that agree in their upper 16 bits (the selection's first bound leaves more than 64
    candidates and has to be refined), descending and ascending runs, for every expert count with a register build."""
    K, nb = 10, 16
    rng = np.random.default_rng(500 + E)
    logits = rng.normal(0, 1, (nb, E + 1)).astype(np.float32)
    n = min(E, 200)
    logits[:2] *= np.float32(0.1)  # the rest of rows 0 and 1 stays below the runs
    logits[0, :n] = (1.0 + np.arange(n) * 2.0 ** -20).astype(np.float32)          # ascending by one part in 2^20
    logits[1, :n] = (1.0 + np.arange(n)[::-1] * 2.0 ** -20).astype(np.float32)    # descending
    logits[2, :E] = -np.float32(2.0) - rng.permutation(E).astype(np.float32) * np.float32(2.0 ** -18)  # all negative, all close
    logits[3, :E] = np.float32(0.5)                                               # all equal
    logits[3, E // 2:E // 2 + 3] = np.float32(0.75)
    logits[4, :E] = np.repeat(rng.normal(0, 1, E // 8).astype(np.float32), 8)     # every value eight times
    got = _select_on_gpu(gpu, logits, nb, E, K)
    _check_sel(got, oracle.select(logits, K, got.gnb), nb, K)
    ids = oracle.topk_ids(logits, K)
    assert list(ids[0]) == list(range(n - 1, n - 11, -1)) and list(ids[1]) == list(range(10))
    assert list(ids[3]) == [E // 2, E // 2 + 1, E // 2 + 2] + list(range(7))


@pytest.mark.parametrize("E,nb", [(64, 16), (512, 16), (1024, 16), (512, 11), (1024, 9), (256, 2)])
def test_selection_inside_the_gate_up_launch_on_crafted_logits(gpu, oracle, E, nb):
    """The gate/up launch makes the selection itself: eight of its twelve waves take the tokens (two a wave above eight
    tokens; with 1024 experts one a wave and a second pass), the other four copy the table and the activations. One-hot
    activations make the router's logits equal to chosen binary16 values, so the cases of the stand-alone selection's
    tests reach that code too: more than 64 equal keys at the bound (the repeated-maximum fallback), every value eight
    times, one-ulp ramps up and down, close negative values, zeros of both signs. The record must be the oracle's."""
    D, I, K = 512, 256, 10
    rng = np.random.default_rng(900 + E + nb)
    m = synth.moe_layer(rng, D, I, E)  # every expert's rows: any of them may be picked
    m["topk"] = K
    cols = rng.normal(0, 1, (nb, E)).astype(np.float16)
    n = min(E, 200)

    def put(t, v):
        if t < nb:
            cols[t] = np.asarray(v, np.float32).astype(np.float16)

    r = np.full(E, 0.5, np.float32)
    r[E // 2:E // 2 + 3] = 0.75
    put(0, r)                                                                        # all equal but three
    put(1, np.repeat(rng.normal(0, 1, E // 8).astype(np.float16).astype(np.float32), 8))  # every value eight times
    up = rng.normal(0, 0.1, E).astype(np.float32)
    up[:n] = 1.0 + np.arange(n) * 2.0 ** -10                                         # ascending by one binary16 ulp
    put(2, up)
    dn = rng.normal(0, 0.1, E).astype(np.float32)
    dn[:n] = 1.0 + np.arange(n)[::-1] * 2.0 ** -10                                   # descending
    put(3, dn)
    put(4, -2.0 - rng.permutation(E).astype(np.float32) * 2.0 ** -9 * (1024 // E))   # all negative, all close, all distinct
    z = np.zeros(E, np.float32)
    z[1::2] = -0.0
    z[[E // 3, E // 3 + 1]] = 2.0 ** -14
    put(5, z)                                                                        # zeros of both signs and two small values
    assert np.array_equal(cols.astype(np.float32).astype(np.float16), cols)
    m["Wr"][:, :nb] = cols.T
    x = np.zeros((nb, D), np.float16)
    x[np.arange(nb), np.arange(nb)] = 1.0                                           # logit[t][e] = Wr[e][t]
    path = q.Path(gpu, D, I, E, K, 16)
    dl = DeviceLayer(gpu, m)
    gpu.profile(True)
    out, lg, selraw, _ = run_moe(gpu, path, dl, x, nb)
    names = [nm for nm, _ in gpu.profile_entries()]
    gpu.profile(False)
    assert "qwk_select" not in names and any(nm.startswith("qwk_gu_") for nm in names), names
    assert np.array_equal(lg[:, :E], cols.astype(np.float32))
    gnb = 8 if nb <= 8 else 16
    _check_sel(oracle.Sel(selraw, gnb, K), oracle.select(lg, K, gnb), nb, K)
    ids = oracle.topk_ids(lg, K)
    assert list(ids[0]) == [E // 2, E // 2 + 1, E // 2 + 2] + list(range(7))
    if nb > 3:
        assert list(ids[2]) == list(range(n - 1, n - 11, -1)) and list(ids[3]) == list(range(10))
    assert maxrel(out, oracle.moe_layer_f64(m, lg, x)) <= TOL
    path.close()
    dl.free()


# ---------------------------------------------------------------- one MoE layer
@pytest.mark.parametrize("nb,fmt", [(1, 21), (3, 21), (8, 21), (16, 21), (8, 8), (16, 8)])
def test_moe_layer_parity(gpu, oracle, nb, fmt):
    D, I, E, K = 2048, 512, 64, 10  # 64 experts keep the host generator and the float64 oracle at seconds
    rng = np.random.default_rng(300 + nb + fmt)
    m = synth.moe_layer(rng, D, I, E, fgu=fmt, fd=fmt, fsh=fmt)
    m["topk"] = K
    x = synth.activations(rng, nb, D)
    path = q.Path(gpu, D, I, E, K, 16)
    dl = DeviceLayer(gpu, m)
    out, lg, selraw, _ = run_moe(gpu, path, dl, x, nb)
    gnb = 8 if nb <= 8 else 16
    # logits and identical indices
    ref_lg = oracle.router(m["Wr"], m["wsg"], x)
    assert maxrel(lg, ref_lg) <= 1e-5
    assert np.array_equal(oracle.topk_ids(lg, K), oracle.topk_ids(ref_lg, K))
    sel = oracle.Sel(selraw, gnb, K)
    _check_sel(sel, oracle.select(lg, K, gnb), nb, K)
    # outputs against the float64 layer driven by the device's logits
    ref = oracle.moe_layer_f64(m, lg, x)
    assert maxrel(out, ref) <= TOL
    # H (SwiGLU output) is stored as binary16 hi + lo planes: compare with the float oracle's H
    o32, H32, _ = oracle.moe_layer_f32(m, lg, x, gnb)
    nbv = 1 if nb <= 1 else 2 if nb <= 2 else 4 if nb <= 4 else 8 if nb <= 8 else 16
    Hraw = path.scratch(1).view(np.float16)
    plane = nbv * (K + 1) * I
    H = (Hraw[:nb * (K + 1) * I].astype(np.float32) + Hraw[plane:plane + nb * (K + 1) * I].astype(np.float32)).reshape(nb, K + 1, I)
    assert maxrel(H, H32) <= 1e-5
    assert maxrel(o32.astype(np.float64), ref) <= TOL
    dl.free()
    path.close()


@pytest.mark.parametrize("D,I,E,K,nb,fgu,fd,fsh,fshd,dev", [
    (2560, 512, 64, 10, 16, 21, 21, 21, 8, True),    # the widest staged activation row; shared down Q8_0; tile-major copies
    (1024, 256, 128, 8, 5, 21, 21, 21, 21, True),    # one IQ3_S block per down row
    (768, 768, 64, 4, 7, 21, 21, 21, 21, False),     # neither a multiple of 512: one block per chunk; I > 512: the any-shape down kernel
    (512, 1024, 32, 6, 12, 8, 8, 8, 8, False),       # Q8_0 throughout, long down rows
    (1536, 512, 256, 16, 16, 21, 8, 8, 21, True),    # sixteen picks per token; mixed formats per projection
    (256, 256, 1024, 10, 3, 21, 21, 21, 21, False),  # the smallest rows, the most experts
    (2048, 512, 48, 10, 9, 21, 21, 21, 21, True),    # an expert count without a register build of the selection
    (2560, 640, 64, 10, 16, 21, 20, 21, 20, True),   # the reference model's shape and routed formats (src/model.h:10-18, bench/moe_bw.c:16-24): IQ4_NL down rows of 640
    (2560, 640, 64, 10, 1, 21, 20, 21, 20, True),    # the same, one token
    (2560, 640, 64, 10, 7, 21, 20, 8, 8, False),     # IQ4_NL routed down beside a Q8_0 shared expert
    (2560, 640, 64, 10, 12, 21, 8, 21, 8, True),     # I = 640 with Q8_0 down rows
    (1024, 384, 32, 4, 5, 8, 20, 8, 20, False),      # I a multiple of 128 only
    (256, 640, 16, 1, 4, 8, 20, 8, 20, True),        # the narrowest layer, one pick per token, tile-major IQ4_NL rows
    (512, 1280, 16, 16, 3, 21, 20, 21, 20, True),    # IQ4_NL rows wider than the staged 640: the any-shape kernel; every expert picked
    (2560, 640, 512, 10, 16, 21, 20, 8, 8, True),    # 512 experts at the reference model's shape, Q8_0 shared expert
    # the other types the reference's kernels take for routed rows (kernels/moe_gg.metal:336-395): the kernels whose type is an argument
    (2048, 512, 64, 10, 16, 23, 23, 21, 21, True),   # IQ4_XS routed rows beside an IQ3_S shared expert
    (2560, 768, 64, 10, 9, 12, 12, 12, 12, True),    # Q4_K everywhere (the minimum term; shared gate/up through the multi-format matvec)
    (1024, 512, 32, 4, 5, 14, 14, 8, 14, False),     # Q6_K routed rows and shared down, Q8_0 shared gate/up
    (1536, 256, 48, 6, 13, 13, 13, 8, 8, True),      # Q5_K routed rows
    (768, 256, 16, 2, 3, 20, 20, 21, 21, False),     # IQ4_NL gate/up; D off the front launch's shapes: the shared IQ3_S gate/up rides in the routed launch
    (1280, 512, 32, 8, 2, 12, 23, 8, 8, False),      # Q4_K gate/up, IQ4_XS down, the Q8_0 shared gate/up in the routed launch
    (2048, 512, 64, 10, 8, 21, 14, 21, 13, True),    # IQ3_S gate/up (tile-major) with Q6_K down rows and a Q5_K shared down
    (2048, 512, 64, 10, 1, 23, 12, 23, 23, True),    # one token
])
def test_moe_layer_shapes(gpu, oracle, D, I, E, K, nb, fgu, fd, fsh, fshd, dev):
    """Shapes and format mixes off the benchmark's: every kernel variant the host can pick is reached by one of them."""
    rng = np.random.default_rng(D + I + E + K + nb)
    m = synth.moe_layer(rng, D, I, E, fgu=fgu, fd=fd, fsh=fsh, fshd=fshd)
    m["topk"] = K
    x = synth.activations(rng, nb, D)
    path = q.Path(gpu, D, I, E, K, 16)
    dl = DeviceLayer(gpu, m, device_only=dev)
    out, lg, selraw, _ = run_moe(gpu, path, dl, x, nb)
    gnb = 8 if nb <= 8 else 16
    ref_lg = oracle.router(m["Wr"], m["wsg"], x)
    assert maxrel(lg, ref_lg) <= 1e-5
    _check_sel(oracle.Sel(selraw, gnb, K), oracle.select(lg, K, gnb), nb, K)
    ref = oracle.moe_layer_f64(m, lg, x)
    assert np.isfinite(out.astype(np.float64)).all()
    assert maxrel(out, ref) <= TOL, maxrel(out, ref)
    dl.free()
    path.close()


@pytest.mark.parametrize("fgu,fd,fsh,fshd,D,want", [
    (23, 23, 21, 21, 2048, ("qwk_gu_rt", "qwk_dn_rt")),       # the shared gate/up in the front launch
    (12, 14, 8, 13, 1280, ("qwk_gu_rt_s8_c1", "qwk_dn_rt")),  # ... in the routed launch (D off the front launch's shapes)
    (21, 21, 21, 12, 2048, ("qwk_gu_f121_c2", "qwk_dn_rt")),  # only the shared down rows are of another type
    (20, 20, 21, 21, 768, ("qwk_gu_rt_s21_c1", "qwk_dn_rt")), # IQ4_NL routed down beside IQ3_S shared down: no build of their own
])
def test_types_without_a_build_of_their_own_take_the_argument_kernels(gpu, oracle, fgu, fd, fsh, fshd, D, want):
    """kernels/moe_gg.metal:336-395 of the reference: every pair of the seven quantised types is a layer it can run. The
    pairs off the fast builds go through qwk_gu_rt* / qwk_dn_rt (the type an argument); against the float64 layer."""
    I, E, K, nb = 512, 32, 6, 11
    rng = np.random.default_rng(fgu * 100 + fd + fshd)
    m = synth.moe_layer(rng, D, I, E, fgu=fgu, fd=fd, fsh=fsh, fshd=fshd)
    m["topk"] = K
    x = synth.activations(rng, nb, D)
    dl = DeviceLayer(gpu, m, device_only=True)
    path = q.Path(gpu, D, I, E, K, 16)
    gpu.profile(True)
    out, lg, _, _ = run_moe(gpu, path, dl, x, nb)
    names = [n for n, _ in gpu.profile_entries()]
    gpu.profile(False)
    assert all(w in names for w in want), names
    assert np.isfinite(out.astype(np.float64)).all()
    assert maxrel(out, oracle.moe_layer_f64(m, lg, x)) <= TOL
    dl.free()
    path.close()


def test_iq4_nl_down_in_the_any_shape_kernel(gpu, oracle):
    """IQ4_NL down rows normally take the range kernel (rows of up to 640 staged in LDS); wider rows, or
    QW_HIP_DN_ANY in the environment, take the any-shape kernel. Both against the float64 layer."""
    D, I, E, K, nb = 1024, 640, 32, 10, 6
    rng = np.random.default_rng(2020)
    m = synth.moe_layer(rng, D, I, E, fgu=21, fd=20, fsh=8, fshd=20)
    m["topk"] = K
    x = synth.activations(rng, nb, D)
    dl = DeviceLayer(gpu, m)  # host-shadowed buffers: no tile-major copies
    for env, want in ((None, "qwk_dnr_f20_c10_s20_c10"), ("1", "qwk_dn_f20_any_s20")):
        with gpu.switches(dn_any=env):
            path = q.Path(gpu, D, I, E, K, 16)
            gpu.profile(True)
            out, lg, _, _ = run_moe(gpu, path, dl, x, nb)
            names = [n for n, _ in gpu.profile_entries()]
            gpu.profile(False)
            assert want in names, names
            assert maxrel(out, oracle.moe_layer_f64(m, lg, x)) <= TOL
            path.close()
    dl.free()


@pytest.mark.parametrize("D,I,nb,fshd", [(2560, 640, 16, 20), (2560, 640, 2, 20), (1024, 640, 9, 8), (1024, 640, 5, 20)])
def test_iq4_nl_down_from_the_tile_major_copy(gpu, oracle, D, I, nb, fshd):
    """Device-only IQ4_NL down matrices with rows of 640 get a tile-major copy (the IQ3_S scheme); the layer from
    the copy equals the layer from the GGUF rows bit for bit (same products in the same order) and meets the float64 layer."""
    if os.environ.get("QW_HIP_REPACK") == "0":
        pytest.skip("tile-major copies are switched off in this environment")
    E, K = 32, 10
    rng = np.random.default_rng(3000 + D + I + nb)
    m = synth.moe_layer(rng, D, I, E, fgu=21, fd=20, fsh=8, fshd=fshd)
    m["topk"] = K
    x = synth.activations(rng, nb, D)
    outs = []
    try:
        for copies in (True, False):
            gpu.L.qw_hip_set_repack(gpu.g, copies)
            path = q.Path(gpu, D, I, E, K, 16)
            dl = DeviceLayer(gpu, m, device_only=True)
            before = gpu.L.qw_hip_packed_bytes(gpu.g)
            gpu.profile(True)
            out, lg, _, _ = run_moe(gpu, path, dl, x, nb)
            names = [n for n, _ in gpu.profile_entries()]
            gpu.profile(False)
            want = ("qwk_dnr_f120_c10", "qwk_dnc_f120_c10") if copies else ("qwk_dnr_f20_c10",)  # dnc: down + combine, one or two tokens
            assert any(n.startswith(want) for n in names), names
            if copies:  # the routed matrix, and the shared one when it is IQ4_NL too (the IQ3_S gate/up copies come on top)
                assert gpu.L.qw_hip_packed_bytes(gpu.g) - before >= (E + (fshd == 20)) * D * I // 32 * 18
            assert maxrel(out, oracle.moe_layer_f64(m, lg, x)) <= TOL
            outs.append(out)
            dl.free()
            path.close()
    finally:
        gpu.L.qw_hip_set_repack(gpu.g, True)
    assert np.array_equal(outs[0].view(np.uint16), outs[1].view(np.uint16))


@pytest.mark.parametrize("nb", [1, 16])
def test_repeated_step_replayed_as_a_graph(gpu, oracle, nb):
    """With graphs switched on, a step recorded again over the same buffers runs as a HIP graph from its second
    repetition on. Six steps with
    fresh activations each, eager work and synchronisations of the program between them (the reference run below):
    every one must equal the eager run bit for bit."""
    gpu.L.qw_hip_set_graphs(gpu.g, True)  # off by default
    D, I, E, K = 1024, 512, 32, 4
    rng = np.random.default_rng(4100 + nb)
    m = synth.moe_layer(rng, D, I, E)
    m["topk"] = K
    path = q.Path(gpu, D, I, E, K, 16)
    dl = DeviceLayer(gpu, m, device_only=True)
    xb, outs = gpu.buf(nb * D * 2), [gpu.buf(nb * D * 2) for _ in range(3)]
    lgs, sels = [gpu.buf(path.logits_bytes(nb)) for _ in range(3)], [gpu.buf(path.sel_bytes(nb)) for _ in range(3)]
    before = gpu.L.qw_hip_graph_launches(gpu.g)
    for step in range(6):
        x = synth.activations(rng, nb, D)
        xb.fill(x)
        b = gpu.batch()
        for i in range(3):  # three layers' worth of launches: long enough to be worth a graph
            path.gg_moe(b, dl.layer, nb, xb, lgs[i], sels[i], outs[i])
        assert b.end() >= 0, gpu.last_error()
        got = [o_.view(np.uint16)[:nb * D].copy() for o_ in outs]
        ref, _, _, _ = run_moe(gpu, path, dl, x, nb)  # fresh buffers: another sequence, launched eagerly
        assert all(np.array_equal(g_, ref.view(np.uint16).ravel()) for g_ in got), step
    gpu.L.qw_hip_set_graphs(gpu.g, os.environ.get("QW_HIP_GRAPH") == "1")
    assert gpu.L.qw_hip_graph_launches(gpu.g) - before >= 4  # steps 1 .. 5 of the fixed buffers at least
    for bb in [xb] + outs + lgs + sels:
        bb.free()
    dl.free()
    path.close()


def test_stack_flush_points_do_not_change_results(gpu, oracle):
    """A stack of layers in one batch with the recorded part submitted after chosen layers (the reference's vb_flush,
    src/engine.c:5997): the same results whatever the mask, and the GPU time still covers every segment."""
    from qwental_amd.gpu import QwBuf, QwMoeLayer
    D, I, E, K, nb, L = 1024, 512, 32, 4, 7, 5
    rng = np.random.default_rng(5150)
    ms = [synth.moe_layer(rng, D, I, E) for _ in range(L)]
    for m in ms:
        m["topk"] = K
    x = synth.activations(rng, nb, D)
    path = q.Path(gpu, D, I, E, K, 16)
    dls = [DeviceLayer(gpu, m, device_only=True) for m in ms]
    layers_c = (QwMoeLayer * L)(*[d.layer.c for d in dls])
    xb, out = gpu.buf_from(x), gpu.buf(nb * D * 2)
    lgs, sels = [gpu.buf(path.logits_bytes(nb)) for _ in range(L)], [gpu.buf(path.sel_bytes(nb)) for _ in range(L)]
    lg_c, sel_c = (QwBuf * L)(*[b_.c for b_ in lgs]), (QwBuf * L)(*[b_.c for b_ in sels])
    res = {}
    for mask in (0, 1, 0b1011, (1 << 64) - 1):
        path.set_flush(mask)
        b = gpu.batch()
        path.gg_moe_stack(b, layers_c, L, nb, xb, lg_c, sel_c, out)
        t = b.end()
        assert t > 0, gpu.last_error()
        res[mask] = (out.view(np.uint16)[:nb * D].copy(), [l_.view(np.uint32)[:nb * (E + 1)].copy() for l_ in lgs], t)
    ref = oracle.moe_layer_f64(ms[L - 1], res[0][1][L - 1].view(np.float32).reshape(nb, E + 1), x)  # out holds the last layer's
    assert maxrel(res[0][0].view(np.float16).reshape(nb, D), ref) <= TOL
    for mask in res:
        assert np.array_equal(res[mask][0], res[0][0]) and all(np.array_equal(a, b_) for a, b_ in zip(res[mask][1], res[0][1]))
    for bb in [xb, out] + lgs + sels:
        bb.free()
    for d in dls:
        d.free()
    path.close()


def test_moe_batched_equals_single(gpu):
    """Each row of a batched layer call equals the single-token call bit for bit (src/engine.c:7977-7987)."""
    D, I, E, K, nb = 2048, 512, 64, 10, 8
    rng = np.random.default_rng(11)
    m = synth.moe_layer(rng, D, I, E)
    x = synth.activations(rng, nb, D)
    x[5] = x[2]  # duplicated token: shared experts across rows
    path = q.Path(gpu, D, I, E, K, 16)
    dl = DeviceLayer(gpu, m)
    out, _, _, _ = run_moe(gpu, path, dl, x, nb)
    bad = 0
    for t in range(nb):
        o1, _, _, _ = run_moe(gpu, path, dl, x[t:t + 1], 1)
        bad += not np.array_equal(o1[0].view(np.uint16), out[t].view(np.uint16))
    assert bad == 0
    assert np.array_equal(out[5].view(np.uint16), out[2].view(np.uint16))
    dl.free()
    path.close()


@pytest.mark.parametrize("nb", [1, 2, 5, 16])
@pytest.mark.parametrize("D,I,fsg,fsu,fsd,fd", [
    (2560, 640, 12, 23, 20, 20),   # the formats of the reference model's layer (bench/moe_bw.c:19-24): Q4_K gate, IQ4_XS up, IQ4_NL down
    (2048, 512, 14, 13, 8, 21),    # Q6_K gate, Q5_K up beside IQ3_S routed rows and a Q8_0 shared down
    (1024, 256, 20, 30, 21, 21),   # IQ4_NL gate, bfloat16 up
    (768, 256, 13, 14, 8, 8),      # three chunks a row: the K range cut three ways
    (256, 256, 23, 12, 21, 21),    # one chunk a row: no cut, so the matvec and the SwiGLU stay two launches
])
def test_shared_expert_in_other_formats(gpu, oracle, nb, D, I, fsg, fsu, fsd, fd):
    """The shared expert's gate and up rows in the K-quant / IQ4 / plain formats (different ones for gate and up):
    the multi-format matvec and a SwiGLU launch stand in for the front launch's shared tiles. Output against the
    float64 layer; H of the shared expert against the float oracle's."""
    E, K = 32, 10
    rng = np.random.default_rng(1700 + nb + D + fsg + fsu)
    m = synth.moe_layer(rng, D, I, E, fgu=21, fd=fd, fsh=fsg, fshu=fsu, fshd=fsd)
    m["topk"] = K
    x = synth.activations(rng, nb, D)
    path = q.Path(gpu, D, I, E, K, 16)
    dl = DeviceLayer(gpu, m, device_only=True)
    gpu.profile(True)
    out, lg, selraw, _ = run_moe(gpu, path, dl, x, nb)
    names = [n for n, _ in gpu.profile_entries()]
    gpu.profile(False)
    # rows of several chunks: inside the front launch, behind the router's workgroups; a single chunk: matvec, then SwiGLU
    assert ("qwk_pre_w1_kq" in names and "qwk_pre_w1" not in names) or ("qwk_qmvm" in names and "qwk_sh_act" in names), names
    gnb = 8 if nb <= 8 else 16
    ref = oracle.moe_layer_f64(m, lg, x)
    assert np.isfinite(out.astype(np.float64)).all()
    assert maxrel(out, ref) <= TOL, maxrel(out, ref)
    _, H32, _ = oracle.moe_layer_f32(m, lg, x, gnb)
    nbv = 1 if nb <= 1 else 2 if nb <= 2 else 4 if nb <= 4 else 8 if nb <= 8 else 16
    Hraw = path.scratch(1).view(np.float16)
    plane = nbv * (K + 1) * I
    H = (Hraw[:nb * (K + 1) * I].astype(np.float32) + Hraw[plane:plane + nb * (K + 1) * I].astype(np.float32)).reshape(nb, K + 1, I)
    assert maxrel(H[:, K], H32[:, K]) <= 1e-5
    # with QW_HIP_SIDE=1 (and no profiling) the shared expert's launches run on a side stream beside the router and the routed gate/up: three layers
    # in one batch (three forks and joins), twice, against the same launches kept in line
    def three(side):
        with gpu.switches(side="1" if side else "0"):  # off by default
            xb = gpu.buf_from(x)
            lgs, sels, outs = [gpu.buf(path.logits_bytes(nb)) for _ in range(3)], [gpu.buf(path.sel_bytes(nb)) for _ in range(3)], [gpu.buf(nb * D * 2) for _ in range(3)]
            b = gpu.batch()
            for i in range(3):
                path.gg_moe(b, dl.layer, nb, xb, lgs[i], sels[i], outs[i])
            assert b.end() >= 0, gpu.last_error()
            res = [o_.view(np.uint16)[:nb * D].copy() for o_ in outs]
            for bb in [xb] + lgs + sels + outs:
                bb.free()
            return res
    inline = three(False)
    assert all(np.array_equal(r, out.view(np.uint16).ravel()) for r in inline)
    for _ in range(2):
        assert all(np.array_equal(r, inline[0]) for r in three(True))
    dl.free()
    path.close()


@pytest.mark.parametrize("nb,limit", [(1, 2), (2, 2), (3, 4), (4, 4)])
@pytest.mark.parametrize("fd,fshd,dev,I", [(21, 21, True, 512), (21, 8, True, 512), (8, 8, False, 512), (8, 8, True, 512), (20, 20, True, 640), (20, 8, True, 640)])
def test_down_and_combine_in_one_launch(gpu, oracle, nb, limit, fd, fshd, dev, I):
    """With a few tokens the down projection and the combine run as one launch (kernels/moe_gg.metal:639-663 in one
    pass). Its output, Pg and Psh must equal bit for bit what the two separate launches leave, and the output must meet
    the float64 layer."""
    if dev and fd != 8 and os.environ.get("QW_HIP_REPACK") == "0":
        pytest.skip("tile-major copies are switched off in this environment")
    D, E, K = 2048, 32, 10
    rng = np.random.default_rng(900 + nb + fd + fshd)
    m = synth.moe_layer(rng, D, I, E, fgu=21, fd=fd, fsh=21 if fshd == 21 else 8, fshd=fshd)
    m["topk"] = K
    x = synth.activations(rng, nb, D)
    if nb > 1:
        x[nb - 1] = x[0]  # two tokens on the same experts: one product serves both
    dl = DeviceLayer(gpu, m, device_only=dev)
    res = {}
    for lim in (0, limit):
        with gpu.switches(dnq_min=0, dnc_nb=lim):  # (the one-launch form by token shares would take these layers from two tokens on)
            path = q.Path(gpu, D, I, E, K, 16)
            gpu.profile(True)
            out, lg, _, _ = run_moe(gpu, path, dl, x, nb)
            names = [n for n, _ in gpu.profile_entries()]
            gpu.profile(False)
            res[lim] = (out, lg, path.scratch(2).view(np.float32)[:nb * D].copy(), path.scratch(3).view(np.float32)[:nb * K * D].copy(), names)
            path.close()
    a, b = res[0], res[limit]
    assert any(n.startswith("qwk_dnc_") for n in b[4]) and not any(n.startswith("qwk_dnc_") for n in a[4]), (a[4], b[4])
    assert np.array_equal(a[0].view(np.uint16), b[0].view(np.uint16))
    assert np.array_equal(a[2].view(np.uint32), b[2].view(np.uint32)) and np.array_equal(a[3].view(np.uint32), b[3].view(np.uint32))
    assert maxrel(b[0], oracle.moe_layer_f64(m, b[1], x)) <= TOL
    dl.free()


@pytest.mark.parametrize("nb", [2, 3, 5, 8, 9, 13, 16])
@pytest.mark.parametrize("fshd,I,E,K,D", [(21, 512, 64, 10, 2048), (8, 512, 64, 10, 2048), (21, 256, 16, 10, 2048), (21, 512, 64, 8, 1024), (8, 256, 32, 4, 2560)])
def test_down_and_combine_by_token_quarters(gpu, oracle, nb, fshd, I, E, K, D):
    """From two tokens on, down + combine run as one launch in which a workgroup owns one or two tiles of output rows and
    a share of the tokens, four at most (qwk_dnq_*). Output, Pg and Psh must equal bit for bit what the range-form down
    launch and the combine launch leave (QW_HIP_DNQ_MIN=0 and QW_HIP_DNC_NB=0), for token counts that split evenly over
    the two or four shares and that do not."""
    if os.environ.get("QW_HIP_REPACK") == "0":
        pytest.skip("tile-major copies are switched off in this environment")
    rng = np.random.default_rng(700 + nb + fshd + I + K)
    m = synth.moe_layer(rng, D, I, E, fgu=21, fd=21, fsh=21 if fshd == 21 else 8, fshd=fshd)
    m["topk"] = K
    x = synth.activations(rng, nb, D)
    x[nb - 1] = x[0]  # two tokens of different quarters on the same experts
    dl = DeviceLayer(gpu, m, device_only=True)
    res = {}
    for lim in (0, 2):
        with gpu.switches(dnc_nb=0, dnq_min=lim, fuse=0):  # (shapes of the fused layer launch would not reach qwk_dnq_*)
            path = q.Path(gpu, D, I, E, K, 16)
            gpu.profile(True)
            out, lg, _, _ = run_moe(gpu, path, dl, x, nb)
            names = [n for n, _ in gpu.profile_entries()]
            gpu.profile(False)
            res[lim] = (out, lg, path.scratch(2).view(np.float32)[:nb * D].copy(), path.scratch(3).view(np.float32)[:nb * K * D].copy(), names)
            path.close()
    a, b = res[0], res[2]
    assert any(n.startswith("qwk_dnq_") for n in b[4]) and "qwk_cmb" not in b[4] and "qwk_cmb" in a[4], (a[4], b[4])
    assert np.array_equal(a[0].view(np.uint16), b[0].view(np.uint16))
    assert np.array_equal(a[2].view(np.uint32), b[2].view(np.uint32)) and np.array_equal(a[3].view(np.uint32), b[3].view(np.uint32))
    assert maxrel(b[0], oracle.moe_layer_f64(m, b[1], x)) <= TOL
    dl.free()


@pytest.mark.parametrize("nb,valu", [(1, False), (3, False), (16, False), (1, True), (2, True), (4, True)])
def test_qmv_packed_and_valu_forms(gpu, oracle, nb, valu):
    """Weights in a device-only buffer take the tile-major copy; with QW_VALU in the block the VALU GEMV runs instead of
    the matrix-core kernel. Both against the float64 oracle."""
    if os.environ.get("QW_HIP_REPACK") == "0":
        pytest.skip("tile-major copies are switched off in this environment")
    N, K = 1024, 2048
    rng = np.random.default_rng(40 + nb)
    W = synth.matrix(rng, 21, N, K)
    x = synth.activations(rng, nb, K)
    rb = synth.row_bytes(21, K)
    name = "qmv_gg_t_n%d_%d" % (nb, valu)
    ok, err = gpu.compile("#define qmv_gg %s\n#define GF 21\n#define KD %d\n#define RB %d\n#define NB %d\n#define YT float\n%s" % (name, K, rb, nb, "#define QW_VALU 1\n" if valu else ""))
    assert ok, err
    wb, xb, yb = gpu.buf_from(W, device_only=True), gpu.buf_from(x), gpu.buf(nb * N * 4)
    before = gpu.L.qw_hip_packed_bytes(gpu.g)
    b = gpu.batch()
    b.kernel(gpu.kernel(name))
    b.buf(0, wb)
    b.buf(3, xb)
    b.buf(4, yb)
    b.bytes(5, np.array([N, K, N, 0], np.uint32))
    b.dispatch((N + 7) // 8, 1, 1, 256, 1, 1)
    assert b.end() >= 0, gpu.last_error()
    assert gpu.L.qw_hip_packed_bytes(gpu.g) == before + N // 16 * (K // 256) * 1792
    y = yb.view(np.float32)[:nb * N].reshape(nb, N)
    assert maxrel(y, oracle.qmv(21, W, N, K, x, f64=True)) <= 1e-5
    wb.free()  # drops the copy
    assert gpu.L.qw_hip_packed_bytes(gpu.g) == before
    for bb in (xb, yb):
        bb.free()


def test_packed_copy_follows_the_source(gpu, oracle):
    """Rewriting a weight buffer after its first use drops the tile-major copy: the next call sees the new bytes."""
    if os.environ.get("QW_HIP_REPACK") == "0":
        pytest.skip("tile-major copies are switched off in this environment")
    N, K, nb = 256, 512, 2
    rng = np.random.default_rng(77)
    x = synth.activations(rng, nb, K)
    rb = synth.row_bytes(21, K)
    ok, err = gpu.compile("#define qmv_gg qmv_gg_follow\n#define GF 21\n#define KD %d\n#define RB %d\n#define NB %d\n#define YT float\n" % (K, rb, nb))
    assert ok, err
    W0, W1 = synth.matrix(rng, 21, N, K), synth.matrix(rng, 21, N, K)
    wb, xb, yb = gpu.buf_from(W0, device_only=True), gpu.buf_from(x), gpu.buf(nb * N * 4)
    for W in (W0, W1):
        wb.fill(W)
        b = gpu.batch()
        b.kernel(gpu.kernel("qmv_gg_follow"))
        b.buf(0, wb)
        b.buf(3, xb)
        b.buf(4, yb)
        b.bytes(5, np.array([N, K, N, 0], np.uint32))
        b.dispatch((N + 7) // 8, 1, 1, 256, 1, 1)
        assert b.end() >= 0, gpu.last_error()
        assert maxrel(yb.view(np.float32)[:nb * N].reshape(nb, N), oracle.qmv(21, W, N, K, x, f64=True)) <= 1e-5
    for bb in (wb, xb, yb):
        bb.free()


def test_explicit_write_to_a_host_shadowed_buffer_survives_its_first_bind(gpu, oracle):
    """A new buffer with a host side is uploaded whole when it is first bound. Bytes put into it through qw_hip_buf_write
    (or from a file) before that must be what the kernel then reads: the explicit writes keep the host side in step."""
    N, K, nb = 4096, 2048, 2   # 3.6 MB of weights: more than the size that is uploaded at every submit anyway
    rng = np.random.default_rng(78)
    W = synth.matrix(rng, 21, N, K)
    x = synth.activations(rng, nb, K)
    rb = synth.row_bytes(21, K)
    ok, err = gpu.compile("#define qmv_gg qmv_gg_written\n#define GF 21\n#define KD %d\n#define RB %d\n#define NB %d\n#define YT float\n" % (K, rb, nb))
    assert ok, err
    import tempfile
    for how in ("write", "write_fd"):
        wb = gpu.buf(W.size + (5 << 20))  # host-shadowed, never touched through its host pointer
        assert wb.size > (4 << 20)
        src = np.ascontiguousarray(W)
        if how == "write":
            assert gpu.L.qw_hip_buf_write(wb.ref(), 0, src.ctypes.data, src.nbytes)
        else:
            with tempfile.NamedTemporaryFile() as f:
                f.write(src.tobytes())
                f.flush()
                fd = os.open(f.name, os.O_RDONLY)
                try:
                    assert gpu.L.qw_hip_buf_write_fd(wb.ref(), 0, fd, 0, src.nbytes)
                finally:
                    os.close(fd)
        xb, yb = gpu.buf_from(x), gpu.buf(nb * N * 4)
        b = gpu.batch()
        b.kernel(gpu.kernel("qmv_gg_written"))
        b.buf(0, wb)
        b.buf(3, xb)
        b.buf(4, yb)
        b.bytes(5, np.array([N, K, N, 0], np.uint32))
        b.dispatch((N + 7) // 8, 1, 1, 256, 1, 1)
        assert b.end() >= 0, gpu.last_error()
        assert maxrel(yb.view(np.float32)[:nb * N].reshape(nb, N), oracle.qmv(21, W, N, K, x, f64=True)) <= 1e-5, how
        for bb in (wb, xb, yb):
            bb.free()


@pytest.mark.parametrize("switch,shape,want", [
    ("QW_HIP_SPLIT_SELECT", (2048, 512, 64, 10, 16, 21, 21, 21, 21, None), "qwk_select"),                 # the selection as a launch of its own
    ("QW_HIP_SHARED_IN_GU", (2048, 512, 64, 10, 16, 21, 21, 21, 21, None), "qwk_gu_f121_c2_s121_c2"),    # shared gate/up inside the gate/up launch
    ("QW_HIP_NL_C4", (1024, 640, 32, 10, 6, 21, 20, 8, 20, None), "qwk_dnr_f20_c4_s20_c4"),              # IQ4_NL down in chunks of four blocks
    ("QW_HIP_NO_SWIGLU_MATVEC", (2560, 640, 32, 10, 4, 21, 20, 12, 20, 23), "qwk_sh_act"),               # shared gate/up: matvec, then SwiGLU
    ("QW_HIP_KQ_OWN_LAUNCH", (2560, 640, 32, 10, 9, 21, 20, 12, 20, 23), "qwk_qmvm_swiglu"),              # shared gate/up: a launch of its own beside the front launch
])
def test_measurement_switches_select_other_kernels_with_the_same_results(gpu, oracle, switch, shape, want):
    """The environment switches that qw_gpu_open / qw_hip_reload_switches read (include/qw_hip_ext.h) route a layer through kernels that other
    shapes reach by themselves; with a switch set the named kernel runs and the layer still meets the float64 oracle."""
    D, I, E, K, nb, fgu, fd, fsh, fshd, fshu = shape
    rng = np.random.default_rng(len(switch) + D)
    m = synth.moe_layer(rng, D, I, E, fgu=fgu, fd=fd, fsh=fsh, fshd=fshd, fshu=fshu)
    m["topk"] = K
    x = synth.activations(rng, nb, D)
    dl = DeviceLayer(gpu, m, device_only=switch != "QW_HIP_NL_C4")  # host-shadowed rows: no tile-major copy of the IQ4_NL matrix
    outs = {}
    for on in (False, True):
        with gpu.switches(**{switch[len("QW_HIP_"):].lower(): "1" if on else None}):
            path = q.Path(gpu, D, I, E, K, 16)
            gpu.profile(True)
            out, lg, _, _ = run_moe(gpu, path, dl, x, nb)
            names = [n for n, _ in gpu.profile_entries()]
            gpu.profile(False)
            assert (want in names) == on, (on, names)
            assert maxrel(out, oracle.moe_layer_f64(m, lg, x)) <= TOL
            outs[on] = out
            path.close()
    if switch in ("QW_HIP_SPLIT_SELECT", "QW_HIP_NO_SWIGLU_MATVEC", "QW_HIP_KQ_OWN_LAUNCH"):  # the same products in the same order (the shared gate/up inside
        # the gate/up launch adds a row's blocks one after the other, the front launch per chunk first)
        assert np.array_equal(outs[False].view(np.uint16), outs[True].view(np.uint16))
    dl.free()


def test_chained_layers_across_a_flush_keep_the_device_results(gpu, oracle):
    """Two layers in one batch, the first one's output the second one's input, with the recorded part submitted in
    between (qw_batch_flush) and every buffer host-visible: the second segment must read what the first one's kernels
    left in HBM, not the buffer's host side (still zero until the batch is waited for)."""
    D, I, E, K, nb = 1024, 512, 32, 4, 8
    rng = np.random.default_rng(77)
    # the first layer's output is a few hundred times larger than N(0, 1): the second layer's block scales are drawn that much
    # smaller, so that its binary16 output stays finite
    ma, mb = synth.moe_layer(rng, D, I, E), synth.moe_layer(rng, D, I, E, d_scale=synth.MOE_D_SCALE / 50)
    ma["topk"] = mb["topk"] = K
    x = synth.activations(rng, nb, D)
    path = q.Path(gpu, D, I, E, K, 16)
    da, db = DeviceLayer(gpu, ma), DeviceLayer(gpu, mb)
    xb, mid, out = gpu.buf_from(x), gpu.buf(nb * D * 2), gpu.buf(nb * D * 2)
    lgs, sels = [gpu.buf(path.logits_bytes(nb)) for _ in range(2)], [gpu.buf(path.sel_bytes(nb)) for _ in range(2)]
    for flush in (False, True):
        mid.view(np.uint16)[:] = 0
        b = gpu.batch()
        path.gg_moe(b, da.layer, nb, xb, lgs[0], sels[0], mid)
        if flush:
            b.flush()
        path.gg_moe(b, db.layer, nb, mid, lgs[1], sels[1], out)
        b.end()
        h = mid.view(np.float16)[:nb * D].reshape(nb, D).copy()
        assert maxrel(h, oracle.moe_layer_f64(ma, lgs[0].view(np.float32)[:nb * (E + 1)].reshape(nb, E + 1), x)) <= TOL
        lg1 = lgs[1].view(np.float32)[:nb * (E + 1)].reshape(nb, E + 1).copy()
        assert maxrel(lg1, oracle.router(mb["Wr"], mb["wsg"], h)) <= 1e-5, flush  # the second layer saw the first one's output
        got = out.view(np.float16)[:nb * D].reshape(nb, D)
        assert np.isfinite(got.astype(np.float64)).all() and np.abs(got.astype(np.float64)).max() > 0
        assert maxrel(got, oracle.moe_layer_f64(mb, lg1, h)) <= TOL, flush
    # the same across two batches, the first one submitted and not waited for when the second is submitted
    mid.view(np.uint16)[:] = 0
    b1 = gpu.batch()
    path.gg_moe(b1, da.layer, nb, xb, lgs[0], sels[0], mid)
    gpu.L.qw_batch_submit(b1.b)
    b2 = gpu.batch()
    path.gg_moe(b2, db.layer, nb, mid, lgs[1], sels[1], out)
    gpu.L.qw_batch_submit(b2.b)
    assert gpu.L.qw_batch_wait(b1.b) >= 0 and gpu.L.qw_batch_wait(b2.b) >= 0
    h = mid.view(np.float16)[:nb * D].reshape(nb, D).copy()
    lg1 = lgs[1].view(np.float32)[:nb * (E + 1)].reshape(nb, E + 1).copy()
    assert maxrel(lg1, oracle.router(mb["Wr"], mb["wsg"], h)) <= 1e-5
    assert maxrel(out.view(np.float16)[:nb * D].reshape(nb, D), oracle.moe_layer_f64(mb, lg1, h)) <= TOL
    for bb in [xb, mid, out] + lgs + sels:
        bb.free()
    da.free()
    db.free()
    path.close()
