"""GGUF files through the reader and the residency of include/qw_gguf.h on the GPU: the bytes in HBM are the bytes of
the file (bit-exact), small float tensors are converted as the reference converts them (src/gguf.c:444-503), a layer
taken from the files computes what the same bytes compute when handed over directly (bit-identical) and what the
float64 oracle computes (max|err| / max|ref| <= 2e-3, top-k indices identical), and a resident tensor dequantizes
bit-exactly (the flow of the reference's tools/dqtest.c on a tensor of a file)."""
import ctypes as C
import os

import numpy as np
import pytest

import qwental_amd as q
from oracle import gguf_file as gf
from qwental_amd import gguf_writer as gw
from qwental_amd import synth
from helpers import DeviceLayer, dq_define_block, maxrel, run_moe

pytestmark = pytest.mark.gpu
TOL = 2e-3
D, I, E, K = 2048, 512, 64, 10
LAYER = 5


def bf16_exact(a):
    """float32 values with the low 16 bits cleared (exact in BF16), and their BF16 bit patterns."""
    u = np.ascontiguousarray(a, np.float32).view(np.uint32) & np.uint32(0xffff0000)
    return u.view(np.float32), (u >> 16).astype(np.uint16)


def write_model(tmp, rng, router_type=30):
    """A two-shard model: layer LAYER's MoE tensors (router BF16, gate vector F32), an lm_head (Q6_K), an embedding that
    stays in the file, and small tensors of every conversion kind."""
    m = synth.moe_layer(rng, D, I, E)
    m["topk"] = K
    wr32, wr_bits = bf16_exact(rng.normal(0.0, 0.02, (E, D)))
    wg32, wg_bits = bf16_exact(rng.normal(0.0, 0.02, D))
    m["Wr"], m["wsg"] = wr_bits, wg_bits
    p = "blk.%d." % LAYER
    router_bytes = wr_bits if router_type == 30 else wr32.astype(np.float16)
    lm = synth.matrix(rng, 14, 1000, D)
    emb = synth.matrix(rng, 8, 64, D)
    dt_bias = rng.normal(0, 1, 48).astype(np.float32)                 # not exact in BF16: stays F32
    ssm_norm = rng.normal(0, 1, 128).astype(np.float16)               # F16 in the file, not exact in BF16: F32
    conv, _ = bf16_exact(rng.normal(0, 1, (4, 96)))                   # exact: BF16
    q_norm, _ = bf16_exact(rng.normal(0, 1, 128))                     # a norm weight is kept F32 even when exact
    shard1 = [(p + "ffn_gate_exps.weight", 21, [D, I, E], m["Wg"]), (p + "ffn_up_exps.weight", 21, [D, I, E], m["Wu"]),
              (p + "ffn_gate_inp.weight", router_type, [D, E], router_bytes), (p + "ffn_gate_inp_shexp.weight", 0, [D], wg32),
              (p + "ssm_dt.bias", 0, [48], dt_bias), (p + "ssm_norm.weight", 1, [128], ssm_norm), ("token_embd.weight", 8, [D, 64], emb)]
    shard2 = [(p + "ffn_down_exps.weight", 21, [I, D, E], m["Wd"]), (p + "ffn_gate_shexp.weight", 21, [D, I], m["Wsg"]),
              (p + "ffn_up_shexp.weight", 21, [D, I], m["Wsu"]), (p + "ffn_down_shexp.weight", 21, [I, D], m["Wsd"]),
              ("output.weight", 14, [D, 1000], lm), (p + "ssm_conv1d.weight", 0, [96, 4], conv), (p + "attn_q_norm.weight", 0, [128], q_norm)]
    # one matrix of every other format the kernels decode, under names of the attention / linear-attention parts
    for suffix, ft, rows in (("attn_q.weight", 12, 24), ("attn_k.weight", 13, 16), ("attn_v.weight", 14, 16), ("attn_output.weight", 20, 24),
                             ("attn_qkv.weight", 23, 16), ("attn_gate.weight", 8, 40), ("ssm_alpha.weight", 30, 16)):
        w = synth.matrix(rng, ft, rows, D)
        (shard1 if ft in (12, 14, 23) else shard2).append((p + suffix, ft, [D, rows], w))
    gw.write_gguf(os.path.join(tmp, "model-00001-of-00002.gguf"), shard1, [("general.architecture", 8, "synthetic")])
    gw.write_gguf(os.path.join(tmp, "model-00002-of-00002.gguf"), shard2, [("general.architecture", 8, "synthetic")], alignment=128)
    small = dict(dt_bias=dt_bias, ssm_norm=ssm_norm, conv=conv, q_norm=q_norm, wg32=wg32)
    return m, lm, small


class _Layer:  # what run_moe expects: .layer.c is the QwMoeLayer
    def __init__(self, c):
        self.layer = self
        self.c = c


class _Ref:  # what Batch.buf expects of a buffer, for a qw_buf that the reader owns
    def __init__(self, pbuf):
        self.p = pbuf

    def ref(self):
        return self.p


@pytest.fixture(scope="module")
def model(tmp_path_factory):
    tmp = str(tmp_path_factory.mktemp("gguf"))
    rng = np.random.default_rng(77)
    m, lm, small = write_model(tmp, rng)
    return tmp, m, lm, small


@pytest.mark.parametrize("threads", ["1", "3", None])
def test_resident_bytes_are_the_files_bytes(gpu, model, threads):
    tmp, m, lm, small = model
    with gpu.switches(load_threads=threads):  # one thread: a 28 MB tensor passes four times through two staging buffers
        g = q.Gguf(tmp)
        g.load(gpu, "moe,shared,router,lm,lin,attn")
    total = 0
    for i in range(len(g)):
        t = g.get(i)
        name = t.name.decode()
        if name == "token_embd.weight":  # its part was not asked for
            assert t.res_type == -1 and g.tensor_at(t) is None
            continue
        at = g.tensor_at(t)
        assert at is not None and at.offset % 256 == 0
        if t.kind in (0, 1):  # matrices: the bytes of the file
            assert t.res_type == t.type == at.type
            assert np.array_equal(g.read_resident(t, t.nbytes), g.host(t)), name
            total += t.nbytes
    def resident(suffix, dtype, n):
        t = g.find("blk.%d.%s" % (LAYER, suffix))
        width = 2 if dtype == np.uint16 else 4
        return t, g.read_resident(t, n * width).view(dtype)
    t, v = resident("ffn_gate_inp_shexp.weight", np.uint16, D)      # F32 in the file, exact: BF16
    assert t.res_type == 30 and np.array_equal(v, m["wsg"])
    t, v = resident("ssm_conv1d.weight", np.uint16, 4 * 96)
    assert t.res_type == 30 and np.array_equal(v, (small["conv"].view(np.uint32) >> 16).astype(np.uint16).ravel())
    t, v = resident("ssm_dt.bias", np.float32, 48)                  # not exact: F32, unchanged
    assert t.res_type == 0 and np.array_equal(v, small["dt_bias"])
    t, v = resident("ssm_norm.weight", np.float32, 128)             # F16 widened
    assert t.res_type == 0 and np.array_equal(v, small["ssm_norm"].astype(np.float32))
    t, v = resident("attn_q_norm.weight", np.float32, 128)          # kept F32 although exact
    assert t.res_type == 0 and np.array_equal(v, small["q_norm"])
    assert g.resident_bytes() == total + 2 * D + 2 * 4 * 96 + 4 * 48 + 4 * 128 + 4 * 128
    assert g.load_seconds() > 0
    with pytest.raises(RuntimeError):
        g.load(gpu, "moe")  # once per object
    g.close()


def test_layer_from_files_parity(gpu, oracle, model):
    tmp, m, _, _ = model
    g = q.Gguf(tmp)
    g.load(gpu, "moe,shared,router")
    M, d, i, e = g.moe_layer(LAYER)
    assert (d, i, e) == (D, I, E)
    assert (M.router.type, M.sh_gate_w.type, M.gate.type, M.up.type, M.down.type) == (30, 30, 21, 21, 21)
    with pytest.raises(ValueError):
        g.moe_layer(LAYER + 1)
    path = q.Path(gpu, D, I, E, K, 16)
    rng = np.random.default_rng(78)
    dl = DeviceLayer(gpu, m, router_type=30, device_only=True)  # the same bytes, handed over directly
    for nb in (16, 3):
        x = synth.activations(rng, nb, D)
        out, lg, selraw, _ = run_moe(gpu, path, _Layer(M), x, nb)
        ref_lg = oracle.router(m["Wr"], m["wsg"], x, wfmt=30)
        assert maxrel(lg, ref_lg) <= 1e-5
        assert np.array_equal(oracle.topk_ids(lg, K), oracle.topk_ids(ref_lg, K))
        assert maxrel(out, oracle.moe_layer_f64(m, lg, x)) <= TOL
        out2, lg2, sel2, _ = run_moe(gpu, path, dl, x, nb)
        assert np.array_equal(out.view(np.uint16), out2.view(np.uint16)) and np.array_equal(lg.view(np.uint32), lg2.view(np.uint32))
        assert np.array_equal(selraw, sel2)
    dl.free()
    path.close()
    g.close()


def test_layer_in_the_reference_models_formats_from_files(gpu, oracle, tmp_path):
    """A layer as a GGUF of the reference's model holds it (bench/moe_bw.c:16-24 of the reference): IQ3_S gate/up,
    IQ4_NL down rows of 640, shared expert Q4_K gate, IQ4_XS up, IQ4_NL down; read from a file, made resident, run."""
    d, i, e, k, layer = 512, 640, 16, 4, 2
    rng = np.random.default_rng(91)
    m = synth.moe_layer(rng, d, i, e, fgu=21, fd=20, fsh=12, fshu=23, fshd=20)
    m["topk"] = k
    wr32, wr_bits = bf16_exact(rng.normal(0.0, 0.02, (e, d)))
    wg32, wg_bits = bf16_exact(rng.normal(0.0, 0.02, d))
    m["Wr"], m["wsg"] = wr_bits, wg_bits
    p = "blk.%d." % layer
    gw.write_gguf(os.path.join(str(tmp_path), "model.gguf"),
                  [(p + "ffn_gate_exps.weight", 21, [d, i, e], m["Wg"]), (p + "ffn_up_exps.weight", 21, [d, i, e], m["Wu"]), (p + "ffn_down_exps.weight", 20, [i, d, e], m["Wd"]),
                   (p + "ffn_gate_inp.weight", 30, [d, e], wr_bits), (p + "ffn_gate_inp_shexp.weight", 0, [d], wg32),
                   (p + "ffn_gate_shexp.weight", 12, [d, i], m["Wsg"]), (p + "ffn_up_shexp.weight", 23, [d, i], m["Wsu"]), (p + "ffn_down_shexp.weight", 20, [i, d], m["Wsd"])],
                  [("general.architecture", 8, "synthetic")])
    g = q.Gguf(str(tmp_path))
    g.load(gpu, "moe,shared,router")
    M, d2, i2, e2 = g.moe_layer(layer)
    assert (d2, i2, e2) == (d, i, e)
    assert (M.gate.type, M.down.type, M.sh_gate.type, M.sh_up.type, M.sh_down.type) == (21, 20, 12, 23, 20)
    path = q.Path(gpu, d, i, e, k, 16)
    for nb in (1, 11):
        x = synth.activations(rng, nb, d)
        out, lg, _, _ = run_moe(gpu, path, _Layer(M), x, nb)
        assert maxrel(lg, oracle.router(m["Wr"], m["wsg"], x, wfmt=30)) <= 1e-5
        assert maxrel(out, oracle.moe_layer_f64(m, lg, x)) <= TOL
    path.close()
    g.close()


def test_resident_tensor_dequantizes_bit_exactly(gpu, oracle, model):
    """The reference's tools/dqtest.py + tools/dqtest.c:26-48 on the files: for every format the first tensor of that
    format, a few rows of it through the dq_test kernel, here out of the resident copy and against the oracle."""
    tmp, m, lm, _ = model
    g = q.Gguf(tmp)
    g.load(gpu, "attn,lin,lm,shared")
    pick = {}
    for i in range(len(g)):
        t = g.get(i)
        if t.kind == 0 and t.res_type >= 0 and t.type not in pick:
            pick[t.type] = t
    assert sorted(pick) == [8, 12, 13, 14, 20, 21, 23, 30]
    for ft, t in sorted(pick.items()):
        at = g.tensor_at(t)
        ok, err = gpu.compile(dq_define_block(t.type))
        assert ok, err
        k = gpu.kernel("dq_test")
        kd, rb, rows, first = int(t.dims[0]), int(t.rowbytes), 8, 7
        y = gpu.buf(rows * kd * 4)
        b = gpu.batch()
        b.kernel(k)
        b.buf(0, _Ref(at.buf), at.offset + first * rb)  # rows 7 .. 14 of the tensor
        b.buf(1, y)
        b.bytes(2, np.array([kd, rb], np.uint32))
        b.dispatch(rows, 1, 1, 32, 1, 1)
        b.end()
        got = y.view(np.float32).reshape(rows, kd).copy()
        raw = g.host(t).reshape(-1, rb)[first:first + rows]
        want = oracle.dq_rows(t.type, raw, kd)
        assert np.array_equal(got.view(np.uint32), want.view(np.uint32)), t.name
        y.free()
    g.close()


class _T:  # a resident tensor in the form Path.qmv_gg / qmv_ggm take (Tensor.c())
    def __init__(self, at):
        self.at = at

    def c(self):
        return self.at


def test_matvec_on_resident_tensors(gpu, oracle, model):
    """The projections of a layer in one multi-matrix launch and the lm_head by the dense matvec, weights straight
    from the arena of the reader."""
    tmp = model[0]
    g = q.Gguf(tmp)
    g.load(gpu, "attn,lin,lm")
    path = q.Path(gpu, D, I, E, K, 16)
    rng = np.random.default_rng(80)
    nb = 5
    x = synth.activations(rng, nb, D)
    xb = gpu.buf_from(x)
    names = ["blk.%d.%s" % (LAYER, n) for n in ("attn_q.weight", "attn_k.weight", "attn_v.weight", "ssm_alpha.weight")]
    ts = [g.find(n) for n in names]
    Ns = [int(t.rows) for t in ts]
    ybs = [gpu.buf(nb * n * 4) for n in Ns]
    b = gpu.batch()
    path.qmv_ggm(b, [_T(g.tensor_at(t)) for t in ts], Ns, D, xb, ybs, nb)
    b.end()
    for t, n, yb in zip(ts, Ns, ybs):
        ref = oracle.qmv(t.type, g.host(t), n, D, x, f64=True)
        assert maxrel(yb.view(np.float32).reshape(nb, n), ref) <= TOL, t.name
        yb.free()
    t = g.find("language_model.lm_head.weight")  # by its model-side name
    n = int(t.rows)
    yb = gpu.buf(nb * n * 4)
    b = gpu.batch()
    path.qmv_gg(b, _T(g.tensor_at(t)), n, D, xb, yb, nb)
    b.end()
    assert maxrel(yb.view(np.float32).reshape(nb, n), oracle.qmv(14, g.host(t), n, D, x, f64=True)) <= TOL
    yb.free()
    xb.free()
    path.close()
    g.close()


def test_float_matrix_other_than_bf16_is_refused(gpu, tmp_path):
    """src/gguf.c:417-419: an F16 or F32 matrix is an error of the load, not of the parse."""
    rng = np.random.default_rng(79)
    w = rng.normal(0, 1, (8, 64)).astype(np.float16)
    gw.write_gguf(str(tmp_path / "m.gguf"), [("blk.0.ffn_gate_inp.weight", 1, [64, 8], w), ("blk.0.ffn_gate_shexp.weight", 21, [256, 4], synth.matrix(rng, 21, 4, 256))])
    g = q.Gguf(str(tmp_path))
    with pytest.raises(RuntimeError) as e:
        g.load(gpu, "router")
    assert "F16" in str(e.value)
    g.close()
    g = q.Gguf(str(tmp_path))
    with pytest.raises(RuntimeError):
        g.load(gpu, "embed")  # nothing of that part
    g.close()
    # a quantized tensor where a float one belongs (src/gguf.c:444)
    gw.write_gguf(str(tmp_path / "m.gguf"), [("blk.0.ffn_gate_inp_shexp.weight", 8, [64], synth.matrix(rng, 8, 1, 64))])
    g = q.Gguf(str(tmp_path))
    with pytest.raises(RuntimeError) as e:
        g.load(gpu, "router")
    assert "floating point" in str(e.value)
    g.close()


def test_hyper_connections_from_files(gpu, oracle, tmp_path):
    """The hyper-connection tensors of a layer and the output mixer (src/gguf.c:222-229, :250-252) made resident and run: the
    same bits as the same weights handed over directly; inject rows given as F32 in the file become BF16 when exact."""
    rng = np.random.default_rng(90)
    d, layer, HC, LR = 2048, 3, 4, 320
    w = synth.hyper_weights(rng, d)
    mixer = synth.hyper_weights(rng, d, inject=False)
    inj32 = (w["inject"].astype(np.uint32) << 16).view(np.float32)  # F32 in the file, exact in BF16
    p = "blk.%d.hc_ffn_" % layer
    tensors = [(p + "norm.weight", 0, [HC * d], w["hc_norm"]), (p + "down.weight", 30, [HC * d, LR], w["mix_down"]), (p + "up.weight", 30, [LR, HC * d], w["mix_up"]),
               (p + "inject.weight", 0, [HC * d, HC], inj32), ("output_hc_norm.weight", 0, [HC * d], mixer["hc_norm"]),
               ("output_hc_down.weight", 30, [HC * d, LR], mixer["mix_down"]), ("output_hc_up.weight", 30, [LR, HC * d], mixer["mix_up"])]
    gw.write_gguf(str(tmp_path / "hc.gguf"), tensors)
    g = q.Gguf(str(tmp_path))
    g.load(gpu, "hyper")
    H, dd = g.hyper(layer, 1)
    Hm, dm = g.hyper(0, 2)
    assert dd == d and dm == d and H["inject"] is not None and Hm["inject"] is None
    with pytest.raises(ValueError):
        g.hyper(layer, 0)  # this file has no hc_attn_* tensors
    path = q.Path(gpu, d, 512, 64, 4, 16)
    nb = 6
    h, out, inj = synth.hyper_state(rng, nb, d)
    pd = gpu.buf(int(gpu.L.qw_path_hyper_pd_bytes(nb)))

    def run(Hw, want_inj):
        hb, ob, ib, io, x = gpu.buf_from(h), gpu.buf_from(out), gpu.buf_from(inj), gpu.buf_from(np.zeros((nb, HC, HC), np.float32)), gpu.buf(nb * d * 2)
        b = gpu.batch()
        path.hyper_gg(b, Hw, nb, 1, hb, ob, ib, io, pd, x)
        b.end()
        res = (hb.view(np.float32).copy(), x.view(np.float16).copy(), io.view(np.float32).copy())
        for bb in (hb, ob, ib, io, x):
            bb.free()
        return res

    for Hw, host in ((H, w), (Hm, mixer)):
        bufs = {k: gpu.buf_from(v) for k, v in host.items() if v is not None}
        direct = {"hc_norm": q.Tensor(bufs["hc_norm"], 0), "mix_down": q.Tensor(bufs["mix_down"], 30), "mix_up": q.Tensor(bufs["mix_up"], 30),
                  "inject": q.Tensor(bufs["inject"], 30) if "inject" in bufs else None}
        a, b2 = run(Hw, host["inject"] is not None), run(direct, host["inject"] is not None)
        for u, v in zip(a, b2):
            assert np.array_equal(u.view(np.uint8), v.view(np.uint8))
        rh, rx, ri = oracle.hyper_gg(h, out, inj, host["hc_norm"], host["mix_down"], host["inject"], host["mix_up"], 1)
        assert np.abs(a[1].reshape(nb, d).astype(np.float64) - rx).max() / np.abs(rx).max() <= 1e-3
        for bb in bufs.values():
            bb.free()
    pd.free()
    path.close()
    g.close()


def test_expert_arena_released_after_first_use(gpu, oracle, model):
    """Two handles on one directory: the routed experts in an arena of their own, everything else in another. After every
    layer ran once the experts' GGUF-order bytes are freed; the layer computes the same bits from the tile-major copies."""
    tmp, m, _, _ = model
    ge, gr = q.Gguf(tmp), q.Gguf(tmp)
    ge.load(gpu, "moe")
    gr.load(gpu, "shared,router")
    with pytest.raises(ValueError):
        gr.release_source()  # holds tensors that are read as they are
    with pytest.raises(ValueError):
        ge.release_source()  # no copy made yet
    # the layer's struct: routed matrices from the experts' handle, the rest from the other
    from qwental_amd.gpu import QwMoeLayer, QwTensor
    M = QwMoeLayer()
    for name, src, key in (("gate", ge, "ffn_gate_exps"), ("up", ge, "ffn_up_exps"), ("down", ge, "ffn_down_exps"), ("router", gr, "ffn_gate_inp"),
                           ("sh_gate_w", gr, "ffn_gate_inp_shexp"), ("sh_gate", gr, "ffn_gate_shexp"), ("sh_up", gr, "ffn_up_shexp"), ("sh_down", gr, "ffn_down_shexp")):
        setattr(M, name, src.tensor_at(src.find("blk.%d.%s.weight" % (LAYER, key))))
    path = q.Path(gpu, D, I, E, K, 16)
    x = synth.activations(np.random.default_rng(80), 16, D)
    before = {nb: run_moe(gpu, path, _Layer(M), x[:nb], nb)[0] for nb in (16, 2)}
    resident = ge.resident_bytes()
    freed0 = gpu.L.qw_hip_released_bytes(gpu.g)
    ge.release_source()
    assert gpu.L.qw_hip_released_bytes(gpu.g) - freed0 >= resident
    for nb in (16, 2):
        out = run_moe(gpu, path, _Layer(M), x[:nb], nb)[0]
        assert np.array_equal(out.view(np.uint16), before[nb].view(np.uint16))
    path.close()
    ge.close()
    gr.close()
