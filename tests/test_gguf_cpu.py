"""The GGUF reader without a GPU: the C parser (include/qw_gguf.h) against files written by qwental_amd/gguf_writer.py and
against the restatement in oracle/gguf_file.py of the reference's parser (src/gguf.c:73-173); names, parts, sizes by closed form;
the failures the reference's parser reports."""
import os
import struct

import numpy as np
import pytest

import qwental_amd as q
from oracle import gguf_file as gf
from qwental_amd import gguf_writer as gw
from qwental_amd import synth

PARTS = dict(moe=1, shared=2, router=4, attn=8, lin=16, hyper=32, lm=64, embed=128, ple=256)  # src/model.h:111-119
KIND = dict(lin=0, exp=1, small=2, f32=3)


def raw(rng, ftype, dims):
    return rng.integers(0, 256, gf.tensor_bytes(ftype, dims), dtype=np.uint8)


def model_files(tmp_path, rng):
    """Two shards: b.gguf (alignment 64, every metadata value type) and a.gguf (default alignment, version 2)."""
    D, I, E = 512, 256, 4
    t_b = [("blk.3.ffn_gate_exps.weight", 21, [D, I, E]), ("blk.3.ffn_up_exps.weight", 21, [D, I, E]), ("blk.3.ffn_down_exps.weight", 8, [I, D, E]),
           ("blk.3.ffn_gate_inp.weight", 30, [D, E]), ("blk.3.ffn_gate_inp_shexp.weight", 0, [D]), ("blk.3.attn_q_norm.weight", 0, [128]),
           ("blk.3.hc_ffn_norm.weight", 0, [64]), ("blk.3.attn_q.weight", 12, [D, 768]), ("blk.12.ssm_a", 0, [32]),
           ("some.other.tensor", 1, [7, 3, 2, 2])]
    t_a = [("output.weight", 14, [D, 1024]), ("token_embd.weight", 13, [D, 300]), ("blk.0.attn_qkv.weight", 23, [D, 96]),
           ("blk.0.ssm_out.weight", 20, [D, 64]), ("blk.10.ffn_down_shexp.weight", 21, [I, D]), ("per_layer_token_embd.weight", 8, [64, 10])]
    meta_b = [("general.architecture", 8, "qwen-like"), ("a.u8", 0, 7), ("a.i8", 1, -7), ("a.u16", 2, 65535), ("a.i16", 3, -2), ("a.u32", 4, 1 << 31),
              ("a.i32", 5, -5), ("a.f32", 6, 1.5), ("a.bool", 7, 1), ("a.u64", 10, 1 << 40), ("a.i64", 11, -(1 << 40)), ("a.f64", 12, 2.25),
              ("tokens", 9, (8, ["<s>", "", "hello world", "x" * 300])), ("ints", 9, (5, [1, -2, 3])), ("u64s", 9, (10, [1, 2])), ("empty", 9, (6, []))]
    data = {}
    for name, ft, dims in t_b + t_a:
        data[name] = raw(rng, ft, dims)
    where = gw.write_gguf(str(tmp_path / "b.gguf"), [(n, ft, d, data[n]) for n, ft, d in t_b], meta_b, alignment=64)
    where.update(gw.write_gguf(str(tmp_path / "a.gguf"), [(n, ft, d, data[n]) for n, ft, d in t_a], [("x", 4, 1)], version=2))
    return t_a, t_b, data, where


def test_parser_against_written_files(tmp_path):
    rng = np.random.default_rng(11)
    t_a, t_b, data, where = model_files(tmp_path, rng)
    (tmp_path / "notes.txt").write_text("not a model file")
    g = q.Gguf(str(tmp_path))
    sh = g.shards()
    assert [os.path.basename(s["path"]) for s in sh] == ["a.gguf", "b.gguf"]  # sorted by name (src/gguf.c:313)
    assert [s["alignment"] for s in sh] == [32, 64]
    assert len(g) == len(t_a) + len(t_b)
    # the restated parser of the reference sees the same table
    for si, s in enumerate(sh):
        ref = gf.read_gguf(s["path"])
        assert ref["alignment"] == s["alignment"] and ref["data_start"] == s["data_start"] and s["data_start"] % s["alignment"] == 0
        mine = [g.get(i) for i in range(len(g)) if g.get(i).shard == si]
        assert len(mine) == len(ref["tensors"])
        for t, r in zip(mine, ref["tensors"]):  # file order is kept
            assert t.name.decode() == r["name"] and t.type == r["type"] and t.nd == len(r["dims"])
            assert list(t.dims[:t.nd]) == r["dims"] and t.offset == r["offset"] and t.nbytes == r["nbytes"]
    # bytes, offsets and sizes as written
    for name, ft, dims in t_a + t_b:
        t = g.find(name)
        assert t is not None and t.offset == where[name] and t.offset % sh[t.shard]["alignment"] == 0
        qb, bb = gf.BLOCKS[ft]
        assert t.rowbytes == dims[0] // qb * bb and t.rows == int(np.prod(dims[1:])) and t.nbytes == t.rows * t.rowbytes
        assert np.array_equal(g.host(t), data[name])
        assert t.res_type == -1
    assert g.find("no.such.tensor") is None and g.find("") is None
    g.close()


def test_names_parts_and_kinds(tmp_path):
    rng = np.random.default_rng(12)
    model_files(tmp_path, rng)
    g = q.Gguf(str(tmp_path))
    lay = "language_model.model.layers.%d."
    want = {  # src/gguf.c:187-258
        "blk.3.ffn_gate_exps.weight": ("moe", lay % 3 + "mlp.switch_mlp.gate_proj.iq", "exp"),
        "blk.3.ffn_up_exps.weight": ("moe", lay % 3 + "mlp.switch_mlp.up_proj.iq", "exp"),
        "blk.3.ffn_down_exps.weight": ("moe", lay % 3 + "mlp.switch_mlp.down_proj.iq", "exp"),
        "blk.3.ffn_gate_inp.weight": ("router", lay % 3 + "mlp.gate.weight", "lin"),
        "blk.3.ffn_gate_inp_shexp.weight": ("router", lay % 3 + "mlp.shared_expert_gate.weight", "small"),
        "blk.3.attn_q_norm.weight": ("attn", lay % 3 + "self_attn.q_norm.weight", "f32"),
        "blk.3.attn_q.weight": ("attn", lay % 3 + "self_attn.q_proj.weight", "lin"),
        "blk.12.ssm_a": ("lin", lay % 12 + "linear_attn.A_neg", "f32"),
        "output.weight": ("lm", "language_model.lm_head.weight", "lin"),
        "token_embd.weight": ("embed", "language_model.model.embed_tokens.weight", "lin"),
        "blk.0.attn_qkv.weight": ("lin", lay % 0 + "linear_attn.in_proj_qkv.weight", "lin"),
        "blk.0.ssm_out.weight": ("lin", lay % 0 + "linear_attn.out_proj.weight", "lin"),
        "blk.10.ffn_down_shexp.weight": ("shared", lay % 10 + "mlp.shared_expert.down_proj.weight", "lin"),
        "blk.3.hc_ffn_norm.weight": ("hyper", lay % 3 + "mlp_hyper_connection.hc_norm.weight", "f32"),
    }
    for name, (part, model, kind) in want.items():
        t = g.find(name)
        assert (t.part, t.model.decode(), t.kind) == (PARTS[part], model, KIND[kind]), name
        assert g.find(model).name.decode() == name  # found by the model-side name too
    for name in ("some.other.tensor", "per_layer_token_embd.weight"):  # not part of this path
        t = g.find(name)
        assert t.part == 0 and t.model == b""
    g.close()


def test_type_table_and_parts():
    L = q.load_lib()
    import ctypes as C
    for ft, (qb, bb) in gf.BLOCKS.items():
        a, b = C.c_int(), C.c_int()
        assert L.qw_ggml_block(ft, C.byref(a), C.byref(b)) and (a.value, b.value) == (qb, bb)
    for ft in (4, 5, 9, 15, 24, 31, 41, -1):
        assert not L.qw_ggml_block(ft, C.byref(C.c_int()), C.byref(C.c_int()))
        assert L.qw_ggml_name(ft) == b"?"
    # the formats this library computes with agree with its own block table
    for ft, (qb, bb) in synth.BLOCK.items():
        assert gf.BLOCKS[ft] == (qb, bb)
    names = {0: "F32", 1: "F16", 30: "BF16", 8: "Q8_0", 12: "Q4_K", 13: "Q5_K", 14: "Q6_K", 20: "IQ4_NL", 21: "IQ3_S", 23: "IQ4_XS"}
    for ft, n in names.items():
        assert L.qw_ggml_name(ft) == n.encode()
    pp = L.qw_gguf_parse_parts
    assert pp(None) == pp(b"") == pp(b"all") == 511  # src/gguf.c:40
    assert pp(b"moe") == 1 and pp(b"moe,shared,router") == 7 and pp(b"lm,embed") == 192 and pp(b"attn,lin,hyper,ple") == 8 + 16 + 32 + 256
    assert pp(b"moe,nonsense,router") == 5 and pp(b"nonsense") == 0 and pp(b"mo") == 0


def _head(version=3, nt=0, nkv=0, magic=b"GGUF"):
    return magic + struct.pack("<IQQ", version, nt, nkv)


@pytest.mark.parametrize("case", ["magic", "version", "short_header", "kv_truncated", "kv_type", "nested_array", "array_type", "long_string",
                                  "tensor_truncated", "five_dims", "beyond_end", "huge_counts", "zero_alignment", "overflow"])
def test_damaged_files_are_refused(tmp_path, case):
    s = lambda t: struct.pack("<Q", len(t)) + t
    tensor = s(b"w") + struct.pack("<IQIQ", 1, 32, 0, 0)  # F32 [32] at offset 0: 128 bytes of data
    body = {
        "magic": _head(magic=b"GGML"),
        "version": _head(version=1),
        "short_header": b"GGUF\x03\x00",
        "kv_truncated": _head(nkv=1) + s(b"key") + struct.pack("<I", 4) + b"\x01",
        "kv_type": _head(nkv=1) + s(b"key") + struct.pack("<I", 13) + b"\0" * 8,
        "nested_array": _head(nkv=1) + s(b"key") + struct.pack("<IIQ", 9, 9, 0),
        "array_type": _head(nkv=1) + s(b"key") + struct.pack("<IIQ", 9, 13, 1) + b"\0" * 8,
        "long_string": _head(nkv=1) + struct.pack("<Q", (1 << 24) + 1) + b"k" * 64,
        "tensor_truncated": _head(nt=1) + s(b"w") + struct.pack("<I", 1),
        "five_dims": _head(nt=1) + s(b"w") + struct.pack("<I", 5) + b"\0" * 64,
        "beyond_end": _head(nt=1) + tensor + b"\0" * 64,  # needs 128 bytes of data, the file holds fewer
        "huge_counts": _head(nt=1 << 60, nkv=0) + b"\0" * 64,
        "zero_alignment": _head(nt=0, nkv=1) + s(b"general.alignment") + struct.pack("<II", 4, 0),
        "overflow": _head(nt=1) + s(b"w") + struct.pack("<IQQQIQ", 3, 1 << 30, 1 << 30, 1 << 30, 0, 0) + b"\0" * 64,  # 2^90 values
    }[case]
    (tmp_path / "m.gguf").write_bytes(body)
    with pytest.raises(ValueError) as e:
        q.Gguf(str(tmp_path))
    assert "GGUF" in str(e.value)
    if case not in ("beyond_end", "huge_counts", "zero_alignment", "overflow"):  # the restated reference parser refuses the same files
        with pytest.raises(ValueError):
            gf.read_gguf(str(tmp_path / "m.gguf"))


def test_directory_errors_and_small_good_file(tmp_path):
    with pytest.raises(ValueError):
        q.Gguf(str(tmp_path / "missing"))
    with pytest.raises(ValueError):
        q.Gguf(str(tmp_path))  # no .gguf in it
    s = lambda t: struct.pack("<Q", len(t)) + t
    tensor = s(b"w") + struct.pack("<IQIQ", 1, 32, 0, 0)
    head = _head(nt=1) + tensor
    pad = (-len(head)) % 32
    (tmp_path / "m.gguf").write_bytes(head + b"\0" * pad + bytes(range(128)))
    g = q.Gguf(str(tmp_path))
    t = g.find("w")
    assert t.offset == len(head) + pad and t.nbytes == 128 and np.array_equal(g.host(t), np.arange(128, dtype=np.uint8))
    g.close()
    # an empty tensor list is a valid file
    (tmp_path / "m.gguf").write_bytes(_head())
    g = q.Gguf(str(tmp_path))
    assert len(g) == 0
    g.close()
