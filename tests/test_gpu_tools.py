"""Clients of the C interface as separate programs: dqhip (this package's block-decode tool) against the oracle's
dqcpu_oracle on the same files, and — where they were built from the reference tree into oracle/_ref/ — the reference's
own tools/dqtest.c and tools/ggmtest.c, compiled unchanged and linked against libqwgpu_hip.so."""
import ctypes as C
import os
import subprocess

import numpy as np
import pytest

from helpers import dq_define_block
from qwental_amd import synth

pytestmark = pytest.mark.gpu
ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
DQHIP = os.path.join(ROOT, "qwental_amd", "dqhip")
DQCPU = os.path.join(ROOT, "oracle", "dqcpu_oracle")
REF = os.path.join(ROOT, "oracle", "_ref")


def run(cmd):
    print("[run] " + " ".join(cmd), flush=True)
    return subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True, timeout=110)


def same_floats(a, b):
    """Bit for bit, +0 and -0 taken as equal (the formats with a minimum can produce either)."""
    x, y = np.fromfile(a, np.float32), np.fromfile(b, np.float32)
    return x.shape == y.shape and np.array_equal(np.where(x == 0, 0.0, x).view(np.uint32), np.where(y == 0, 0.0, y).view(np.uint32))


# (type, K, rows): the last IQ3_S case is 9.4 MB of blocks, more than the size up to which a host-visible buffer is
# copied at every submit, and its float output (89 MB) needs more than one slice of rows
@pytest.mark.parametrize("ftype,K,rows", [(21, 2048, 96), (8, 2048, 96), (12, 2048, 64), (14, 2048, 64), (21, 2048, 10880)])
def test_dqhip_against_the_oracle_tool(oracle, tmp_path, ftype, K, rows):
    assert os.path.exists(DQHIP) and os.path.exists(DQCPU), "tools are not built (python -m qwental_amd.build; make -C oracle)"
    raw = synth.matrix(np.random.default_rng(ftype + rows), ftype, rows, K)
    fin, fg, fc = str(tmp_path / "w.bin"), str(tmp_path / "gpu.f32"), str(tmp_path / "cpu.f32")
    raw.tofile(fin)
    r = run([DQHIP, str(ftype), str(K), str(rows), fin, fg])
    assert r.returncode == 0, r.stdout
    r = run([DQCPU, str(ftype), str(K), str(rows), fin, fc])
    assert r.returncode == 0, r.stdout
    assert same_floats(fg, fc)


def test_dqhip_exit_codes(tmp_path):
    fin = str(tmp_path / "w.bin")
    np.zeros(110 * 8, np.uint8).tofile(fin)
    assert run([DQHIP, "21", "2048"]).returncode == 2                                   # usage
    assert run([DQHIP, "21", "2000", "1", fin, str(tmp_path / "o")]).returncode == 2       # K not a multiple of the block
    assert run([DQHIP, "99", "2048", "1", fin, str(tmp_path / "o")]).returncode == 3       # no such type
    assert run([DQHIP, "10", "2048", "1", fin, str(tmp_path / "o")]).returncode == 3       # a ggml type without a decoder here (Q2_K)
    assert run([DQHIP, "21", "2048", "2", fin, str(tmp_path / "o")]).returncode == 1       # the file is shorter than two rows
    assert run([DQHIP, "21", "2048", "1", str(tmp_path / "none"), str(tmp_path / "o")]).returncode == 1


def test_large_buffer_filled_through_ptr_reaches_the_gpu(gpu, oracle):
    """A host-visible buffer of more than 4 MiB that the caller fills through qw_buf.ptr and never marks (what the
    reference's clients do: fread / memcpy into ptr, tools/dqtest.c:37) is copied at its first bind."""
    K, rows = 2048, 6000  # 5.3 MB of IQ3_S blocks
    raw = synth.matrix(np.random.default_rng(5), 21, rows, K)
    ok, err = gpu.compile(dq_define_block(21))
    assert ok, err
    w, y = gpu.buf(raw.nbytes), gpu.buf(rows * K * 4)
    C.memmove(w.c.ptr, raw.ctypes.data, raw.nbytes)  # straight into the shadow: no fill(), no mark_dirty
    b = gpu.batch()
    b.kernel(gpu.kernel("dq_test"))
    b.buf(0, w)
    b.buf(1, y)
    b.bytes(2, np.array([K, raw.nbytes // rows], np.uint32))
    b.dispatch(rows, 1, 1, 32, 1, 1)
    b.end()
    got = y.view(np.float32).reshape(rows, K)
    sample = np.random.default_rng(6).choice(rows, 64, replace=False)
    ref = oracle.dq_rows(21, raw.reshape(rows, -1)[sample], K)
    assert np.array_equal(got[sample].view(np.uint32), ref.view(np.uint32))
    assert np.abs(got).max() > 0
    w.free()
    y.free()


@pytest.mark.parametrize("ftype", [21, 8])
def test_reference_dqtest_runs_unchanged(oracle, tmp_path, ftype):
    """The reference's tools/dqtest.c (its src/gpu.h, its embedded Metal text, its call sequence), linked against this
    backend: same floats as the oracle tool. Skipped where oracle/_ref was not built (no reference tree)."""
    exe = os.path.join(REF, "dqtest_ref")
    if not os.path.exists(exe):
        pytest.skip("oracle/_ref/dqtest_ref is not built (the reference tree was absent at build time)")
    K, rows = 2048, 3000  # IQ3_S: 2.6 MB; Q8_0: 6.5 MB, beyond the copy-at-every-submit size
    raw = synth.matrix(np.random.default_rng(40 + ftype), ftype, rows, K)
    fin, fg, fc = str(tmp_path / "w.bin"), str(tmp_path / "gpu.f32"), str(tmp_path / "cpu.f32")
    raw.tofile(fin)
    r = run([exe, str(ftype), str(K), str(rows), fin, fg])
    assert r.returncode == 0, r.stdout
    assert run([DQCPU, str(ftype), str(K), str(rows), fin, fc]).returncode == 0
    assert same_floats(fg, fc)


@pytest.mark.parametrize("ftype,nb", [(12, 1), (14, 4), (23, 8), (30, 2)])
def test_reference_ggmtest_runs_unchanged(oracle, tmp_path, ftype, nb):
    """The reference's tools/ggmtest.c over this backend: y = W x for one matrix of a K-quant / IQ4_XS / bfloat16 format
    against the oracle's float64 product (the method of tools/ggmtest.py:44-53)."""
    exe = os.path.join(REF, "ggmtest_ref")
    if not os.path.exists(exe):
        pytest.skip("oracle/_ref/ggmtest_ref is not built (the reference tree was absent at build time)")
    K, rows = 2048, 1024
    rng = np.random.default_rng(50 + ftype)
    raw = synth.matrix(rng, ftype, rows, K) if ftype != 30 else synth.blocks(rng, 30, rows * K).reshape(-1)
    x = synth.activations(rng, nb, K)
    fw, fx, fy = str(tmp_path / "w.bin"), str(tmp_path / "x.bin"), str(tmp_path / "y.f32")
    raw.tofile(fw)
    x.tofile(fx)
    r = run([exe, str(ftype), str(K), str(rows), str(nb), fw, fx, fy])
    assert r.returncode == 0, r.stdout
    got = np.fromfile(fy, np.float32).reshape(nb, rows).astype(np.float64)
    ref = oracle.qmv(ftype, raw, rows, K, x, f64=True)
    assert np.abs(got - ref).max() / np.abs(ref).max() <= 2e-3


def bw_block(base, name, sl, ld, rb, ub):
    """The define block bench/moe_bw.c:34 puts before the reference's kernels/moe_bw.metal."""
    return "#define SL %d\n#define LD %d\n#define RB %d\n#define UB %d\n#define %s %s\n" % (sl, ld, rb, ub, base, name)


def test_bw_chunks_reads_the_slices_the_reference_kernel_reads(gpu):
    """kernels/moe_bw.metal:7-26 folds what it reads into a sink that is only stored when it equals one constant. An
    arena of zeros with that constant in one place shows which workgroup and thread read that place: unit
    start + SL + nt + 44 belongs to slice 1, second load of thread 44."""
    sl, ld, nt = 1024, 4, 256
    ok, err = gpu.compile(bw_block("bw_chunks", "bw_chunks_t", sl, ld, 0, 0))
    assert ok, err
    n16 = 8192
    arena = np.zeros((n16, 4), np.uint32)
    start, length = 100, 3000
    arena[start + sl + nt + 44, 2] = 0x9e3779b9
    a, out = gpu.buf_from(arena), gpu.buf_from(np.zeros(1024, np.uint32))
    ch = gpu.buf_from(np.array([[7, 9], [start, length], [start + 5000, 10**9]], np.uint32))  # the last record reaches past the arena: clamped
    b = gpu.batch()
    b.kernel(gpu.kernel("bw_chunks_t"))
    b.buf(0, a)
    b.buf(1, ch, 8)  # from the second record on, as the driver binds a layer's records at an offset
    b.buf(2, out)
    b.dispatch((length + sl - 1) // sl, 2, 1, nt, 1, 1)
    b.end()
    got = out.view(np.uint32)
    want = np.zeros(1024, np.uint32)
    want[44] = 0x9e3779b9
    assert np.array_equal(got, want)
    for x in (a, out, ch):
        x.free()


def test_bw_rows_and_refusals(gpu):
    ok, err = gpu.compile(bw_block("bw_rows", "bw_rows_t", 1, 1, 1100, 8))
    assert ok, err
    a, out = gpu.buf_from(np.ones(1 << 20, np.uint8)), gpu.buf_from(np.zeros(1024, np.uint32))
    ch = gpu.buf_from(np.array([[64, 4096], [60000, 5536]], np.uint32))  # rows of the second chunk run past the arena: not read
    b = gpu.batch()
    b.kernel(gpu.kernel("bw_rows_t"))
    b.buf(0, a)
    b.buf(1, ch)
    b.buf(2, out)
    b.dispatch(8, 2, 1, 256, 1, 1)
    b.end()
    assert not out.view(np.uint32).any()
    # an odd unit, a thread count the row kernel is not written for, more records than the buffer holds
    ok, err = gpu.compile(bw_block("bw_rows", "bw_rows_odd", 1, 1, 1100, 7))
    assert ok, err
    for name, gy, tx in (("bw_rows_odd", 2, 256), ("bw_rows_t", 2, 128), ("bw_rows_t", 3, 256)):
        b = gpu.batch()
        b.kernel(gpu.kernel(name))
        b.buf(0, a)
        b.buf(1, ch)
        b.buf(2, out)
        b.dispatch(8, gy, 1, tx, 1, 1)
        assert b.end(check=False) < 0 and gpu.last_error()
    for x in (a, out, ch):
        x.free()


def test_reference_moe_bw_runs_unchanged():
    """The reference's bench/moe_bw.c (read-pattern ceiling of a decode layer) over this backend: it allocates a 2 GiB
    arena, compiles its kernels/moe_bw.metal with four parameters and prints a table of microseconds per layer."""
    exe = os.path.join(REF, "moe_bw_ref")
    if not os.path.exists(exe):
        pytest.skip("oracle/_ref/moe_bw_ref is not built (the reference tree was absent at build time)")
    r = run([exe])
    assert r.returncode == 0, r.stdout
    rows = [ln for ln in r.stdout.splitlines() if ln.startswith("| ") and ln.count("|") == 7 and ln.split("|")[5].strip().replace(".", "").isdigit()]
    assert len(rows) == 5, r.stdout  # three dispatches a layer; front, gate/up, down alone; the row pattern
    for ln in rows:
        us, gbs = float(ln.split("|")[5]), float(ln.split("|")[6])
        assert 1 < us < 1e4 and 50 < gbs < 8000, ln
    print(r.stdout)
