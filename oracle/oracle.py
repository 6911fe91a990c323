"""TEST INFRASTRUCTURE — ctypes front end of the CPU oracle (oracle/qw_oracle.c).

Only tests, the smoke check and the benchmark's cpu_baseline leg import this module; the product
library never does. `load()` builds libqworacle.so with `make` when it is missing.
"""
import ctypes as C
import os
import subprocess

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
_lib = None


def build(force=False):
    if force or not os.path.exists(os.path.join(HERE, "libqworacle.so")):
        subprocess.run(["make", "-C", HERE, "libqworacle.so", "dqcpu_oracle"] + (["-B"] if force else []), check=True,
                       stdout=subprocess.DEVNULL)
    if os.path.isdir("/root/reference") and (force or not os.path.exists(os.path.join(HERE, "_ref", "libggml_dq_ref.so"))):
        subprocess.run(["make", "-C", HERE, "ref"], check=True, stdout=subprocess.DEVNULL)


def load():
    global _lib
    if _lib is not None:
        return _lib
    build()
    L = C.CDLL(os.path.join(HERE, "libqworacle.so"))
    vp, i, sz = C.c_void_p, C.c_int, C.c_size_t
    L.qwo_h2f.restype = C.c_float
    L.qwo_h2f.argtypes = [C.c_uint16]
    L.qwo_f2h.restype = C.c_uint16
    L.qwo_f2h.argtypes = [C.c_float]
    L.qwo_row_bytes.restype = sz
    L.qwo_row_bytes.argtypes = [i, i]
    L.qwo_dq_ok.restype = C.c_bool
    L.qwo_dq_ok.argtypes = [i]
    for f in (L.qwo_dq_row, L.qwo_dq_row_tab):
        f.restype = C.c_bool
        f.argtypes = [i, vp, vp, i]
    L.qwo_tab_iq3ss.argtypes = [vp]
    L.qwo_iq3s_table.restype = C.POINTER(C.c_uint32)
    for f in (L.qwo_qmv_f32, L.qwo_qmv_f64):
        f.restype = None
        f.argtypes = [i, vp, i, i, vp, i, i, vp, i, i]
    L.qwo_router.argtypes = [i, vp, vp, vp, i, i, i, vp]
    L.qwo_sel_bytes.restype = sz
    L.qwo_sel_bytes.argtypes = [i, i]
    L.qwo_select.argtypes = [vp, i, i, i, i, vp]
    L.qwo_topk.argtypes = [vp, i, i, i, vp]
    L.qwo_moe_layer_f32.argtypes = [vp, vp, vp, i, i, vp, vp, vp, i]
    L.qwo_moe_layer_f64.argtypes = [vp, vp, vp, i, vp, i]
    L.qwo_moe_pack.restype = i
    L.qwo_moe_pack.argtypes = [vp, i, i, i, vp, vp, vp, vp, i]
    L.qwo_hyper_gg.restype = None
    L.qwo_hyper_gg.argtypes = [i, i, i, i, i] + [vp] * 10
    L.qwo_max_threads.restype = i
    _lib = L
    return L


def _p(a):
    return a.ctypes.data_as(C.c_void_p)


def row_bytes(ftype, K):
    return int(load().qwo_row_bytes(ftype, K))


def dq_rows(ftype, raw, K, tab=False):
    """raw: uint8 [rows, row_bytes] -> float32 [rows, K]."""
    L = load()
    raw = np.ascontiguousarray(raw, dtype=np.uint8)
    rows = raw.shape[0]
    if not L.qwo_dq_ok(ftype):
        raise ValueError("oracle: unsupported ggml type %d" % ftype)
    assert raw.shape[1] == row_bytes(ftype, K)
    out = np.empty((rows, K), np.float32)
    fn = L.qwo_dq_row_tab if tab else L.qwo_dq_row
    for r in range(rows):
        ok = fn(ftype, C.c_void_p(raw.ctypes.data + r * raw.shape[1]), C.c_void_p(out.ctypes.data + r * K * 4), K)
        if not ok:
            raise ValueError("oracle: unsupported ggml type %d" % ftype)
    return out


def tab_iq3ss():
    t = np.empty(8192 * 4, np.uint16)
    load().qwo_tab_iq3ss(_p(t))
    return t.view(np.float16).reshape(8192, 4)


def iq3s_table():
    return np.ctypeslib.as_array(load().qwo_iq3s_table(), shape=(512,)).copy()


def qmv(ftype, W, N, K, x, f64=False, threads=0):
    """W uint8 [N*row_bytes]; x float16 [nb, K] -> y [nb, N] (float32, or float64 when f64)."""
    L = load()
    W = np.ascontiguousarray(W, np.uint8)
    x = np.ascontiguousarray(x, np.float16)
    nb = x.shape[0]
    y = np.empty((nb, N), np.float64 if f64 else np.float32)
    (L.qwo_qmv_f64 if f64 else L.qwo_qmv_f32)(ftype, _p(W), N, K, _p(x), nb, K, _p(y), N, threads)
    return y


def router(Wr, Wsg, x, wfmt=1):
    """Wr [E, D], Wsg [D], x [nb, D] as uint16 bit patterns / float16 -> logits float32 [nb, E + 1]."""
    L = load()
    Wr = np.ascontiguousarray(Wr).view(np.uint16)
    Wsg = np.ascontiguousarray(Wsg).view(np.uint16)
    x = np.ascontiguousarray(x, np.float16)
    E, D = Wr.shape
    nb = x.shape[0]
    lg = np.empty((nb, E + 1), np.float32)
    L.qwo_router(wfmt, _p(Wr), _p(Wsg), _p(x), nb, D, E, _p(lg))
    return lg


class Sel:
    """Decoded view of a selection record (layout in qw_oracle.h)."""

    def __init__(self, raw, gnb, topk):
        gu = gnb * topk
        raw = np.ascontiguousarray(raw, np.uint8)
        self.raw = raw
        self.gnb, self.topk = gnb, topk
        self.U = int(raw[:4].view(np.uint32)[0])
        self.ue = raw[4:4 + 4 * gu].view(np.uint32)
        self.mask = raw[4 + 4 * gu:4 + 8 * gu].view(np.uint32)
        o = 4 + 8 * gu
        self.slot = raw[o:o + gu * gnb].reshape(gu, gnb)
        o += gu * gnb
        self.w = raw[o:o + 4 * gnb * (topk + 1)].view(np.float32).reshape(gnb, topk + 1)


def sel_bytes(gnb, topk):
    return int(load().qwo_sel_bytes(gnb, topk))


def select(logits, topk, gnb):
    L = load()
    logits = np.ascontiguousarray(logits, np.float32)
    nbr, E1 = logits.shape
    raw = np.zeros(sel_bytes(gnb, topk), np.uint8)
    L.qwo_select(_p(logits), nbr, E1 - 1, topk, gnb, _p(raw))
    return Sel(raw, gnb, topk)


def topk_ids(logits, topk):
    L = load()
    logits = np.ascontiguousarray(logits, np.float32)
    nbr, E1 = logits.shape
    ids = np.empty((nbr, topk), np.uint32)
    L.qwo_topk(_p(logits), nbr, E1 - 1, topk, _p(ids))
    return ids


class _MoeW(C.Structure):
    _fields_ = [(n, C.c_int) for n in ("D", "I", "E", "topk", "fgu", "fd", "fsg", "fsu", "fsd")] + \
               [(n, C.c_void_p) for n in ("Wg", "Wu", "Wd", "Wsg", "Wsu", "Wsd")]


def _moew(m):
    keep = [np.ascontiguousarray(m[k], np.uint8) for k in ("Wg", "Wu", "Wd", "Wsg", "Wsu", "Wsd")]
    s = _MoeW(m["D"], m["I"], m["E"], m["topk"], m["fgu"], m["fd"], m["fsg"], m["fsu"], m["fsd"], *[a.ctypes.data for a in keep])
    return s, keep


def moe_layer_f32(m, logits, x, gnb, threads=0):
    """m: dict with D, I, E, topk, fgu, fd, fsg, fsu, fsd and uint8 arrays Wg, Wu, Wd, Wsg, Wsu, Wsd.
    Returns (out float16 [nb, D], H float32 [nb, topk+1, I], Sel)."""
    L = load()
    s, keep = _moew(m)
    logits = np.ascontiguousarray(logits, np.float32)
    x = np.ascontiguousarray(x, np.float16)
    nb = x.shape[0]
    out = np.empty((nb, m["D"]), np.float16)
    H = np.empty((nb, m["topk"] + 1, m["I"]), np.float32)
    raw = np.zeros(sel_bytes(gnb, m["topk"]), np.uint8)
    L.qwo_moe_layer_f32(C.byref(s), _p(logits), _p(x), nb, gnb, _p(out), _p(H), _p(raw), threads)
    del keep
    return out, H, Sel(raw, gnb, m["topk"])


def moe_layer_f64(m, logits, x, threads=0):
    L = load()
    s, keep = _moew(m)
    logits = np.ascontiguousarray(logits, np.float32)
    x = np.ascontiguousarray(x, np.float16)
    nb = x.shape[0]
    out = np.empty((nb, m["D"]), np.float64)
    L.qwo_moe_layer_f64(C.byref(s), _p(logits), _p(x), nb, _p(out), threads)
    del keep
    return out


def hyper_gg(h, out, inj, w, Wd, Wi, Wu, apply):
    """The GGUF profile's hyper-connection in float64. h float32 [nb, HC, D]; out float16 [nb, D]; inj float32
    [nb, HC, HC]; w float32 [HC * D]; Wd, Wi, Wu bfloat16 bit patterns (uint16) [LR, HC * D], [HC, HC * D] or None,
    [HC * D, LR]. Returns (h1 [nb, HC, D], x [nb, D], inject sums [nb, HC, HC] or None), all float64."""
    L = load()
    h = np.ascontiguousarray(h, np.float32)
    nb, HC, D = h.shape
    out = np.ascontiguousarray(out, np.float16)
    inj = np.ascontiguousarray(inj, np.float32)
    w = np.ascontiguousarray(w, np.float32)
    Wd, Wu = np.ascontiguousarray(Wd, np.uint16), np.ascontiguousarray(Wu, np.uint16)
    LR = Wd.shape[0]
    assert Wd.shape == (LR, HC * D) and Wu.shape == (HC * D, LR) and w.size == HC * D and out.shape == (nb, D) and inj.shape == (nb, HC, HC)
    Wi = None if Wi is None else np.ascontiguousarray(Wi, np.uint16)
    h1, x = np.empty((nb, HC, D), np.float64), np.empty((nb, D), np.float64)
    io = None if Wi is None else np.empty((nb, HC, HC), np.float64)
    L.qwo_hyper_gg(D, HC, LR, nb, 1 if apply else 0, _p(h), _p(out), _p(inj), _p(w), _p(Wd), None if Wi is None else _p(Wi), _p(Wu), _p(h1), _p(x),
                   None if io is None else _p(io))
    return h1, x, io


def moe_pack(ids, E, tm, max_tiles):
    L = load()
    ids = np.ascontiguousarray(ids, np.uint32).ravel()
    P = ids.size
    counts = np.empty(E, np.uint32)
    offs = np.empty(E, np.uint32)
    pos = np.empty(P, np.uint32)
    tiles = np.empty((max_tiles, 4), np.uint32)
    nt = L.qwo_moe_pack(_p(ids), P, E, tm, _p(counts), _p(offs), _p(pos), _p(tiles), max_tiles)
    return counts, offs, pos, tiles, nt


def max_threads():
    return int(load().qwo_max_threads())


def ref_dq_rows(ftype, raw, K):
    """The reference's own qw_ggml_dq_row (src/ggml_dq.c compiled into oracle/_ref); None when not built."""
    p = os.path.join(HERE, "_ref", "libggml_dq_ref.so")
    if not os.path.exists(p):
        return None
    R = C.CDLL(p)
    R.qw_ggml_dq_row.restype = C.c_bool
    R.qw_ggml_dq_row.argtypes = [C.c_int, C.c_void_p, C.c_void_p, C.c_int]
    raw = np.ascontiguousarray(raw, np.uint8)
    out = np.empty((raw.shape[0], K), np.float32)
    for r in range(raw.shape[0]):
        if not R.qw_ggml_dq_row(ftype, C.c_void_p(raw.ctypes.data + r * raw.shape[1]), C.c_void_p(out.ctypes.data + r * K * 4), K):
            return None
    return out
