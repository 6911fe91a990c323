"""ctypes binding of libqwgpu_hip.so: the GPU interface (include/gpu.h), its HIP additions (include/qw_hip_ext.h),
the host side of the path (include/qw_path.h), the GGUF reader (include/qw_gguf.h) and the step planner
(include/qw_par.h). Thin by design: one Python
method per C function."""
import contextlib
import ctypes as C
import os

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
_lib = None


def lib_path():
    """The built library; QW_HIP_LIB selects another build of it (experiments)."""
    return os.environ.get("QW_HIP_LIB") or os.path.join(HERE, "libqwgpu_hip.so")


class QwBuf(C.Structure):
    _fields_ = [("handle", C.c_void_p), ("ptr", C.c_void_p), ("size", C.c_size_t)]


class QwTensor(C.Structure):
    _fields_ = [("buf", C.POINTER(QwBuf)), ("offset", C.c_size_t), ("type", C.c_int)]


class QwMoeLayer(C.Structure):
    _fields_ = [(n, QwTensor) for n in ("router", "sh_gate_w", "gate", "up", "down", "sh_gate", "sh_up", "sh_down")]


class QwHyperW(C.Structure):
    _fields_ = [(n, QwTensor) for n in ("hc_norm", "mix_down", "mix_up", "inject")]


class QwMoeWeightsDev(C.Structure):
    _fields_ = [(n, C.c_void_p) for n in ("router", "sh_gate_w", "gate", "up", "down", "sh_gate", "sh_up", "sh_down")] + \
               [(n, C.c_int) for n in ("router_type", "gate_type", "down_type", "sh_gate_type", "sh_up_type", "sh_down_type")]


class QwVstepInfo(C.Structure):
    _fields_ = [("rows", C.c_int), ("ngroups", C.c_int), ("groups", C.c_int * 64), ("r0", C.c_int * 64), ("gpu_ms", C.c_double), ("wall_ms", C.c_double)]


class QwGgufTensor(C.Structure):
    _fields_ = [("name", C.c_char_p), ("model", C.c_char_p), ("part", C.c_uint), ("kind", C.c_int), ("type", C.c_uint32), ("nd", C.c_uint32),
                ("dims", C.c_uint64 * 4), ("rows", C.c_uint64), ("rowbytes", C.c_uint64), ("nbytes", C.c_uint64), ("shard", C.c_int),
                ("offset", C.c_uint64), ("res_type", C.c_int)]


# every symbol include/gpu.h, include/qw_hip_ext.h, include/qw_path.h and include/qw_gguf.h declare: (name, restype, argtypes)
_vp, _sz, _u, _i, _b, _d = C.c_void_p, C.c_size_t, C.c_uint, C.c_int, C.c_bool, C.c_double
_pb, _pt, _pm, _pg = C.POINTER(QwBuf), C.POINTER(QwTensor), C.POINTER(QwMoeLayer), C.POINTER(QwGgufTensor)
_pi = C.POINTER(C.c_int)
SYMBOLS = [
    ("qw_gpu_open", _vp, []), ("qw_gpu_close", None, [_vp]), ("qw_gpu_name", C.c_char_p, [_vp]), ("qw_gpu_max_working_set", _sz, [_vp]),
    ("qw_gpu_compile", _b, [_vp, C.c_char_p, _sz, C.c_char_p, _sz]), ("qw_kernel_get", _vp, [_vp, C.c_char_p]),
    ("qw_kernel_max_threads", _u, [_vp]), ("qw_kernel_simd_width", _u, [_vp]),
    ("qw_buf_new", _b, [_vp, _sz, _pb]), ("qw_buf_free", None, [_pb]), ("qw_pool_push", _vp, []), ("qw_pool_pop", None, [_vp]),
    ("qw_buf_wrap", _b, [_vp, _vp, _sz, _pb]),
    ("qw_batch_begin", _vp, [_vp, _b]), ("qw_batch_kernel", None, [_vp, _vp]), ("qw_batch_buf", None, [_vp, _u, _pb, _sz]),
    ("qw_batch_bytes", None, [_vp, _u, _vp, _sz]), ("qw_batch_threadgroup_mem", None, [_vp, _u, _sz]),
    ("qw_batch_dispatch", None, [_vp, _u, _u, _u, _u, _u, _u]), ("qw_batch_barrier", None, [_vp]), ("qw_batch_flush", None, [_vp]),
    ("qw_batch_end", _d, [_vp]), ("qw_batch_submit", None, [_vp]), ("qw_batch_wait", _d, [_vp]), ("qw_batch_poll", _b, [_vp]),
    ("qw_gpu_set_stream", None, [_vp, _i]),
    ("qw_profile_enable", None, [_vp, _b]), ("qw_profile_count", _i, [_vp]), ("qw_profile_get", C.c_char_p, [_vp, _i, C.POINTER(_d)]),
    ("qw_gpu_empty_commit_latency", _d, [_vp, _vp, _i]), ("qw_power_desc", None, [C.c_char_p, _sz]), ("qw_on_battery", _b, []),
    ("qw_now", _d, []),
    # qw_hip_ext.h
    ("qw_hip_buf_new_device", _b, [_vp, _sz, _pb]), ("qw_hip_buf_mark_dirty", None, [_pb]),
    ("qw_hip_buf_upload", _b, [_pb, _sz, _sz]), ("qw_hip_buf_download", _b, [_pb, _sz, _sz]),
    ("qw_hip_buf_write", _b, [_pb, _sz, _vp, _sz]), ("qw_hip_buf_read", _b, [_pb, _sz, _vp, _sz]), ("qw_hip_buf_devptr", _vp, [_pb]),
    ("qw_hip_buf_write_fd", _b, [_pb, _sz, _i, C.c_uint64, _sz]),
    ("qw_hip_reload_switches", None, [_vp]), ("qw_hip_sync_words", _b, [_vp, _vp, _sz]),
    ("qw_hip_set_repack", None, [_vp, _b]), ("qw_hip_graph_launches", C.c_uint, [_vp]), ("qw_hip_set_graphs", None, [_vp, _b]),
    ("qw_hip_packed_bytes", _sz, [_vp]), ("qw_hip_buf_release_source", _b, [_pb]), ("qw_hip_released_bytes", _sz, [_vp]),
    ("qw_hip_compile_check", _b, [C.c_char_p, _sz, C.c_char_p, _sz, C.c_char_p, _sz]),
    ("qw_hip_last_error", C.c_char_p, [_vp]), ("qw_hip_cu_count", _i, [_vp]), ("qw_hip_arch", C.c_char_p, []),
    ("qw_hip_profile_mean", _d, [_vp, C.c_char_p, C.POINTER(_i)]),
    ("qw_hip_profile_entry", C.c_char_p, [_vp, _i, C.POINTER(_d)]),
    # qw_path.h
    ("qw_path_open", _vp, [_vp, _i, _i, _i, _i, _i, _b]), ("qw_path_close", None, [_vp]),
    ("qw_path_sel_bytes", _sz, [_vp, _i]), ("qw_path_logits_bytes", _sz, [_vp, _i]), ("qw_path_nbv", _i, [_i]),
    ("qw_path_qmv_gg", _b, [_vp, _vp, _pt, _i, _i, _pb, _sz, _pb, _sz, _i, _b]),
    ("qw_path_qmv_ggm", _b, [_vp, _vp, _vp, _vp, _i, _i, _pb, _vp, _i, _b]),
    ("qw_path_gg_router", _b, [_vp, _vp, _pm, _i, _pb, _pb]),
    ("qw_path_gg_moe", _b, [_vp, _vp, _pm, _i, _pb, _pb, _pb, _pb]),
    ("qw_path_gg_moe_lg", _b, [_vp, _vp, _pm, _i, _pb, _pb, _pb, _pb]),
    ("qw_path_gg_moe_stack", _b, [_vp, _vp, _pm, _i, _i, _pb, _pb, _pb, _pb]), ("qw_path_set_flush", None, [_vp, C.c_uint64]),
    ("qw_path_scratch", _pb, [_vp, _i]),
    ("qw_path_hyper_pd_bytes", _sz, [_i]),
    ("qw_path_hyper_moe_stack", _b, [_vp, _vp, C.POINTER(QwHyperW), _pm, _i, _i, _b, _pb, _pb, _pb, _pb, _pb, _pb, _pb]),
    ("qw_path_hyper_gg", _b, [_vp, _vp, C.POINTER(QwHyperW), _i, _b, _b, _pb, _pb, _pb, _pb, _pb, _pb]),
    ("qw_path_par_vstep", _b, [_vp, _vp, _pm, _pi, _i, _pb, _pb, C.POINTER(QwVstepInfo)]),
    ("qw_path_gg_moe_noalloc", _b, [_vp, _i, _i, _i, _i, C.POINTER(QwMoeWeightsDev), _i, _vp, _vp, _vp]),
    ("qw_path_pf_reserve", _b, [_vp, _i, _i]), ("qw_path_pf_moe", _b, [_vp, _vp, _pm, _i, _pb, _pb, _pb, _pb]),
    ("qw_path_pf_scratch", _pb, [_vp, _i]), ("qw_path_pf_max_tiles", C.c_uint, [_vp]),
    # qw_gguf.h
    ("qw_gguf_parse_parts", _u, [C.c_char_p]), ("qw_ggml_block", _b, [_i, _pi, _pi]), ("qw_ggml_name", C.c_char_p, [_i]),
    ("qw_gguf_open", _vp, [C.c_char_p, C.c_char_p, _sz]), ("qw_gguf_close", None, [_vp]), ("qw_gguf_shards", _i, [_vp]),
    ("qw_gguf_shard_path", C.c_char_p, [_vp, _i]), ("qw_gguf_shard_alignment", C.c_uint32, [_vp, _i]),
    ("qw_gguf_shard_data_start", C.c_uint64, [_vp, _i]), ("qw_gguf_count", _i, [_vp]), ("qw_gguf_get", _pg, [_vp, _i]),
    ("qw_gguf_find", _pg, [_vp, C.c_char_p]), ("qw_gguf_host", _vp, [_vp, _pg]),
    ("qw_gguf_load", _b, [_vp, _vp, _u, C.c_char_p, _sz]), ("qw_gguf_resident_bytes", _sz, [_vp]), ("qw_gguf_load_seconds", _d, [_vp]),
    ("qw_gguf_release_source", _b, [_vp, C.c_char_p, _sz]),
    ("qw_gguf_hyper", _b, [_vp, _i, _i, C.POINTER(QwHyperW), _pi, C.c_char_p, _sz]),
    ("qw_gguf_tensor_at", _b, [_vp, _pg, _pt]), ("qw_gguf_moe_layer", _b, [_vp, _i, _pm, _pi, _pi, _pi, C.c_char_p, _sz]),
    # qw_par.h
    ("qw_par_new", _vp, []), ("qw_par_free", None, [_vp]), ("qw_par_observe", None, [_vp, _i, _d]), ("qw_par_group_cost", _d, [_vp, _i]),
    ("qw_par_cost", _d, [_vp, _i]), ("qw_par_split", _i, [_vp, _i, _pi]), ("qw_par_observe_packed", None, [_vp, _i, _d]),
    ("qw_par_packed_cost", _d, [_vp, _i]), ("qw_par_choose", _b, [_vp, _i, _pi, _pi]),
    ("qw_par_want_slice", _b, [_vp, _i, _b, _d, C.POINTER(_d), _d, _d]),
]


def load_lib():
    """Load the built library; raises if it has not been built (python -m qwental_amd.build)."""
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(lib_path()):
        raise RuntimeError("libqwgpu_hip.so is not built: run `python -m qwental_amd.build` (needs hipcc and clang from ROCm)")
    L = C.CDLL(lib_path())
    for name, res, args in SYMBOLS:
        if os.environ.get("QW_HIP_LIB") and not hasattr(L, name):
            continue  # another build of the library (experiments) may predate a symbol
        f = getattr(L, name)  # AttributeError if the library lacks a declared symbol
        f.restype = res
        f.argtypes = args
    _lib = L
    return L


def compile_check(defs):
    """(ok, error text, kernel names) of a define block, without a device."""
    L = load_lib()
    err, names = C.create_string_buffer(4096), C.create_string_buffer(4096)
    src = defs.encode()
    ok = L.qw_hip_compile_check(src, len(src), err, len(err), names, len(names))
    return ok, err.value.decode(), [n for n in names.value.decode().split(",") if n]


class Buf:
    """A qw_buf plus a numpy view of its host shadow."""

    def __init__(self, gpu, size, device_only=False, wrap=None):
        self.gpu, self.L = gpu, gpu.L
        self.c = QwBuf()
        self._keep = wrap
        if wrap is not None:
            ok = self.L.qw_buf_wrap(gpu.g, wrap.ctypes.data, wrap.nbytes, C.byref(self.c))
        elif device_only:
            ok = self.L.qw_hip_buf_new_device(gpu.g, size, C.byref(self.c))
        else:
            ok = self.L.qw_buf_new(gpu.g, size, C.byref(self.c))
        if not ok:
            raise MemoryError("qw_buf allocation of %d bytes failed: %s" % (size, gpu.last_error()))
        self.size = self.c.size

    def view(self, dtype=np.uint8):
        if not self.c.ptr:
            raise ValueError("device-only buffer has no host view")
        raw = (C.c_uint8 * self.size).from_address(self.c.ptr)
        return np.frombuffer(raw, dtype=np.uint8).view(dtype)

    def fill(self, arr, offset=0):
        """Copy a numpy array into the buffer (shadow for host-visible buffers, HBM for device-only ones)."""
        a = np.ascontiguousarray(arr)
        if offset + a.nbytes > self.size:
            raise ValueError("fill beyond the buffer")
        if self.c.ptr and self._keep is None:
            self.view()[offset:offset + a.nbytes] = a.view(np.uint8).ravel()
            self.L.qw_hip_buf_mark_dirty(C.byref(self.c))
        elif not self.L.qw_hip_buf_write(C.byref(self.c), offset, a.ctypes.data, a.nbytes):
            raise RuntimeError("qw_hip_buf_write failed")

    def read(self, nbytes=None, offset=0, dtype=np.uint8):
        """Bytes straight from HBM (independent of the shadow rules)."""
        n = self.size - offset if nbytes is None else nbytes
        out = np.empty(n, np.uint8)
        if not self.L.qw_hip_buf_read(C.byref(self.c), offset, out.ctypes.data, n):
            raise RuntimeError("qw_hip_buf_read failed")
        return out.view(dtype)

    def free(self):
        if self.c.handle:
            self.L.qw_buf_free(C.byref(self.c))

    def ref(self):
        return C.byref(self.c)


class SelRecord:
    """The selection record a layer leaves (kernels/moe_gg.metal:110-116 of the reference; QW_SEL_* in csrc/kernels/qw_kargs.h):
    U | ue[GU] | mask[GU] | slot[GU][gnb] | w[gnb][topk + 1] with GU = gnb * topk; gnb = 8 for up to 8 tokens, else 16."""

    def __init__(self, raw, gnb, topk):
        gu = gnb * topk
        raw = np.ascontiguousarray(raw, np.uint8)
        self.gnb, self.topk = gnb, topk
        self.U = int(raw[:4].view(np.uint32)[0])
        self.ue = raw[4:4 + 4 * gu].view(np.uint32)
        self.mask = raw[4 + 4 * gu:4 + 8 * gu].view(np.uint32)
        o = 4 + 8 * gu
        self.slot = raw[o:o + gu * gnb].reshape(gu, gnb)
        o += gu * gnb
        self.w = raw[o:o + 4 * gnb * (topk + 1)].view(np.float32).reshape(gnb, topk + 1)


class Tensor:
    def __init__(self, buf, ftype, offset=0):
        self.buf, self.ftype, self.offset = buf, ftype, offset

    def c(self):
        return QwTensor(C.pointer(self.buf.c), self.offset, self.ftype)


class MoeLayer:
    """Weights of one layer as tensors in HBM. Fields as in include/qw_path.h."""

    def __init__(self, **t):
        self.t = t
        self.c = QwMoeLayer(*[t[n].c() for n, _ in QwMoeLayer._fields_])


class Batch:
    def __init__(self, gpu, concurrent=False):
        self.gpu, self.L = gpu, gpu.L
        self.b = self.L.qw_batch_begin(gpu.g, concurrent)

    def kernel(self, k):
        self.L.qw_batch_kernel(self.b, k)

    def buf(self, index, buf, offset=0):
        self.L.qw_batch_buf(self.b, index, buf.ref(), offset)

    def bytes(self, index, arr):
        a = np.ascontiguousarray(arr)
        self.L.qw_batch_bytes(self.b, index, a.ctypes.data, a.nbytes)

    def dispatch(self, gx, gy=1, gz=1, tx=1, ty=1, tz=1):
        self.L.qw_batch_dispatch(self.b, gx, gy, gz, tx, ty, tz)

    def flush(self):
        self.L.qw_batch_flush(self.b)

    def end(self, check=True):
        t = self.L.qw_batch_end(self.b)
        self.b = None
        if check and t < 0:
            raise RuntimeError("GPU batch failed: " + self.gpu.last_error())
        return t


class Gpu:
    def __init__(self):
        self.L = load_lib()
        self.g = self.L.qw_gpu_open()
        if not self.g:
            raise RuntimeError("qw_gpu_open: no usable gfx950 device")

    def close(self):
        if self.g:
            self.L.qw_gpu_close(self.g)
            self.g = None

    def name(self):
        return self.L.qw_gpu_name(self.g).decode()

    def cu_count(self):
        return self.L.qw_hip_cu_count(self.g)

    def last_error(self):
        return self.L.qw_hip_last_error(self.g).decode()

    def compile(self, defs):
        err = C.create_string_buffer(8192)
        src = defs.encode()
        ok = self.L.qw_gpu_compile(self.g, src, len(src), err, len(err))
        return ok, err.value.decode()

    def kernel(self, name):
        return self.L.qw_kernel_get(self.g, name.encode())

    def buf(self, size, device_only=False):
        return Buf(self, size, device_only=device_only)

    def buf_from(self, arr, device_only=False):
        a = np.ascontiguousarray(arr)
        b = Buf(self, max(a.nbytes, 16), device_only=device_only)
        b.fill(a)
        return b

    def wrap(self, arr):
        return Buf(self, arr.nbytes, wrap=arr)

    def batch(self, concurrent=False):
        return Batch(self, concurrent)

    def profile(self, on):
        self.L.qw_profile_enable(self.g, on)

    @contextlib.contextmanager
    def switches(self, **env):
        """Measurement switches of include/qw_hip_ext.h for the batches begun inside the block: QW_HIP_<NAME> is set to the
        value given (None: unset), the device reads its switches again, and both are put back afterwards. The library
        reads the environment only when a device is opened or asked to."""
        old = {}
        for k, v in env.items():
            name = "QW_HIP_" + k.upper()
            old[name] = os.environ.get(name)
            if v is None:
                os.environ.pop(name, None)
            else:
                os.environ[name] = str(v)
        self.L.qw_hip_reload_switches(self.g)
        try:
            yield
        finally:
            for name, v in old.items():
                if v is None:
                    os.environ.pop(name, None)
                else:
                    os.environ[name] = v
            self.L.qw_hip_reload_switches(self.g)

    def profile_entries(self, entry_points=True):
        """(name, microseconds) per launch of the last profiled batch; entry-point names, or the callers' kernel names."""
        out = []
        us = C.c_double()
        get = self.L.qw_hip_profile_entry if entry_points else self.L.qw_profile_get
        for i in range(self.L.qw_profile_count(self.g)):
            n = get(self.g, i, C.byref(us))
            out.append((n.decode(), us.value))
        return out

    def profile_mean(self, prefix):
        n = C.c_int()
        s = self.L.qw_hip_profile_mean(self.g, prefix.encode(), C.byref(n))
        return s, n.value


class Path:
    """Host side of the path (include/qw_path.h)."""

    def __init__(self, gpu, D, I, E, topk, nbmax, device_scratch=False):
        self.gpu, self.L = gpu, gpu.L
        self.D, self.I, self.E, self.topk, self.nbmax = D, I, E, topk, nbmax
        self.p = self.L.qw_path_open(gpu.g, D, I, E, topk, nbmax, device_scratch)
        if not self.p:
            raise RuntimeError("qw_path_open failed: " + gpu.last_error())

    def close(self):
        if self.p:
            self.L.qw_path_close(self.p)
            self.p = None

    def sel_bytes(self, nb):
        return self.L.qw_path_sel_bytes(self.p, nb)

    def logits_bytes(self, nb):
        return self.L.qw_path_logits_bytes(self.p, nb)

    def qmv_gg(self, batch, W, N, K, x, y, nb, fout=True, xoff=0, yoff=0):
        t = W.c()
        if not self.L.qw_path_qmv_gg(self.p, batch.b, C.byref(t), N, K, x.ref(), xoff, y.ref(), yoff, nb, fout):
            raise RuntimeError("qw_path_qmv_gg failed")

    def qmv_ggm(self, batch, Ws, Ns, K, x, ys, nb, fout=True):
        """Up to four matrices (Tensor list) over the same x in one launch; ys: one output buffer per matrix."""
        n = len(Ws)
        wt = (QwTensor * n)(*[w.c() for w in Ws])
        na = (C.c_int * n)(*Ns)
        ya = (C.POINTER(QwBuf) * n)(*[C.pointer(y.c) for y in ys])
        if not self.L.qw_path_qmv_ggm(self.p, batch.b, wt, na, n, K, x.ref(), ya, nb, fout):
            raise RuntimeError("qw_path_qmv_ggm failed")

    def gg_router(self, batch, layer, nb, x, lg):
        if not self.L.qw_path_gg_router(self.p, batch.b, C.byref(layer.c), nb, x.ref(), lg.ref()):
            raise RuntimeError("qw_path_gg_router failed")

    def gg_moe(self, batch, layer, nb, x, lg, sel, out):
        if not self.L.qw_path_gg_moe(self.p, batch.b, C.byref(layer.c), nb, x.ref(), lg.ref(), sel.ref(), out.ref()):
            raise RuntimeError("qw_path_gg_moe failed")

    def gg_moe_lg(self, batch, layer, nb, x, lg, sel, out):
        """The layer with the caller's logits (forced routing)."""
        if not self.L.qw_path_gg_moe_lg(self.p, batch.b, C.byref(layer.c), nb, x.ref(), lg.ref(), sel.ref(), out.ref()):
            raise RuntimeError("qw_path_gg_moe_lg failed")

    def hyper_gg(self, batch, H, nb, apply, h, out, inj, inj_out, pd, x, three=False):
        """H: dict of Tensor (hc_norm, mix_down, mix_up and, optionally, inject)."""
        w = QwHyperW()
        for n in ("hc_norm", "mix_down", "mix_up", "inject"):
            if H.get(n) is not None:
                setattr(w, n, H[n].c())
        ok = self.L.qw_path_hyper_gg(self.p, batch.b, C.byref(w), nb, bool(apply), bool(three), h.ref(), out.ref(), inj.ref(),
                                     inj_out.ref() if inj_out is not None else None, pd.ref(), x.ref())
        if not ok:
            raise RuntimeError("qw_path_hyper_gg failed: " + self.gpu.last_error())

    def hyper_moe_stack(self, batch, hyper_c, layers_c, nlayers, nb, pending, h, inj_c, pd, x, lg_c, sel_c, out):
        if not self.L.qw_path_hyper_moe_stack(self.p, batch.b, hyper_c, layers_c, nlayers, nb, bool(pending), h.ref(), inj_c, pd.ref(), x.ref(), lg_c, sel_c, out.ref()):
            raise RuntimeError("qw_path_hyper_moe_stack failed: " + self.gpu.last_error())

    def set_flush(self, mask):
        self.L.qw_path_set_flush(self.p, mask)

    def gg_moe_stack(self, batch, layers_c, nlayers, nb, x, lg_c, sel_c, out):
        """layers_c: ctypes array of QwMoeLayer; lg_c / sel_c: ctypes arrays of QwBuf, one per layer."""
        if not self.L.qw_path_gg_moe_stack(self.p, batch.b, layers_c, nlayers, nb, x.ref(), lg_c, sel_c, out.ref()):
            raise RuntimeError("qw_path_gg_moe_stack failed")

    def par_vstep(self, par, layer, n, x, out):
        """A ragged step (slot i: n[i] rows) cut by the planner `par`; returns the QwVstepInfo of the cut."""
        na = (C.c_int * len(n))(*[int(v) for v in n])
        info = QwVstepInfo()
        if not self.L.qw_path_par_vstep(self.p, par.p, C.byref(layer.c), na, len(n), x.ref(), out.ref(), C.byref(info)):
            raise RuntimeError("qw_path_par_vstep failed: " + self.gpu.last_error())
        return info

    def pf_reserve(self, tmax, tm):
        if not self.L.qw_path_pf_reserve(self.p, tmax, tm):
            raise RuntimeError("qw_path_pf_reserve failed: " + self.gpu.last_error())

    def pf_moe(self, batch, layer, T, x, ids, w, out):
        """Ragged batch through the packing path: ids / w are [T * topk] uint32 / float32 buffers."""
        if not self.L.qw_path_pf_moe(self.p, batch.b, C.byref(layer.c), T, x.ref(), ids.ref(), w.ref(), out.ref()):
            raise RuntimeError("qw_path_pf_moe failed")

    def pf_scratch(self, which, dtype=np.uint8):
        """0 counts, 1 offsets, 2 tile table, 3 pos_of, 4 packed x, 5 H, 6 packed down output (device bytes)."""
        pb = self.L.qw_path_pf_scratch(self.p, which)
        out = np.empty(pb.contents.size, np.uint8)
        if not self.L.qw_hip_buf_read(pb, 0, out.ctypes.data, out.nbytes):
            raise RuntimeError("qw_hip_buf_read failed")
        return out.view(dtype)

    def pf_max_tiles(self):
        return int(self.L.qw_path_pf_max_tiles(self.p))

    def scratch(self, which):
        """0 = lookup tables, 1 = H, 2 = Psh, 3 = Pg; returns (device bytes as uint8)."""
        pb = self.L.qw_path_scratch(self.p, which)
        out = np.empty(pb.contents.size, np.uint8)
        if not self.L.qw_hip_buf_read(pb, 0, out.ctypes.data, out.nbytes):
            raise RuntimeError("qw_hip_buf_read failed")
        return out


class Gguf:
    """include/qw_gguf.h: the *.gguf files of a directory, parsed and mapped; load() makes the chosen parts resident."""

    def __init__(self, directory):
        self.L = load_lib()
        err = C.create_string_buffer(1024)
        self.f = self.L.qw_gguf_open(os.fsencode(directory), err, len(err))
        if not self.f:
            raise ValueError(err.value.decode())

    def close(self):
        if self.f:
            self.L.qw_gguf_close(self.f)
            self.f = None

    def shards(self):
        n = self.L.qw_gguf_shards(self.f)
        return [dict(path=os.fsdecode(self.L.qw_gguf_shard_path(self.f, i)), alignment=self.L.qw_gguf_shard_alignment(self.f, i),
                     data_start=self.L.qw_gguf_shard_data_start(self.f, i)) for i in range(n)]

    def __len__(self):
        return self.L.qw_gguf_count(self.f)

    def get(self, i):
        p = self.L.qw_gguf_get(self.f, i)
        return p.contents if p else None

    def find(self, name):
        p = self.L.qw_gguf_find(self.f, name.encode())
        return p.contents if p else None

    def host(self, t):
        """The tensor's bytes in the mapping of its file (a copy)."""
        a = self.L.qw_gguf_host(self.f, C.byref(t))
        if not a:
            return None
        return np.frombuffer((C.c_uint8 * t.nbytes).from_address(a), np.uint8).copy()

    def load(self, gpu, parts="all"):
        err = C.create_string_buffer(1024)
        bits = parts if isinstance(parts, int) else self.L.qw_gguf_parse_parts(parts.encode())
        if not self.L.qw_gguf_load(self.f, gpu.g, bits, err, len(err)):
            raise RuntimeError(err.value.decode())

    def resident_bytes(self):
        return self.L.qw_gguf_resident_bytes(self.f)

    def load_seconds(self):
        return self.L.qw_gguf_load_seconds(self.f)

    def tensor_at(self, t):
        """QwTensor (buffer, offset, type) of a resident tensor, or None."""
        out = QwTensor()
        return out if self.L.qw_gguf_tensor_at(self.f, C.byref(t), C.byref(out)) else None

    def read_resident(self, t, nbytes):
        """nbytes of the tensor's resident copy, read back from HBM."""
        at = self.tensor_at(t)
        if at is None:
            return None
        out = np.empty(nbytes, np.uint8)
        if not self.L.qw_hip_buf_read(at.buf, at.offset, out.ctypes.data, nbytes):
            raise RuntimeError("qw_hip_buf_read failed")
        return out

    def moe_layer(self, layer):
        """(QwMoeLayer, D, I, E) of blk.<layer>; the struct points into this object's arena."""
        M, D, I, E = QwMoeLayer(), C.c_int(), C.c_int(), C.c_int()
        err = C.create_string_buffer(1024)
        if not self.L.qw_gguf_moe_layer(self.f, layer, C.byref(M), C.byref(D), C.byref(I), C.byref(E), err, len(err)):
            raise ValueError(err.value.decode())
        return M, D.value, I.value, E.value

    def release_source(self):
        err = C.create_string_buffer(1024)
        if not self.L.qw_gguf_release_source(self.f, err, len(err)):
            raise ValueError(err.value.decode())

    def hyper(self, layer, which):
        """(HyperW, D) of blk.<layer>.hc_attn_* (which 0), hc_ffn_* (1) or the output mixer (2)."""
        H, D = QwHyperW(), C.c_int()
        err = C.create_string_buffer(1024)
        if not self.L.qw_gguf_hyper(self.f, layer, which, C.byref(H), C.byref(D), err, len(err)):
            raise ValueError(err.value.decode())
        return HyperW(H), D.value


class HyperW:
    """A QwHyperW filled by the GGUF reader, in the form Path.hyper_gg takes."""

    def __init__(self, c):
        self.c = c

    def get(self, name):
        t = getattr(self.c, name)
        return _Fixed(t) if t.buf else None

    def __getitem__(self, name):
        return self.get(name)


class _Fixed:
    def __init__(self, t):
        self.t = t

    def c(self):
        return self.t


class Par:
    """include/qw_par.h: the cut of a step into groups (or the packing path) from measured times."""

    def __init__(self):
        self.L = load_lib()
        self.p = self.L.qw_par_new()

    def free(self):
        if self.p:
            self.L.qw_par_free(self.p)
            self.p = None

    def observe(self, b, ms):
        self.L.qw_par_observe(self.p, b, ms)

    def group_cost(self, b):
        return self.L.qw_par_group_cost(self.p, b)

    def cost(self, B):
        return self.L.qw_par_cost(self.p, B)

    def split(self, B):
        g = (C.c_int * 64)()
        return list(g[:self.L.qw_par_split(self.p, B, g)])

    def observe_packed(self, rows, ms):
        self.L.qw_par_observe_packed(self.p, rows, ms)

    def packed_cost(self, rows):
        return self.L.qw_par_packed_cost(self.p, rows)

    def choose(self, rows):
        """(use the packing path, group sizes otherwise)."""
        g, n = (C.c_int * 64)(), C.c_int()
        packed = self.L.qw_par_choose(self.p, rows, g, C.byref(n))
        return bool(packed), list(g[:n.value])

    def want_slice(self, n, slicing_now, sliced_rate=0.0, solo_rates=None, solo_default=0.0, batched_rate=0.0):
        """Time slices (True) or a joint step (False) for n decoding conversations; rates in tokens/s, 0 = not measured."""
        arr = (C.c_double * max(n, 1))(*(list(solo_rates) + [0.0] * n)[:max(n, 1)]) if solo_rates is not None else None
        return bool(self.L.qw_par_want_slice(self.p, n, slicing_now, sliced_rate, arr, solo_default, batched_rate))
