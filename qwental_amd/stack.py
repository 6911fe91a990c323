"""The MoE FFN stack of the benchmark: L layers of the synthetic layer shape, every layer with its own weights
resident in HBM (device-only buffers filled by the library's block generator), decoded for nb tokens per step.

Mixed quantisation: with q8_every = 4, layers 3, 7, 11, ... carry their shared expert's three projections in Q8_0
and everything else in IQ3_S — the reference's SC117 recipe puts Q8_0 on the shared / dense projections only
(CHANGELOG.md:154), which keeps the stack near 33 GB.
"""
import ctypes as C

import numpy as np

from . import synth
from .gpu import Buf, MoeLayer, Path, QwBuf, QwHyperW, QwMoeLayer, Tensor

MEM_DEFS = "#define QW_HIP_MEM 1\n"


def fill_blocks(gpu, batch, buf, offset, nblocks, ftype, seed, sigma):
    ok, err = gpu.compile(MEM_DEFS)
    if not ok:
        raise RuntimeError(err)
    batch.kernel(gpu.kernel("qw_fill_blocks"))
    batch.buf(1, buf, offset)
    a = np.zeros(1, np.dtype([("n", "<u8"), ("seed", "<u8"), ("type", "<u4"), ("sigma", "<f4")]))
    a["n"], a["seed"], a["type"], a["sigma"] = nblocks, seed, ftype, sigma
    batch.bytes(2, a)
    batch.dispatch(1)


class MoeStack:
    """model_formats: None for the benchmark's layer (IQ3_S throughout, Q8_0 shared expert every q8_every-th layer), or
    (routed down, shared gate, shared up, shared down) ggml types for a layer of other formats — (20, 12, 23, 20) with
    D = 2560, I = 640 is the reference model's layer (src/model.h:10-18, bench/moe_bw.c:16-24). The routed rows are
    generated on the device, a shared expert of other formats on the host."""

    def __init__(self, gpu, layers=48, D=2048, I=512, E=512, topk=10, nbmax=16, q8_every=4, seed=1234, d_scale=synth.MOE_D_SCALE, model_formats=None):
        self.gpu, self.L, self.D, self.I, self.E, self.topk, self.nbmax = gpu, layers, D, I, E, topk, nbmax
        self.path = Path(gpu, D, I, E, topk, nbmax, device_scratch=True)
        rng = np.random.default_rng(seed)
        self.fd = fd = model_formats[0] if model_formats else 21
        rb_gu, rb_d = synth.row_bytes(21, D), synth.row_bytes(fd, I)
        self.exp_bytes = 2 * I * rb_gu + D * rb_d           # one routed expert
        self.gu_bytes = 2 * I * rb_gu
        self.layers, self.bufs, self.shared_fmt = [], [], []
        self.router_bytes = (E + 1) * D * 2
        sigma = lambda f: (synth.D_SIGMA[f] if f in synth.D_SIGMA else synth.SCALE_FIELDS[f][1]) * d_scale
        b = gpu.batch()
        for l in range(layers):
            fsh = 8 if q8_every and l % q8_every == q8_every - 1 else 21
            fs3 = tuple(model_formats[1:]) if model_formats else (fsh, fsh, fsh)
            sz_gu, sz_d = E * I * rb_gu, E * D * rb_d         # gate and up each; down
            sh_g, sh_u, sh_d = I * synth.row_bytes(fs3[0], D), I * synth.row_bytes(fs3[1], D), D * synth.row_bytes(fs3[2], I)
            w = gpu.buf(2 * sz_gu + sz_d, device_only=True)
            fill_blocks(gpu, b, w, 0, 2 * sz_gu // 110, 21, seed * 1000003 + l * 7919, sigma(21))
            fill_blocks(gpu, b, w, 2 * sz_gu, sz_d // synth.BLOCK[fd][1], fd, seed * 1000003 + l * 7919 + 2, sigma(fd))
            if model_formats:
                hr = np.random.default_rng(seed * 31 + l)
                sh = gpu.buf_from(np.concatenate([synth.matrix(hr, fs3[0], I, D, d_scale), synth.matrix(hr, fs3[1], I, D, d_scale), synth.matrix(hr, fs3[2], D, I, d_scale)]), device_only=True)
            else:
                sh = gpu.buf(sh_g + sh_u + sh_d, device_only=True)
                fill_blocks(gpu, b, sh, 0, (sh_g + sh_u + sh_d) // synth.BLOCK[fsh][1], fsh, seed * 1000003 + l * 7919 + 1, sigma(fsh))
            Wr, wsg = synth.router(rng, E, D)
            r = gpu.buf_from(np.concatenate([Wr.ravel(), wsg]).view(np.uint16), device_only=True)
            T = Tensor
            self.layers.append(MoeLayer(router=T(r, 1), sh_gate_w=T(r, 1, E * D * 2), gate=T(w, 21), up=T(w, 21, sz_gu), down=T(w, fd, 2 * sz_gu),
                                        sh_gate=T(sh, fs3[0]), sh_up=T(sh, fs3[1], sh_g), sh_down=T(sh, fs3[2], sh_g + sh_u)))
            self.bufs += [w, sh, r]
            self.shared_fmt.append(fs3)
        b.end()
        self.layers_c = (QwMoeLayer * layers)(*[m.c for m in self.layers])
        self.lg = [gpu.buf(self.path.logits_bytes(nbmax), device_only=True) for _ in range(layers)]
        self.sel = [gpu.buf(self.path.sel_bytes(nbmax), device_only=True) for _ in range(layers)]
        self.lg_c = (QwBuf * layers)(*[x.c for x in self.lg])
        self.sel_c = (QwBuf * layers)(*[x.c for x in self.sel])
        self.out = gpu.buf(nbmax * D * 2)
        self.bufs += self.lg + self.sel + [self.out]
        self.weight_bytes = sum(x.size for x in self.bufs[:3 * layers])

    def add_hyper(self, seed=99):
        """A hyper-connection in front of every layer (GGUF profile: F32 norm weights, BF16 mix_down / mix_up / inject): one
        drawn set of weights, rotated by a different amount for every layer, plus the buffers of the step."""
        gpu, D, L = self.gpu, self.D, self.L
        w = synth.hyper_weights(np.random.default_rng(seed), D)
        self.hyper_host, self.hyper_bufs, hw = [], [], []
        for l in range(L):
            wl = {k: np.roll(v.ravel(), 977 * l).reshape(v.shape) for k, v in w.items()}
            bufs = {k: gpu.buf_from(v, device_only=True) for k, v in wl.items()}
            c = QwHyperW()
            for k in ("hc_norm", "mix_down", "mix_up", "inject"):
                setattr(c, k, Tensor(bufs[k], 0 if k == "hc_norm" else 30).c())
            hw.append(c)
            self.hyper_host.append(wl)
            self.hyper_bufs += list(bufs.values())
        self.hyper_c = (QwHyperW * L)(*hw)
        nb = self.nbmax
        self.h = gpu.buf(nb * 4 * D * 4)
        self.inj = [gpu.buf(nb * 16 * 4), gpu.buf(nb * 16 * 4)]
        self.inj_c = (QwBuf * 2)(*[x.c for x in self.inj])
        self.pd = gpu.buf(int(gpu.L.qw_path_hyper_pd_bytes(nb)), device_only=True)
        self.x = gpu.buf(nb * D * 2)
        self.hyper_bufs += [self.h, self.pd, self.x] + self.inj
        self.hyper_bytes = sum(v.nbytes for v in w.values())
        return self

    def step_hyper(self, nb, nlayers=None, pending=False):
        """One decode step of the FFN halves: hyper-connection -> MoE layer, layer after layer, on the streams in self.h and the
        inject sums in self.inj[0]; returns GPU seconds."""
        b = self.gpu.batch()
        self.path.hyper_moe_stack(b, self.hyper_c, self.layers_c, self.L if nlayers is None else nlayers, nb, pending, self.h, self.inj_c, self.pd, self.x,
                                  self.lg_c, self.sel_c, self.out)
        return b.end()

    def release_sources(self):
        """Keep only the tile-major copies of the routed experts' matrices (made by the first step): frees the GGUF-order
        bytes of every layer's routed weights. Returns the bytes freed. The weights can no longer be read back."""
        before = self.gpu.L.qw_hip_released_bytes(self.gpu.g)
        for l in range(self.L):
            w = self.bufs[3 * l]
            if not self.gpu.L.qw_hip_buf_release_source(w.ref()):
                raise RuntimeError("layer %d: no tile-major copy to keep (run a step first)" % l)
        return int(self.gpu.L.qw_hip_released_bytes(self.gpu.g) - before)

    def shared_bytes(self, l):
        f = self.shared_fmt[l]
        return self.I * (synth.row_bytes(f[0], self.D) + synth.row_bytes(f[1], self.D)) + self.D * synth.row_bytes(f[2], self.I)

    def step(self, x, nb, nlayers=None):
        """One decode step over the stack; returns GPU seconds (events around the kernels)."""
        b = self.gpu.batch()
        self.path.gg_moe_stack(b, self.layers_c, self.L if nlayers is None else nlayers, nb, x, self.lg_c, self.sel_c, self.out)
        return b.end()

    def unique_experts(self, nb):
        """U per layer, read from the selection records of the last step."""
        return [int(s.read(4).view(np.uint32)[0]) for s in self.sel]

    def algorithmic_bytes(self, nb, U):
        """Per layer: router + (U_l + 1 shared) experts + activations in and out (the reference's accounting,
        src/engine.c:8020-8038, with U distinct experts for the routed part)."""
        return [self.router_bytes + U[l] * self.exp_bytes + self.shared_bytes(l) + nb * self.D * 4 for l in range(self.L)]

    def layer_weights_host(self, l):
        """The layer's weights copied back from HBM, as the dict the oracle takes (bytes exactly as resident)."""
        w, sh, r = self.bufs[3 * l:3 * l + 3]
        E, I, D = self.E, self.I, self.D
        sz_e = E * I * synth.row_bytes(21, D)
        f = self.shared_fmt[l]
        sh_g, sh_u = I * synth.row_bytes(f[0], D), I * synth.row_bytes(f[1], D)
        wb, sb, rb = w.read(), sh.read(), r.read(dtype=np.uint16)
        return dict(D=D, I=I, E=E, topk=self.topk, fgu=21, fd=self.fd, fsg=f[0], fsu=f[1], fsd=f[2], Wg=wb[:sz_e], Wu=wb[sz_e:2 * sz_e], Wd=wb[2 * sz_e:],
                    Wsg=sb[:sh_g], Wsu=sb[sh_g:sh_g + sh_u], Wsd=sb[sh_g + sh_u:], Wr=rb[:E * D].view(np.float16).reshape(E, D), wsg=rb[E * D:].view(np.float16))

    def free(self):
        for b in self.bufs + getattr(self, "hyper_bufs", []):
            b.free()
        self.path.close()
