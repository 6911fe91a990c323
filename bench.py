#!/usr/bin/env python3
"""Benchmark of the batched IQ3_S MoE decode path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--layers 48] [--nb 16]

Workload (BASELINE.json configs[4]): the 48-layer MoE FFN stack decode step at B = 16 — hidden 2048, 512 experts of
gate/up 2 x (512 x 2048) and down 2048 x 512 in IQ3_S plus one shared expert per layer, top-10 routing by each
layer's own binary16 router on x ~ N(0, 1), every 4th layer's shared-expert projections in Q8_0; about 33 GB of
weights resident in HBM, generated on the device (seeded). One step = one pass of the stack over one batch of 16
tokens. The timed region holds exactly K steps between device synchronisations; inputs are resident before it.

Prints one JSON line: tokens/s (whole job, one GPU), the HBM roofline of the dominant kernel (routed gate/up),
and the CPU oracle timed on a bounded sample of the same layers on this machine's cores.
"""
import argparse
import json
import os
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0  # MI355X published HBM3E bandwidth
DOMINANT = "qwk_gu_f"


def timed_steps(stack, x, nb, steps, warmup):
    for _ in range(warmup):
        stack.step(x, nb)
    stack.gpu.L.qw_gpu_empty_commit_latency(stack.gpu.g, None, 1)  # drains the stream (event record + synchronise)
    t0 = time.perf_counter()
    gpu_s = 0.0
    for _ in range(steps):
        gpu_s += stack.step(x, nb)
    stack.gpu.L.qw_gpu_empty_commit_latency(stack.gpu.g, None, 1)
    return time.perf_counter() - t0, gpu_s


def model_shape_leg(gpu, layers, steps, warmup, cpu_check):
    """The same decode step on the reference model's own layer (src/model.h:10-18 and bench/moe_bw.c:16-24 of the
    reference): D = 2560, I = 640, 512 experts, top-10; routed gate/up IQ3_S, routed down IQ4_NL, shared expert Q4_K
    gate, IQ4_XS up, IQ4_NL down. Tokens/s, GPU time and algorithmic GB/s per batch size and mean launch times at
    B = 16. cpu_check (part of the CPU baseline leg: off under --no-cpu) also compares the layer-0 output at B = 16
    with the CPU oracle's while the stack is resident; main() files that figure under cpu_baseline."""
    from qwental_amd import synth
    from qwental_amd.stack import MoeStack
    stack = MoeStack(gpu, layers=layers, D=2560, I=640, nbmax=16, model_formats=(20, 12, 23, 20))
    xh = synth.activations(np.random.default_rng(2025), 16, stack.D)
    x = gpu.buf_from(xh, device_only=True)
    res = {"workload": "%d-layer MoE FFN stack decode, D=2560 I=640 E=512 top-10; IQ3_S gate/up, IQ4_NL down; shared Q4_K / IQ4_XS / IQ4_NL" % layers,
           "resident_weight_bytes": int(stack.weight_bytes), "by_batch": {}}
    for _ in range(30):  # the legs before this one may have left the device idle for seconds: bring the clocks back up
        stack.step(x, 16)
    for nb in (1, 8, 16):
        wall, gpu_s = timed_steps(stack, x, nb, steps, warmup)
        U = stack.unique_experts(nb)
        byts = stack.algorithmic_bytes(nb, U)
        res["by_batch"][str(nb)] = {"tokens_per_s": nb * steps / wall, "gpu_ms_per_step": gpu_s / steps * 1e3, "stack_GBps": sum(byts) / (gpu_s / steps) / 1e9, "mean_U": float(np.mean(U))}
    gpu.profile(True)
    stack.step(x, 16)
    gpu.profile(False)
    per = {}
    for name, us in gpu.profile_entries():
        per.setdefault(name, []).append(us)
    res["kernel_us_mean"] = {k: float(np.mean(v)) for k, v in per.items()}
    if cpu_check:
        from oracle import oracle as o  # the checker of the CPU baseline leg
        # one 16-token step of the first layer alone: `out` is the last layer's otherwise
        stack.step(x, 16, nlayers=1)
        lg = stack.lg[0].read(dtype=np.float32)[:16 * (stack.E + 1)].reshape(16, stack.E + 1).copy()
        got = stack.out.view(np.float16)[:16 * stack.D].reshape(16, stack.D).astype(np.float64)
        ref = o.moe_layer_f64(stack.layer_weights_host(0), lg, xh)
        res["layer0_max_rel_err"] = float(np.abs(got - ref).max() / np.abs(ref).max())
    x.free()
    stack.free()
    return res


def ablation_leg(gpu, stack, x, nb, full_us):
    """Where the dominant launch's time goes, measured in this run: the launch as it is (full_us), the same launch without
    its arithmetic (QW_HIP_ABLATE: selection, table and activation staging, loads and stores stay; the decoding and the
    matrix instructions go; its results are meaningless and nothing here looks at them), and — from read_ceiling — a
    kernel that only reads the same bytes. Microseconds per launch, HIP events around every launch of one step."""
    with gpu.switches(ablate="1"):
        stack.step(x, nb)  # (warm: first use of that entry point)
        gpu.profile(True)
        stack.step(x, nb)
        gpu.profile(False)
        t, n = gpu.profile_mean("qwk_gu_f122")
    stack.step(x, nb)  # leaves the buffers as a real step leaves them
    return {"full_us": full_us, "without_arithmetic_us": t * 1e6 if n else None, "launches": n}


def committed_traffic():
    """HBM bytes per launch of the dominant kernel as the committed counter summary states them (two rocprofv3
    --pmc runs of this file with --copy-calib, FETCH_SIZE and WRITE_SIZE, scaled by the copy kernel); None without it."""
    try:
        for ln in open(os.path.join(ROOT, "profiles", "moe_stack_b16_hbm_traffic.txt")):
            if ln.startswith(DOMINANT + " traffic bytes per launch ="):
                return float(ln.split("=")[1])
    except OSError:
        pass
    return None


def copy_calibration(gpu, nbytes=1 << 30):
    """qwk_copy over nbytes: reads nbytes and writes nbytes, a dispatch of known traffic for the counter runs."""
    ok, err = gpu.compile("#define QW_HIP_MEM 1\n")
    assert ok, err
    src, dst = gpu.buf(nbytes, device_only=True), gpu.buf(nbytes, device_only=True)
    for _ in range(3):
        b = gpu.batch()
        b.kernel(gpu.kernel("qw_copy"))
        b.buf(0, src)
        b.buf(1, dst)
        b.bytes(2, np.array([nbytes // 16, 0], np.uint64))
        b.dispatch(256 * 16)
        b.end()
    src.free()
    dst.free()


def cpu_baseline(stack, x_dev, xh, nb, budget_s=20.0):
    """The CPU oracle (float dot products over dequantized rows, OpenMP over all cores) on the first layers of the
    same stack, timed; stops after about budget_s seconds of oracle time. Every sampled layer is also the full-size
    parity check of the benchmarked configuration: the stack call with l + 1 layers leaves layer l's output, which is
    compared with the oracle's (binary16 both), and the layer's picks with the oracle's own router and top-k."""
    from oracle import oracle as o
    cores = o.max_threads()
    t_used, n, worst, topk_ok = 0.0, 0, 0.0, True
    while t_used < budget_s and n < stack.L:
        stack.step(x_dev, nb, nlayers=n + 1)
        got = stack.out.view(np.float16)[:nb * stack.D].reshape(nb, stack.D).astype(np.float64)
        lg = stack.lg[n].read(dtype=np.float32)[:nb * (stack.E + 1)].reshape(nb, stack.E + 1).copy()
        m = stack.layer_weights_host(n)
        t0 = time.perf_counter()
        out32, _, _ = o.moe_layer_f32(m, lg, xh[:nb], 8 if nb <= 8 else 16)
        t_used += time.perf_counter() - t0
        ref = out32.astype(np.float64)
        worst = max(worst, float(np.abs(got - ref).max() / np.abs(ref).max()))
        topk_ok = topk_ok and bool(np.array_equal(o.topk_ids(lg, stack.topk), o.topk_ids(o.router(m["Wr"], m["wsg"], xh[:nb]), stack.topk)))
        n += 1
        del m
    per_layer = t_used / n
    return {"value": nb / (per_layer * stack.L), "unit": "tokens/s", "cores": cores, "kind": "port",
            "sample": "oracle moe_layer_f32 on layers 0..%d of the stack (B = %d), %.1f s; scaled to %d layers" % (n - 1, nb, t_used, stack.L),
            "max_rel_err": worst, "topk_identical": topk_ok, "layers_compared": n, "tolerance": 2e-3}


def read_ceiling(gpu, stack, nb, reps=5):
    """What this device gives a kernel that only reads (the method of bench/moe_bw.c:50-89 and kernels/ceiling_mem.metal of
    the reference): (a) the pure-read kernel over the resident gate/up rows of the experts the last step picked, one
    launch per layer over the same bytes the gate/up launch streams (one contiguous range per layer of the same
    size: the experts' rows themselves are contiguous pieces of 901,120 bytes); (b) the same kernel over 1 GiB; (c) the
    copy kernel over 1 GiB (read + write)."""
    ok, err = gpu.compile("#define QW_HIP_MEM 1\n")
    assert ok, err
    sink = gpu.buf(64, device_only=True)
    U = stack.unique_experts(nb)

    def timed(kernel, launches):
        best = 1e9
        for _ in range(reps):
            b = gpu.batch()
            b.kernel(gpu.kernel(kernel))
            for src, off, n, dst in launches:
                b.buf(0, src, off)
                b.buf(1, dst)
                b.bytes(2, np.array([n // 16, 0], np.uint64))
                b.dispatch(256 * 8)
            best = min(best, b.end())
        return best
    # (a) per layer: U_l experts' gate/up bytes out of the layer's weight buffer (each layer another 692 MB allocation)
    launches = [(stack.bufs[3 * l], 0, U[l] * stack.gu_bytes, sink) for l in range(stack.L)]
    t = timed("qw_bw_read", launches)
    out = {"gate_up_bytes_per_layer_GBps": sum(n for _, _, n, _ in launches) / t / 1e9, "us_per_launch": t / stack.L * 1e6}
    big, big2 = gpu.buf(1 << 30, device_only=True), gpu.buf(1 << 30, device_only=True)
    out["read_1GiB_GBps"] = (1 << 30) / timed("qw_bw_read", [(big, 0, 1 << 30, sink)]) / 1e9
    out["copy_1GiB_GBps_read_plus_write"] = 2 * (1 << 30) / timed("qw_copy", [(big, 0, 1 << 30, big2)]) / 1e9
    for bb in (sink, big, big2):
        bb.free()
    return out


def hyper_ffn_leg(gpu, stack, steps, warmup):
    """The FFN half of the decode loop with its layer-to-layer dependency: hyper-connection (GGUF profile: F32 norm, BF16
    mix_down / mix_up / inject) -> MoE layer, for every layer of the stack, at B = 1, 8, 16. Tokens/s and GPU time per
    step, and the mean launch times of the two hyper-connection kernels with the bytes they read."""
    from qwental_amd import synth
    stack.add_hyper()
    D = stack.D
    h0, _, inj0 = synth.hyper_state(np.random.default_rng(77), 16, D)
    res = {"workload": "%d x (hyper-connection HC=4 LR=320 -> MoE layer), D=%d" % (stack.L, D), "hyper_weight_bytes_per_layer": int(stack.hyper_bytes), "by_batch": {}}
    for nb in (1, 8, 16):
        def step():
            # the streams grow with every residual: every step starts from the same state
            stack.h.fill(h0)
            stack.inj[0].fill(inj0)
            return stack.step_hyper(nb)
        for _ in range(warmup):
            step()
        gpu_s, t0, wall = 0.0, 0.0, 0.0
        for _ in range(steps):
            stack.h.fill(h0)
            stack.inj[0].fill(inj0)
            t0 = time.perf_counter()
            gpu_s += stack.step_hyper(nb)
            wall += time.perf_counter() - t0
        gpu.profile(True)
        step()
        gpu.profile(False)
        per = {}
        for name, us in gpu.profile_entries():
            if name.startswith("qwk_hc"):
                per.setdefault(name, []).append(us)
        k = {n: float(np.mean(v)) for n, v in per.items()}
        kd = next((v for n, v in k.items() if n.startswith("qwk_hc_down")), None)
        # down reads mix_down and inject once, up reads mix_up once; h, out and the norm weights are small beside them
        lr, hc = 320, 4
        b_down, b_up = (lr + hc) * hc * D * 2 + nb * hc * D * 4 + hc * D * 4, hc * D * lr * 2 + nb * hc * D * 4
        res["by_batch"][str(nb)] = {"tokens_per_s": nb * steps / wall, "gpu_ms_per_step": gpu_s / steps * 1e3, "kernel_us_mean": k,
                                    "down_GBps": b_down / (kd * 1e-6) / 1e9 if kd else None,
                                    "up_GBps": b_up / (k["qwk_hc_up"] * 1e-6) / 1e9 if "qwk_hc_up" in k else None}
    return res


def ragged_steps(gpu, stack, reps=5):
    """BASELINE.json configs[3]: a continuous-batching step of one layer (layer 0 of the stack): 16 slots with seeded
    uniform row counts in 1..16 redrawn until the total is near the target, Zipf(1.1) routing forced through the
    logits. Timed two ways on the same rows: the decode path in groups of at most 16 rows (one batch), and the packing
    path (count -> prefix sums -> scatter -> grouped product -> combine) in one pass. Routed experts' bytes are read
    once per group on the first way and once on the second; the table gives the crossover in rows per step."""
    from qwental_amd import synth
    from qwental_amd.gpu import SelRecord
    layer, path, E, K, D = stack.layers[0], stack.path, stack.E, stack.topk, stack.D
    out = []
    for target in (16, 32, 64, 128):
        rng = np.random.default_rng(1000 + target)
        while True:
            n = rng.integers(1, 17, 16) if target >= 48 else rng.integers(1, max(2, target // 8 + 1), 16)
            if abs(int(n.sum()) - target) <= max(2, target // 8):
                break
        T = int(n.sum())
        x = synth.activations(rng, T, D)
        ids = synth.zipf_ids(rng, T, E, K)
        lg = synth.logits_for_ids(rng, ids, E)
        groups = [(g0, min(16, T - g0)) for g0 in range(0, T, 16)]
        bufs = [(gpu.buf_from(x[g0:g0 + nb]), gpu.buf_from(lg[g0:g0 + nb]), gpu.buf(path.sel_bytes(nb)), gpu.buf(nb * D * 2)) for g0, nb in groups]
        t_dec = 1e9
        for _ in range(reps):
            b = gpu.batch()
            for (g0, nb), (xb, lb, sb, ob) in zip(groups, bufs):
                path.gg_moe_lg(b, layer, nb, xb, lb, sb, ob)
            t_dec = min(t_dec, b.end())
        w = np.concatenate([SelRecord(sb.view(np.uint8).copy(), 8 if nb <= 8 else 16, K).w[:nb, :K] for (g0, nb), (xb, lb, sb, ob) in zip(groups, bufs)])
        path.pf_reserve(T, 16)
        xb, ib, wb, ob = gpu.buf_from(x), gpu.buf_from(ids.astype(np.uint32).ravel()), gpu.buf_from(w.astype(np.float32).ravel()), gpu.buf(T * D * 2)
        t_pk = 1e9
        for _ in range(reps):
            b = gpu.batch()
            path.pf_moe(b, layer, T, xb, ib, wb, ob)
            t_pk = min(t_pk, b.end())
        counts = np.bincount(ids.ravel(), minlength=E)
        U = int((counts > 0).sum())
        U_groups = sum(len(np.unique(ids[g0:g0 + nb])) for g0, nb in groups)
        out.append({"rows": T, "slots": n.tolist(), "unique_experts": U, "unique_experts_summed_over_groups": U_groups, "max_rows_per_expert": int(counts.max()),
                    "experts_by_rows": {"1": int((counts == 1).sum()), "2-4": int(((counts >= 2) & (counts <= 4)).sum()), "5-16": int(((counts >= 5) & (counts <= 16)).sum()),
                                        ">16": int((counts > 16).sum())},
                    "decode_groups_us": t_dec * 1e6, "packing_path_us": t_pk * 1e6,
                    "decode_groups_GBps": (U_groups * stack.exp_bytes) / t_dec / 1e9, "packing_path_GBps": (U * stack.exp_bytes) / t_pk / 1e9})
        for bb in [xb, ib, wb, ob] + [y for t4 in bufs for y in t4]:
            bb.free()
    # the step planner (include/qw_par.h) on these measurements: one group of b rows timed for a few sizes, the packing
    # path from the table above; what it would run for each row count, with its two estimates
    import qwental_amd as q
    par = q.Par()
    rng = np.random.default_rng(999)
    for b_ in (1, 2, 4, 8, 12, 16):
        ids = synth.zipf_ids(rng, b_, E, K)
        bufs = (gpu.buf_from(synth.activations(rng, b_, D)), gpu.buf_from(synth.logits_for_ids(rng, ids, E)), gpu.buf(path.sel_bytes(b_)), gpu.buf(b_ * D * 2))
        for _ in range(reps + 1):  # the planner drops the first sample of a size
            b = gpu.batch()
            path.gg_moe_lg(b, layer, b_, *bufs)
            par.observe(b_, b.end() * 1e6)
        for bb in bufs:
            bb.free()
    for row in out:
        for _ in range(2):
            par.observe_packed(row["rows"], row["packing_path_us"])
    for row in out:
        packed, groups = par.choose(row["rows"])
        row["planner"] = {"form": "packing path" if packed else "groups", "groups": groups, "estimate_groups_us": par.cost(min(row["rows"], 64)) if row["rows"] <= 64 else None,
                          "estimate_packing_us": par.packed_cost(row["rows"])}
    par.free()
    return out


def qmv_table(gpu, reps=5, nmat=64):
    """BASELINE.json configs[0..1]: y = W x for a 4096 x 2048 matrix, IQ3_S and Q8_0, 1..16 activations. nmat matrices
    at different addresses go into one batch so that no cache holds the weights (the method of bench/moe_bw.c:50-89);
    the figure is GPU time per matrix. For IQ3_S and up to 4 activations the VALU GEMV form is timed beside the
    matrix-core form."""
    from qwental_amd import synth
    from qwental_amd.stack import fill_blocks
    import qwental_amd as q
    N, K = 4096, 2048
    path = q.Path(gpu, 2048, 512, 512, 10, 16)
    rng = np.random.default_rng(1)
    x = gpu.buf_from(synth.activations(rng, 16, K), device_only=True)
    y = gpu.buf(16 * N * 4, device_only=True)
    out = {}
    for ft in (21, 8):
        rb = synth.row_bytes(ft, K)
        W = gpu.buf(nmat * N * rb, device_only=True)
        b = gpu.batch()
        fill_blocks(gpu, b, W, 0, nmat * N * rb // synth.BLOCK[ft][1], ft, 99 + ft, synth.D_SIGMA[ft])
        b.end()
        for nb in (1, 2, 4, 8, 16):
            algo = N * rb + nb * (K * 2 + N * 4)
            for valu in ((False, True) if ft == 21 and nb <= 4 else (False,)):
                name = "qmv_gg_bench_f%d_n%d%s" % (ft, nb, "_valu" if valu else "")
                ok, err = gpu.compile("#define qmv_gg %s\n#define GF %d\n#define KD %d\n#define RB %d\n#define NB %d\n#define YT float\n%s" % (name, ft, K, rb, nb, "#define QW_VALU 1\n" if valu else ""))
                assert ok, err
                k = gpu.kernel(name)
                best = 1e9
                for _ in range(reps + 1):
                    b = gpu.batch()
                    b.kernel(k)
                    b.buf(3, x)
                    b.buf(4, y)
                    b.bytes(5, np.array([N, K, N, 0], np.uint32))
                    for i in range(nmat):
                        b.buf(0, W, i * N * rb)
                        b.dispatch((N + 7) // 8, 1, 1, 256, 1, 1)
                    best = min(best, b.end())
                # (frac_of_peak: the launch's algorithmic bytes over its time against the 8 TB/s of the data sheet; at this size a
                # launch is mostly its own fixed cost, an empty launch of the same grid takes 2.5 us)
                out["%s_B%d%s" % ("iq3_s" if ft == 21 else "q8_0", nb, "_valu" if valu else "")] = {"us_per_matvec": best / nmat * 1e6, "GBps": algo / (best / nmat) / 1e9,
                                                                                                  "algorithmic_bytes": algo, "frac_of_peak": algo / (best / nmat) / 1e9 / HBM_PEAK_GBS}
        W.free()
    path.close()
    x.free()
    y.free()
    return out


FORMAT_NAMES = {12: "q4_k", 13: "q5_k", 14: "q6_k", 20: "iq4_nl", 23: "iq4_xs", 1: "f16", 30: "bf16"}


def formats_table(gpu, reps=4, nmat=32):
    """The other GGUF formats of the dense matvec (4096 x 2048, 1 and 16 activations, method of qmv_table), a vocabulary
    sized Q6_K matrix (131072 x 2048: the lm_head case) and four projections of mixed formats in one launch
    (kernels/qmv_ggm.metal). One matrix is drawn on the host and copied to nmat addresses."""
    from qwental_amd import synth
    import qwental_amd as q
    K = 2048
    rng = np.random.default_rng(2)
    path = q.Path(gpu, 2048, 512, 512, 10, 16)
    x = gpu.buf_from(synth.activations(rng, 16, K), device_only=True)
    out = {}

    def timed(ft, N, copies, nb):
        rb = synth.row_bytes(ft, K)
        one = synth.matrix(rng, ft, min(N, 4096), K)
        W = gpu.buf(copies * N * rb, device_only=True)
        for i in range(copies * (N // min(N, 4096))):
            W.fill(one, i * one.nbytes)
        y = gpu.buf(16 * N * 4, device_only=True)
        name = "qmv_gg_bench_f%d_n%d" % (ft, nb)
        ok, err = gpu.compile("#define qmv_gg %s\n#define GF %d\n#define KD %d\n#define RB %d\n#define NB %d\n#define YT float\n" % (name, ft, K, rb, nb))
        assert ok, err
        k = gpu.kernel(name)
        best = 1e9
        for _ in range(reps):
            b = gpu.batch()
            b.kernel(k)
            b.buf(3, x)
            b.buf(4, y)
            b.bytes(5, np.array([N, K, N, 0], np.uint32))
            for i in range(copies):
                b.buf(0, W, i * N * rb)
                b.dispatch((N + 7) // 8, 1, 1, 256, 1, 1)
            best = min(best, b.end())
        W.free()
        y.free()
        t = best / copies
        return {"us_per_matvec": t * 1e6, "GBps": (N * rb + nb * (K * 2 + N * 4)) / t / 1e9}

    for ft, nm in FORMAT_NAMES.items():
        for nb in (1, 16):
            out["%s_B%d" % (nm, nb)] = timed(ft, 4096, nmat, nb)
    for nb in (1, 16):
        out["q6_k_131072rows_B%d" % nb] = timed(14, 131072, 2, nb)
    # q / k / v / indexer of one decode step: four matrices, one launch
    fm, Ns = (12, 12, 14, 30), (4096, 512, 512, 128)
    sets = 16
    Ws = [gpu.buf_from(np.tile(synth.matrix(rng, f, n, K), sets), device_only=True) for f, n in zip(fm, Ns)]
    ys = [gpu.buf(16 * n * 4, device_only=True) for n in Ns]
    wbytes = sum(n * synth.row_bytes(f, K) for f, n in zip(fm, Ns))
    for nb in (1, 16):
        best = 1e9
        for _ in range(reps):
            b = gpu.batch()
            for i in range(sets):
                path.qmv_ggm(b, [q.Tensor(w, f, i * n * synth.row_bytes(f, K)) for w, f, n in zip(Ws, fm, Ns)], list(Ns), K, x, ys, nb)
            best = min(best, b.end())
        t = best / sets
        out["ggm_q4k_q4k_q6k_bf16_B%d" % nb] = {"us_per_launch": t * 1e6, "GBps": wbytes / t / 1e9, "rows": list(Ns)}
    for bb in Ws + ys + [x]:
        bb.free()
    path.close()
    return out


def gguf_load(gpu, layers=2, reps=3):
    """Weight residency from GGUF files (include/qw_gguf.h): `layers` full-size MoE layers (513 experts each, IQ3_S,
    random bytes) written to a temporary directory, then loaded into HBM by the reader; the files are in the page
    cache (just written). Best of `reps` loads with the default worker threads, and with one thread; for scale, the
    same bytes through one plain host-to-device copy out of the file mapping."""
    import shutil
    import tempfile

    import qwental_amd as q
    from qwental_amd import gguf_writer as gf
    D, I, E = 2048, 512, 512
    rng = np.random.default_rng(99)
    tmp = tempfile.mkdtemp(prefix="qw_gguf_")
    try:
        for l in range(layers):
            p = "blk.%d." % l
            rb = lambda ft, dims: np.frombuffer(rng.bytes(gf.tensor_bytes(ft, dims)), np.uint8)
            router = (rng.normal(0, 0.02, (E, D)).astype(np.float32).view(np.uint32) >> 16).astype(np.uint16)
            gate_v = (router[0].astype(np.uint32) << 16).view(np.float32)
            ts = [(p + "ffn_gate_exps.weight", 21, [D, I, E], None), (p + "ffn_up_exps.weight", 21, [D, I, E], None), (p + "ffn_down_exps.weight", 21, [I, D, E], None),
                  (p + "ffn_gate_shexp.weight", 21, [D, I], None), (p + "ffn_up_shexp.weight", 21, [D, I], None), (p + "ffn_down_shexp.weight", 21, [I, D], None)]
            ts = [(n, ft, d, rb(ft, d)) for n, ft, d, _ in ts] + [(p + "ffn_gate_inp.weight", 30, [D, E], router), (p + "ffn_gate_inp_shexp.weight", 0, [D], gate_v)]
            gf.write_gguf(os.path.join(tmp, "layer-%05d.gguf" % l), ts)
            del ts
        out = {"layers": layers, "source": "page cache (files just written)"}
        for label, threads in (("default_threads", None), ("one_thread", "1"), ("two_threads", "2"), ("eight_threads", "8")):
            best = None
            for _ in range(reps):
                if threads:
                    os.environ["QW_HIP_LOAD_THREADS"] = threads
                g = q.Gguf(tmp)
                try:
                    g.load(gpu, "moe,shared,router")
                finally:
                    os.environ.pop("QW_HIP_LOAD_THREADS", None)
                n, sec = g.resident_bytes(), g.load_seconds()
                if label == "default_threads" and best is None:  # what arrived is what the file holds
                    t = g.find("blk.%d.ffn_down_exps.weight" % (layers - 1))
                    tail = g.read_resident(t, t.nbytes)[-(1 << 20):]
                    assert np.array_equal(tail, g.host(t)[-(1 << 20):]), "resident bytes differ from the file"
                    M, d, i, e = g.moe_layer(0)
                    assert (d, i, e) == (D, I, E)
                g.close()
                best = sec if best is None else min(best, sec)
            out[label] = {"bytes": int(n), "seconds": best, "GBps": n / best / 1e9}
        # for scale: the same bytes of one tensor by one plain copy call, out of a fresh mapping of the file (what
        # handing a mapped file to qw_buf_wrap() amounts to) and out of ordinary process memory
        g = q.Gguf(tmp)
        t = g.find("blk.0.ffn_gate_exps.weight")
        path0, off0, nb0 = g.shards()[t.shard]["path"], int(t.offset), int(t.nbytes)
        src = g.host(t)  # a private copy in pageable memory
        dst = gpu.buf(src.nbytes, device_only=True)
        best = bestm = None
        for _ in range(reps):
            t0 = time.perf_counter()
            dst.fill(src)
            best = min(best or 1e9, time.perf_counter() - t0)
            mm = np.memmap(path0, np.uint8, "r", off0, (nb0,))
            t0 = time.perf_counter()
            dst.fill(mm)
            bestm = min(bestm or 1e9, time.perf_counter() - t0)
            del mm
        out["plain_copy_file_mapping"] = {"bytes": nb0, "seconds": bestm, "GBps": nb0 / bestm / 1e9}
        out["plain_copy_pageable"] = {"bytes": int(src.nbytes), "seconds": best, "GBps": src.nbytes / best / 1e9}
        dst.free()
        g.close()
        return out
    finally:
        shutil.rmtree(tmp, ignore_errors=True)


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=3)
    ap.add_argument("--layers", type=int, default=48)
    ap.add_argument("--nb", type=int, default=16)
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--quick", action="store_true", help="B = 16 only, no ragged-step table (profiling runs)")
    ap.add_argument("--copy-calib", action="store_true", help="also run the copy kernel over 1 GiB three times (scale for the memory counters)")
    ap.add_argument("--traffic", type=float, default=None, help="HBM bytes per launch of the dominant kernel from the counter runs, to report")
    ap.add_argument("--dense-only", action="store_true", help="only the dense matvec tables (configs 1-2 and the other formats): for profiling runs")
    ap.add_argument("--gguf-only", action="store_true", help="only the GGUF load measurement")
    ap.add_argument("--model-shape-only", action="store_true", help="only the stack of the reference model's layer shape and formats")
    ap.add_argument("--release-source", action="store_true", help="after the first step keep only the tile-major copies of the routed experts (frees their GGUF-order bytes); implies --no-cpu --quick")
    ap.add_argument("--hyper-only", action="store_true", help="only the hyper-connection -> MoE layer loop")
    ap.add_argument("--ragged-only", action="store_true", help="only the continuous-batching step table (config 4) on a one-layer stack: for profiling runs")
    a = ap.parse_args()
    if a.gpus != 1:
        print("bench.py: this build runs on one GPU; --gpus %d is not supported (no collectives, no sharding)" % a.gpus, file=sys.stderr)
        return 2
    import qwental_amd as q
    from qwental_amd import synth
    from qwental_amd.stack import MoeStack

    gpu = q.Gpu()
    if a.dense_only:
        print(json.dumps({"qmv": qmv_table(gpu), "qmv_formats": formats_table(gpu)}))
        return 0
    if a.gguf_only:
        print(json.dumps({"gguf_load": gguf_load(gpu)}))
        return 0
    if a.model_shape_only:
        print(json.dumps({"model_shape": model_shape_leg(gpu, a.layers, a.steps, a.warmup, not a.no_cpu)}))
        return 0
    if a.hyper_only:
        stack = MoeStack(gpu, layers=a.layers, nbmax=16)
        print(json.dumps({"hyper_ffn_step": hyper_ffn_leg(gpu, stack, a.steps, a.warmup)}))
        stack.free()
        return 0
    if a.ragged_only:
        stack = MoeStack(gpu, layers=1, nbmax=16)
        print(json.dumps({"ragged_step": ragged_steps(gpu, stack)}))
        stack.free()
        return 0
    t0 = time.perf_counter()
    stack = MoeStack(gpu, layers=a.layers, nbmax=16)
    rng = np.random.default_rng(2024)
    xh = synth.activations(rng, 16, stack.D)
    x = gpu.buf_from(xh, device_only=True)
    setup_s = time.perf_counter() - t0

    if a.copy_calib:
        copy_calibration(gpu)
    released = None
    if a.release_source:  # the oracle leg reads the weights back from HBM, so it cannot follow
        a.no_cpu = a.quick = True
        stack.step(x, 16)
        released = stack.release_sources()
    res = {}
    for nb in ([a.nb] if a.quick else sorted({1, 8, a.nb})):
        wall, gpu_s = timed_steps(stack, x, nb, a.steps, a.warmup)
        U = stack.unique_experts(nb)
        byts = stack.algorithmic_bytes(nb, U)
        res[nb] = {"tokens_per_s": nb * a.steps / wall, "ms_per_step": wall / a.steps * 1e3, "gpu_ms_per_step": gpu_s / a.steps * 1e3,
                   "stack_GBps": sum(byts) / (gpu_s / a.steps) / 1e9, "mean_U": float(np.mean(U)), "bytes_per_step": int(sum(byts))}
    nb = a.nb
    # the dominant kernel, launch by launch: HIP events around every launch of one more step, on the stream it runs on
    gpu.profile(True)
    stack.step(x, nb)
    gpu.profile(False)
    ent = gpu.profile_entries()
    mean_s, n_l = gpu.profile_mean(DOMINANT)
    U = stack.unique_experts(nb)
    # the gate/up launch of layer l reads U_l routed experts' gate and up rows (901,120 GGUF bytes each), the logits
    # it makes the selection from and the nb x 4 KB activations (the shared expert's rows belong to the front launch)
    gu_bytes = float(np.mean([u * stack.gu_bytes + nb * (stack.E + 1) * 4 + nb * stack.D * 2 for u in U]))
    per_kernel = {}
    for name, us in ent:
        per_kernel.setdefault(name, []).append(us)
    roof = {"bound": "hbm", "kernel": DOMINANT, "achieved": gu_bytes / mean_s / 1e9 if mean_s > 0 else None, "peak": HBM_PEAK_GBS, "unit": "GB/s",
            "frac": gu_bytes / mean_s / 1e9 / HBM_PEAK_GBS if mean_s > 0 else None, "traffic": a.traffic if a.traffic is not None else committed_traffic(),
            "traffic_source": "--traffic argument (counter runs of this command)" if a.traffic is not None else
                              "constant from the committed counter summary profiles/moe_stack_b16_hbm_traffic.txt, not measured in this run",
            "launches": n_l, "mean_launch_us": mean_s * 1e6, "algorithmic_bytes_per_launch": gu_bytes}
    line = {"metric": "batched IQ3_S MoE decode tokens/s at B=16 (48-layer FFN stack); achieved HBM GB/s", "value": res[nb]["tokens_per_s"], "unit": "tokens/s",
            "n_gpus": 1, "steps": a.steps, "warmup": a.warmup, "ms_per_step": res[nb]["ms_per_step"], "higher_is_better": True, "scaling": "weak",
            "vs_baseline": None, "dtype": "u8 blocks -> f16 matrix-core operands, f32 accumulate", "data": "synthetic (seeded, generated on device); block scales d drawn as BASELINE states them times %g (synth.MOE_D_SCALE: the stated |N(0, 0.02)| "
                    "overflows the binary16 layer output; bytes and work are unchanged)" % synth.MOE_D_SCALE,
            "config": {"workload": "configs[4]: %d-layer MoE FFN stack decode, B=%d, D=2048 I=512 E=512 top-10, IQ3_S experts, shared expert Q8_0 every 4th layer; "
                                   "every layer reads the same x and overwrites one out, launched in order on one stream (a bandwidth bench: no overlap between layers is used)" % (stack.L, nb),
                       "resident_weight_bytes": int(stack.weight_bytes), "packed_copy_bytes": int(gpu.L.qw_hip_packed_bytes(gpu.g)), "released_source_bytes": released, "device": gpu.name()},
            "roofline": roof,
            "read_ceiling": None if released else read_ceiling(gpu, stack, nb),  # it reads the GGUF-order bytes
            "ablation": ablation_leg(gpu, stack, x, nb, mean_s * 1e6),
            "stack": {"GBps_algorithmic": res[nb]["stack_GBps"], "frac_of_peak": res[nb]["stack_GBps"] / HBM_PEAK_GBS, "gpu_ms_per_step": res[nb]["gpu_ms_per_step"],
                      "mean_unique_experts": res[nb]["mean_U"], "bytes_per_step": res[nb]["bytes_per_step"]},
            "by_batch": {str(k): v for k, v in res.items()},
            "kernel_us_mean": {k: float(np.mean(v)) for k, v in per_kernel.items()},
            "setup_s": setup_s}
    if line["read_ceiling"]:
        line["ablation"]["pure_read_of_the_same_bytes_us"] = line["read_ceiling"]["us_per_launch"]
    if not a.quick:
        line["hyper_ffn_step"] = hyper_ffn_leg(gpu, stack, min(a.steps, 10), a.warmup)
        line["ragged_step"] = ragged_steps(gpu, stack)
        line["qmv"] = qmv_table(gpu)
        line["qmv_formats"] = formats_table(gpu)
        line["gguf_load"] = gguf_load(gpu)
        line["model_shape"] = model_shape_leg(gpu, a.layers, min(a.steps, 10), a.warmup, not a.no_cpu)  # 92 GB beside the 67 GB of the main stack
    if not a.no_cpu:
        line["cpu_baseline"] = cpu_baseline(stack, x, xh, nb)
        if "model_shape" in line and "layer0_max_rel_err" in line["model_shape"]:
            line["cpu_baseline"]["model_shape_layer0_max_rel_err"] = line["model_shape"].pop("layer0_max_rel_err")
    x.free()
    stack.free()
    print(json.dumps(line))
    gpu.close()
    return 0


if __name__ == "__main__":
    sys.exit(main())
