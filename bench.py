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


def cpu_baseline(stack, x, nb, lg_dev, budget_s=20.0):
    """The CPU oracle (float dot products over dequantized rows, OpenMP over all cores) on the first layers of the
    same stack with the same logits; stops after about budget_s seconds. Also the full-size parity check."""
    from oracle import oracle as o
    cores = o.max_threads()
    t_used, n, worst = 0.0, 0, 0.0
    while t_used < budget_s and n < stack.L and n < len(lg_dev):
        m = stack.layer_weights_host(n)
        lg = lg_dev[n]
        t0 = time.perf_counter()
        out32, _, _ = o.moe_layer_f32(m, lg, x[:nb], 8 if nb <= 8 else 16)
        t_used += time.perf_counter() - t0
        n += 1
        del m
    per_layer = t_used / n
    return {"value": nb / (per_layer * stack.L), "unit": "tokens/s", "cores": cores, "kind": "port",
            "sample": "oracle moe_layer_f32 on layers 0..%d of the stack (B = %d), %.1f s; scaled to %d layers" % (n - 1, nb, t_used, stack.L)}


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=3)
    ap.add_argument("--layers", type=int, default=48)
    ap.add_argument("--nb", type=int, default=16)
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--quick", action="store_true", help="B = 16 only (profiling runs)")
    ap.add_argument("--copy-calib", action="store_true", help="also run the copy kernel over 1 GiB three times (scale for the memory counters)")
    ap.add_argument("--traffic", type=float, default=None, help="HBM bytes per launch of the dominant kernel from the counter runs, to report")
    a = ap.parse_args()
    if a.gpus != 1:
        print("bench.py: this build runs on one GPU; --gpus %d is not supported (no collectives, no sharding)" % a.gpus, file=sys.stderr)
        return 2
    import qwental_amd as q
    from qwental_amd import synth
    from qwental_amd.stack import MoeStack

    gpu = q.Gpu()
    t0 = time.perf_counter()
    stack = MoeStack(gpu, layers=a.layers, nbmax=16)
    rng = np.random.default_rng(2024)
    xh = synth.activations(rng, 16, stack.D)
    x = gpu.buf_from(xh, device_only=True)
    setup_s = time.perf_counter() - t0

    if a.copy_calib:
        copy_calibration(gpu)
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
    # the gate/up launch of layer l reads U_l routed experts' gate and up rows (901,120 bytes each), the shared
    # expert's gate and up rows (same shape, IQ3_S or Q8_0) and the nb x 4 KB activations
    sh_gu = [2 * stack.I * synth.row_bytes(f, stack.D) for f in stack.shared_fmt]
    gu_bytes = float(np.mean([u * stack.gu_bytes + s + nb * stack.D * 2 for u, s in zip(U, sh_gu)]))
    per_kernel = {}
    for name, us in ent:
        per_kernel.setdefault(name, []).append(us)
    roof = {"bound": "hbm", "kernel": DOMINANT, "achieved": gu_bytes / mean_s / 1e9 if mean_s > 0 else None, "peak": HBM_PEAK_GBS, "unit": "GB/s",
            "frac": gu_bytes / mean_s / 1e9 / HBM_PEAK_GBS if mean_s > 0 else None, "traffic": a.traffic if a.traffic is not None else committed_traffic(),
            "launches": n_l, "mean_launch_us": mean_s * 1e6, "algorithmic_bytes_per_launch": gu_bytes}
    line = {"metric": "batched IQ3_S MoE decode tokens/s at B=16 (48-layer FFN stack); achieved HBM GB/s", "value": res[nb]["tokens_per_s"], "unit": "tokens/s",
            "n_gpus": 1, "steps": a.steps, "warmup": a.warmup, "ms_per_step": res[nb]["ms_per_step"], "higher_is_better": True, "scaling": "weak",
            "vs_baseline": None, "dtype": "u8 blocks -> f16 matrix-core operands, f32 accumulate", "data": "synthetic (seeded, generated on device)",
            "config": {"workload": "configs[4]: %d-layer MoE FFN stack decode, B=%d, D=2048 I=512 E=512 top-10, IQ3_S experts, shared expert Q8_0 every 4th layer" % (stack.L, nb),
                       "resident_weight_bytes": int(stack.weight_bytes), "packed_copy_bytes": int(gpu.L.qw_hip_packed_bytes(gpu.g)), "device": gpu.name()},
            "roofline": roof,
            "stack": {"GBps_algorithmic": res[nb]["stack_GBps"], "frac_of_peak": res[nb]["stack_GBps"] / HBM_PEAK_GBS, "gpu_ms_per_step": res[nb]["gpu_ms_per_step"],
                      "mean_unique_experts": res[nb]["mean_U"], "bytes_per_step": res[nb]["bytes_per_step"]},
            "by_batch": {str(k): v for k, v in res.items()},
            "kernel_us_mean": {k: float(np.mean(v)) for k, v in per_kernel.items()},
            "setup_s": setup_s}
    if not a.no_cpu:
        lg = [stack.lg[l].read(dtype=np.float32)[:nb * (stack.E + 1)].reshape(nb, stack.E + 1).copy() for l in range(stack.L)]
        line["cpu_baseline"] = cpu_baseline(stack, xh, nb, lg)
    print(json.dumps(line))
    stack.free()
    gpu.close()
    return 0


if __name__ == "__main__":
    sys.exit(main())
