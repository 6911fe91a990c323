"""Short text summaries of rocprofv3 CSV output for this library's kernels.

    python -m qwental_amd.profsum stats <dir>            per-kernel calls / mean / min / max from *_kernel_stats.csv
    python -m qwental_amd.profsum pmc <dir> <counter>    per-kernel mean of one counter from *_counter_collection.csv,
                                                          with the scale the known-size copy kernel gives it
    python -m qwental_amd.profsum counters <dir> [prefix ...]
                                                         every counter of the run, mean per dispatch, for the kernels
                                                          whose names start with one of the prefixes (default qwk_),
                                                          and the ratios that two counters of the same run define

The copy kernel (qwk_copy over n 16-byte words) reads n * 16 bytes and writes n * 16 bytes; `bench.py --copy-calib`
runs it over 1 GiB, so FETCH_SIZE and WRITE_SIZE (KiB per dispatch) of that dispatch fix the counter's scale.
"""
import csv
import glob
import os
import sys
from collections import defaultdict

CALIB_BYTES = 1 << 30


def _one(d, pat):
    f = sorted(glob.glob(os.path.join(d, "**", pat), recursive=True))
    if not f:
        raise SystemExit("no %s under %s" % (pat, d))
    return f[0]


def stats(d):
    rows = list(csv.DictReader(open(_one(d, "*kernel_stats.csv"))))
    out = ["%-28s %7s %12s %10s %10s %7s" % ("kernel", "calls", "mean_us", "min_us", "max_us", "share%")]
    for r in rows:
        out.append("%-28s %7d %12.2f %10.2f %10.2f %7.2f" % (r["Name"][:28], int(r["Calls"]), float(r["AverageNs"]) / 1e3, float(r["MinNs"]) / 1e3,
                                                          float(r["MaxNs"]) / 1e3, float(r["Percentage"])))
    return "\n".join(out)


def pmc(d, counter):
    per = defaultdict(list)
    for r in csv.DictReader(open(_one(d, "*counter_collection.csv"))):
        if r["Counter_Name"] == counter:
            per[r["Kernel_Name"]].append(float(r["Counter_Value"]))
    if not per:
        raise SystemExit("counter %s not in the file" % counter)
    scale = None
    if "qwk_copy" in per:  # KiB the counter shows for 1 GiB moved
        scale = (CALIB_BYTES / 1024.0) / (sum(per["qwk_copy"]) / len(per["qwk_copy"]))
    out = ["%-28s %7s %16s %16s" % ("kernel", "calls", counter + "_mean", "bytes_scaled" if scale else "")]
    for k in sorted(per, key=lambda k: -sum(per[k])):
        m = sum(per[k]) / len(per[k])
        out.append("%-28s %7d %16.1f %16s" % (k[:28], len(per[k]), m, "%.0f" % (m * 1024 * scale) if scale else ""))
    if scale:
        out.append("scale from qwk_copy over %d bytes: %.4f (true KiB per counted KiB)" % (CALIB_BYTES, scale))
    return "\n".join(out)


# (name, numerator, denominator, what it says)
RATIOS = [
    ("lds_conflict_frac", "SQ_LDS_BANK_CONFLICT", "SQ_LDS_IDX_ACTIVE", "cycles the LDS spent on bank conflicts / cycles it was indexing"),
    ("lds_active_frac", "SQ_LDS_IDX_ACTIVE", "SQ_BUSY_CYCLES", "LDS indexing cycles summed over the compute units' LDS pipes / busy cycles summed over the shader engines"),
    ("valu_inst_cycles_per_wave_cycle", "SQ_ACTIVE_INST_VALU", "SQ_WAVE_CYCLES", "quad-cycles a wave had a vector ALU instruction in flight / quad-cycles waves were resident"),
    ("mfma_busy_per_busy_cycle", "SQ_VALU_MFMA_BUSY_CYCLES", "SQ_BUSY_CYCLES", "cycles the matrix pipes were busy (summed over them) / busy cycles"),
    ("mfma_share_of_valu_insts", "SQ_INSTS_MFMA", "SQ_INSTS_VALU", "matrix instructions / vector ALU instructions issued"),
    ("tcp_pending_stall_frac", "TCP_PENDING_STALL_CYCLES_sum", "TCP_GATE_EN1_sum", "cycles the vector L1 stalled on a pending request / cycles it was clocked"),
    ("l1_miss_frac", "TCP_TCC_READ_REQ_sum", "TCP_TOTAL_CACHE_ACCESSES_sum", "read requests the vector L1 sent to L2 / its accesses"),
    ("wait_frac", "SQ_WAIT_INST_ANY", "SQ_WAVE_CYCLES", "quad-cycles waves waited for any instruction's result / quad-cycles waves were resident"),
    ("icache_miss_frac", "SQC_ICACHE_MISSES", "SQC_ICACHE_REQ", "instruction cache misses / requests"),
]


def counters(d, prefixes):
    per = defaultdict(lambda: defaultdict(list))
    for r in csv.DictReader(open(_one(d, "*counter_collection.csv"))):
        per[r["Kernel_Name"]][r["Counter_Name"]].append(float(r["Counter_Value"]))
    names = sorted({c for k in per for c in per[k]})
    out = []
    for k in sorted(per):
        if not any(k.startswith(p) for p in prefixes):
            continue
        mean = {c: sum(v) / len(v) for c, v in per[k].items()}
        out.append("%s (%d dispatches)" % (k, max(len(v) for v in per[k].values())))
        for c in names:
            if c in mean:
                out.append("    %-34s %16.0f" % (c, mean[c]))
        for nm, a, b, what in RATIOS:
            if a in mean and b in mean and mean[b] > 0:
                out.append("    %-34s %16.3f   (%s)" % (nm, mean[a] / mean[b], what))
    return "\n".join(out)


if __name__ == "__main__":
    if len(sys.argv) >= 3 and sys.argv[1] == "stats":
        print(stats(sys.argv[2]))
    elif len(sys.argv) >= 4 and sys.argv[1] == "pmc":
        print(pmc(sys.argv[2], sys.argv[3]))
    elif len(sys.argv) >= 3 and sys.argv[1] == "counters":
        print(counters(sys.argv[2], sys.argv[3:] or ["qwk_"]))
    else:
        raise SystemExit(__doc__)
