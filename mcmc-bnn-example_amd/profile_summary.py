#!/usr/bin/env python3
"""Condenses the raw rocprofv3 output written by profile.sh into a few lines of text."""
import collections
import csv
import glob
import json
import os
import sys


def find(d, pat):
    hits = glob.glob(os.path.join(d, "**", pat), recursive=True)
    return hits[0] if hits else None


def counter_totals(path, kernel_substr):
    """{dispatch: {counter: sum over instances}} for kernels whose name contains kernel_substr"""
    agg = collections.defaultdict(lambda: collections.defaultdict(float))
    for r in csv.DictReader(open(path)):
        if kernel_substr in r["Kernel_Name"]:
            agg[r["Dispatch_Id"]][r["Counter_Name"]] += float(r["Counter_Value"])
    return agg


def median_launch(tot, size):
    """(dispatch, counters) of the launch of median size among the launches of transitions (the evaluation
    launches, thousands of times smaller, are left out): the shape most of the run was spent in"""
    items = sorted(tot.items(), key=lambda kv: size(kv[1]))
    big = [kv for kv in items if size(kv[1]) >= 0.02 * size(items[-1][1])]
    return big[len(big) // 2]


def bench_json(path):
    try:
        return json.loads(open(path).read().strip().splitlines()[-1])
    except Exception:  # noqa: BLE001
        return None


def main(out):
    lines = []
    stats = find(os.path.join(out, "trace"), "*kernel_stats.csv")
    if stats:
        lines.append("kernel stats (rocprofv3 --kernel-trace --stats):")
        lines.append("  %-70s %8s %14s %14s %7s" % ("kernel", "calls", "total ms", "avg ms", "%"))
        for r in csv.DictReader(open(stats)):
            lines.append("  %-70s %8s %14.3f %14.3f %7.2f" % (
                r["Name"][:70], r["Calls"], float(r["TotalDurationNs"]) / 1e6,
                float(r["AverageNs"]) / 1e6, float(r["Percentage"])))
    kt = find(os.path.join(out, "trace"), "*kernel_trace.csv")
    if kt:
        durs = [(int(r["End_Timestamp"]) - int(r["Start_Timestamp"])) / 1e6
                for r in csv.DictReader(open(kt)) if "hmc_kernel" in r["Kernel_Name"]]
        # launches of transitions take a hundred milliseconds and more (the tail batch of a 200-window
        # run a sixth of a full batch); the bootstrap and state evaluations that precede them a few at most
        trans = [d for d in durs if d > 0.05 * max(durs)]
        lines.append("hmc_kernel dispatches: %d evaluation launches (%.3f ms in all), %d launches of "
                     "transitions: %s ms" % (len(durs) - len(trans), sum(durs) - sum(trans), len(trans),
                                             ", ".join("%.1f" % d for d in trans)))
        if trans:
            lines.append("average over the %d launches of transitions: %.3f ms" % (
                len(trans), sum(trans) / len(trans)))
        dt = bench_json(os.path.join(out, "bench_trace.json"))
        if dt and 0 < dt["roofline"]["launches"] <= len(trans):
            timed = trans[-dt["roofline"]["launches"]:]
            lines.append("average over the last %d of them (the timed region of bench.py; the ones before are its "
                         "warm-up): %.3f ms" % (len(timed), sum(timed) / len(timed)))
    d = bench_json(os.path.join(out, "bench_trace.json"))
    if d:
        lines.append("bench.py under the tracer: %.0f grad-evals/s, roofline frac %.3f, %.3f ms per launch "
                     "(HIP events over the timed region), %d launches" % (
                         d["value"], d["roofline"]["frac"], d["roofline"]["ms_per_launch"],
                         d["roofline"]["launches"]))
    scale, total_bytes, evals = {}, 0.0, None
    for c in ("FETCH_SIZE", "WRITE_SIZE"):
        cp = find(os.path.join(out, "copy_" + c), "*counter_collection.csv")
        kp = find(os.path.join(out, "pmc_" + c), "*counter_collection.csv")
        if cp:
            tot = counter_totals(cp, "copy_kernel")
            v = max(x[c] for x in tot.values())
            scale[c] = (1024.0 * 1024.0) / v  # true KiB per counted unit
            lines.append("%s on the 1 GiB copy kernel: %.0f counted -> scale factor %.4f true KiB per unit"
                         % (c, v, scale[c]))
        if kp:
            tot = counter_totals(kp, "hmc_kernel")
            allv = sum(v[c] for v in tot.values())
            big = sorted(tot.items(), key=lambda kv: -kv[1][c])[:2]
            for disp, v in big:
                lines.append("%s, largest hmc_kernel dispatch %s: %.0f counted = %.1f MiB after scaling" % (
                    c, disp, v[c], v[c] * scale.get(c, 1.0) / 1024.0))
            lines.append("%s, all %d hmc_kernel dispatches: %.0f counted = %.1f MiB after scaling" % (
                c, len(tot), allv, allv * scale.get(c, 1.0) / 1024.0))
            total_bytes += allv * scale.get(c, 1.0) * 1024.0
            b = bench_json(os.path.join(out, "bench_%s.json" % c))
            if b:
                evals = b["roofline"]["grad_evals_per_launch"] * b["roofline"]["launches"] * (
                    b["steps"] + b["warmup"]) / b["steps"]
    if total_bytes and evals:
        lines.append("HBM traffic: %.4g bytes over %.0f gradient evaluations = %.0f bytes per evaluation" % (
            total_bytes, evals, total_bytes / evals))
        if d:
            lines.append("  = %.2f TB/s at the %.0f evaluations/s of the traced run (HBM peak 8 TB/s)" % (
                total_bytes / evals * d["value"] / 1e12, d["value"]))
        key = "hmc_kernel_wide_64x128" if d and "64->128" in d["config"]["workload"] else (
            "hmc_kernel_%s_22x40" % (d["config"]["layer"] if d else "mfma"))
        json.dump({key: {"bytes_per_grad_eval": total_bytes / evals,
                         "source": "rocprofv3 --pmc FETCH_SIZE and WRITE_SIZE over every trajectory-kernel "
                                   "dispatch of one bench.py run, each scaled by the same counter on a 1 GiB "
                                   "copy kernel",
                         "launches_chains_x_workgroups_per_chain":
                             d["config"].get("launches_chains_x_workgroups_per_chain") if d else None}},
                  open(os.path.join(out, "traffic.json"), "w"), indent=1)
    sq = find(os.path.join(out, "pmc_SQ"), "*counter_collection.csv")
    if sq:
        tot = counter_totals(sq, "hmc_kernel")
        disp, v = median_launch(tot, lambda c: c.get("GRBM_GUI_ACTIVE", 0))
        simd_cycles = 1024.0 * v["GRBM_GUI_ACTIVE"] / 8.0  # 8 XCDs report, 1024 SIMDs
        lines.append("SQ counters, hmc_kernel dispatch %s, the median launch of transitions (fractions of all SIMD cycles):" % disp)
        lines.append("  MFMA pipe busy %.3f | VALU (non-MFMA) active %.3f | any instruction active %.3f | "
                     "VALU insts per MFMA %.2f" % (
                         v["SQ_VALU_MFMA_BUSY_CYCLES"] / simd_cycles, 4 * v["SQ_ACTIVE_INST_VALU"] / simd_cycles,
                         4 * v["SQ_ACTIVE_INST_ANY"] / simd_cycles,
                         (v["SQ_INSTS_VALU"] - v["SQ_INSTS_MFMA"]) / max(1.0, v["SQ_INSTS_MFMA"])))
    tcc = find(os.path.join(out, "pmc_TCC"), "*counter_collection.csv")
    if tcc:
        tot = counter_totals(tcc, "hmc_kernel")
        disp, v = median_launch(tot, lambda c: c.get("TCC_HIT_sum", 0) + c.get("TCC_MISS_sum", 0))
        hit, miss = v["TCC_HIT_sum"], v["TCC_MISS_sum"]
        lines.append("L2 (TCC), hmc_kernel dispatch %s, the median launch of transitions: hits %.4g, misses %.4g -> hit rate %.3f; read requests to "
                     "the fabric %.4g of which marked DRAM %.4g" % (disp, hit, miss, hit / max(1.0, hit + miss),
                                                                   v["TCC_EA0_RDREQ_sum"], v["TCC_EA0_RDREQ_DRAM_sum"]))
    text = "\n".join(lines)
    print(text)
    open(os.path.join(out, "summary.txt"), "w").write(text + "\n")


if __name__ == "__main__":
    main(sys.argv[1] if len(sys.argv) > 1 else "gpurun_out/profile")
