"""Turns rocprofv3 output of `bench.py --kernels-only` runs into the short text summaries under
profiles/ and into profiles/hbm_traffic_per_launch.json (which bench.py reads for `roofline.traffic`).

Each run directory holds `bench.json` (the benchmark's stdout of that run, with its `dispatch_log`)
and, anywhere below it, the CSV files rocprofv3 wrote:

    cd /tmp && export TMPDIR=/tmp
    rocprofv3 --kernel-trace --stats --output-format csv -d RUN/trace -o bench -- \\
        python3 bench.py --kernels-only > RUN/trace/bench.json
    rocprofv3 --pmc FETCH_SIZE --output-format csv -d RUN/FETCH_SIZE -o bench -- \\
        python3 bench.py --kernels-only --steps 20 --warmup 2 > RUN/FETCH_SIZE/bench.json
    ... one run per counter: WRITE_SIZE VALUBusy VALUUtilization LDSBankConflict MemUnitStalled MeanOccupancyPerCU
    python3 -m inferspore_amd.profile_summary RUN --out profiles

Dispatches are attributed to workloads through the benchmark's own `dispatch_log` (workload, kernel,
number of launches, in launch order): the trace is walked in start-time order and every log entry
consumes its number of dispatches of its kernel, so nothing depends on guessing from kernel names.
"""
import argparse
import csv
import glob
import json
import os
import sys

COUNTERS = ["VALUBusy", "VALUUtilization", "LDSBankConflict", "MemUnitStalled", "MeanOccupancyPerCU"]


def base_name(kernel):
    """'void isp::copy_vec<1>(char*, ...)' and 'isp::copy_vec<1>' -> 'isp::copy_vec'."""
    k = kernel.replace("void ", "").strip()
    for stop in "<(":
        i = k.find(stop)
        if i >= 0:
            k = k[:i]
    return k.strip()


def find_one(run_dir, pattern):
    hits = sorted(glob.glob(os.path.join(run_dir, "**", pattern), recursive=True))
    if not hits:
        raise SystemExit("profile_summary: no %s under %s" % (pattern, run_dir))
    return hits[0]


def load_bench(run_dir):
    with open(os.path.join(run_dir, "bench.json")) as f:
        lines = [l for l in f.read().splitlines() if l.startswith("{")]
    return json.loads(lines[-1])


def attribute(rows, dispatch_log, value_of):
    """rows: this library's dispatches in start order.  Returns {workload: {kernel base name: [values]}}."""
    out = {}
    i = 0
    for workload, kernel, launches in dispatch_log:
        names = set(base_name(k) for k in kernel.split(" + "))
        got = {}
        taken = 0
        while taken < launches:
            if i >= len(rows):
                raise SystemExit("profile_summary: trace ends inside workload %s (%d of %d dispatches found)"
                                 % (workload, taken, launches))
            b = base_name(rows[i]["Kernel_Name"])
            if b in names:
                got.setdefault(b, []).append(value_of(rows[i]))
                taken += 1
            i += 1
        out[workload] = got
    return out


def library_rows(path, counter=None):
    with open(path, newline="") as f:
        rows = [r for r in csv.DictReader(f) if "isp::" in r["Kernel_Name"]
                and (counter is None or r.get("Counter_Name") == counter)]
    rows.sort(key=lambda r: int(r["Start_Timestamp"]))
    return rows


def median(v):
    v = sorted(v)
    return v[len(v) // 2]


def tail_of(values, skip):
    """Drops the warm-up dispatches at the front of a workload's list."""
    return values[skip:] if len(values) > skip else values


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("run", help="directory with trace/ and one sub-directory per counter run")
    ap.add_argument("--out", default="profiles")
    a = ap.parse_args()
    os.makedirs(a.out, exist_ok=True)
    prefix = os.path.join(a.out, "all_kernels_benchmark_shapes")

    # ---------------------------------------------------------------- kernel trace
    tdir = os.path.join(a.run, "trace")
    bench = load_bench(tdir)
    per_config = bench["roofline"]["per_config"]
    log = bench["dispatch_log"]
    rows = library_rows(find_one(tdir, "*kernel_trace.csv"))
    # gap between a dispatch's start and the end of the dispatch before it (this library's kernels only;
    # nothing else runs inside a timed pass)
    prev_end = None
    for r in rows:
        r["_gap"] = (int(r["Start_Timestamp"]) - prev_end) if prev_end is not None else 0
        prev_end = int(r["End_Timestamp"])
    dur = attribute(rows, log, lambda r: (int(r["End_Timestamp"]) - int(r["Start_Timestamp"]), r["_gap"]))
    # the dispatch log lists warm-up, gate and timed launches separately; the first `lead_in` timed launches are untimed
    warm = bench.get("lead_in", bench["warmup"])
    steps = bench["steps"]
    ahead_of = bench.get("regions_ahead", {})

    def in_ahead_regions(v, workload, per_step):
        """The dispatches of the regions in which the host stayed ahead of the device (the ones the benchmark's
        median is taken over); all timed dispatches if the benchmark did not say."""
        flags = ahead_of.get(workload)
        if not flags or sum(flags) < min(3, len(flags)):
            return tail_of(v, warm * per_step)
        sel = []
        for r, ok in enumerate(flags):
            if ok:
                sel += v[(warm + r * steps) * per_step:(warm + (r + 1) * steps) * per_step]
        return sel

    out = ["rocprofv3 kernel-trace summary: every kernel of the library at its benchmark shape (bench.py, all workloads)", "",
           "command (run from /tmp with TMPDIR=/tmp on the MI355X box):",
           "  rocprofv3 --kernel-trace --stats --output-format csv -d RUN/trace -o bench -- python3 bench.py --kernels-only",
           "  python3 -m inferspore_amd.profile_summary RUN --out profiles",
           "  (--steps %d --warmup %d; launches rotate over >1 GiB of buffer sets; warm-up, gate and lead-in dispatches excluded)"
           % (steps, bench["warmup"]), "",
           "per workload from the kernel trace -- durations in microseconds; GB/s = algorithmic bytes / average duration.",
           "calls .. max_us cover the dispatches of the timed regions in which the host stayed ahead of the device, i.e. the",
           "launches that ran back to back -- the same regions the benchmark's median is taken over (`regions` = how many of",
           "the timed regions those are; under the profiler a launch costs the host 12 us, so it falls behind on short kernels).",
           "`events` = the benchmark's own HIP-event time per launch in the same (profiled) run; `idle_us` (`n`) = average",
           "duration of the timed dispatches that started 1 us or more after the previous one had ended, i.e. on an idle device.",
           "%-48s %-50s %7s %6s %8s %8s %8s %8s %7s %8s %8s %5s" % (
               "workload", "kernel", "regions", "calls", "avg_us", "med_us", "min_us", "max_us", "GB/s", "events", "idle_us", "n")]
    for workload, kernel, _ in log:
        if workload not in per_config:
            continue
        rec = per_config[workload]
        parts = dur[workload]
        steps_per = rec.get("launches_per_step", 1)
        flags = ahead_of.get(workload)
        reg = ("%d/%d" % (sum(flags), len(flags))) if flags else "-"
        for b, pairs in parts.items():
            v = [d for d, _ in in_ahead_regions(pairs, workload, 1)]
            idle = [d for d, g in tail_of(pairs, warm) if g >= 1000]
            avg = sum(v) / len(v)
            full = [k for k in kernel.split(" + ") if base_name(k) == b][0]
            gbs = ("%7.0f" % (rec["bytes"] / avg)) if steps_per == 1 else "      -"
            idle_s = ("%8.2f %5d" % (sum(idle) / len(idle) / 1e3, len(idle))) if idle else "       - %5d" % 0
            out.append("%-48s %-50s %7s %6d %8.2f %8.2f %8.2f %8.2f %s %8.2f %s" % (
                workload, full[:50], reg, len(v), avg / 1e3, median(v) / 1e3, min(v) / 1e3, max(v) / 1e3, gbs,
                rec["us"], idle_s))
    stats = find_one(tdir, "*kernel_stats.csv")
    out += ["", "rows of the --stats table for this library's kernels (Name, Calls, AverageNs, MinNs, MaxNs; kernels used by",
            "several workloads and the device warm-up copies are merged in these rows):"]
    with open(stats, newline="") as f:
        for r in csv.DictReader(f):
            if "isp::" in r["Name"]:
                out.append("  %s, %s, %.0f, %s, %s" % (r["Name"].split("(")[0].replace("void ", ""), r["Calls"],
                                                       float(r["AverageNs"]), r["MinNs"], r["MaxNs"]))
    with open(prefix + ".kernel_trace_stats.txt", "w") as f:
        f.write("\n".join(out) + "\n")

    # ---------------------------------------------------------------- counters
    def counter_medians(name):
        d = os.path.join(a.run, name)
        if not os.path.isdir(d):
            return None
        b = load_bench(d)
        rows = library_rows(find_one(d, "*counter_collection.csv"), name)
        vals = attribute(rows, b["dispatch_log"], lambda r: float(r["Counter_Value"]))
        return {w: sum(median(tail_of(v, b.get("lead_in", b["warmup"]))) for v in parts.values())
                for w, parts in vals.items() if parts}, b

    fetch, write = counter_medians("FETCH_SIZE"), counter_medians("WRITE_SIZE")
    if fetch and write:
        F, fb = fetch
        W, _ = write
        cal64, cal512 = "calibration_copy_64MiB_traffic", "calibration_copy_512MiB_traffic"
        f_scale = 32768.0 / F[cal64]
        w_scale = 32768.0 / W[cal64]
        pc = fb["roofline"]["per_config"]
        out = ["rocprofv3 --pmc HBM traffic: every kernel of the library at its benchmark shape (bench.py, all workloads)", "",
               "commands (one counter per run, from /tmp with TMPDIR=/tmp on the MI355X box):",
               "  rocprofv3 --pmc FETCH_SIZE --output-format csv -d RUN/FETCH_SIZE -o bench -- python3 bench.py --kernels-only --steps %d --warmup %d"
               % (fb["steps"], fb["warmup"]),
               "  rocprofv3 --pmc WRITE_SIZE --output-format csv -d RUN/WRITE_SIZE -o bench -- python3 bench.py --kernels-only --steps %d --warmup %d"
               % (fb["steps"], fb["warmup"]),
               "  python3 -m inferspore_amd.profile_summary RUN --out profiles", "",
               "calibration: isp_calibration_copy of 32 MiB (32768 KiB read, 32768 KiB written) / 256 MiB",
               "  FETCH_SIZE reads %.1f / %.1f  => scale factor %.4f" % (F[cal64], F[cal512], f_scale),
               "  WRITE_SIZE reads %.1f / %.1f  => scale factor %.4f" % (W[cal64], W[cal512], w_scale), "",
               "median counter value per dispatch (KiB; summed over the launches of a step for multi-launch workloads),",
               "scaled traffic, and the algorithmic bytes the benchmark prices the workload at",
               "%-48s %12s %12s %14s %14s %7s" % ("workload", "FETCH_SIZE", "WRITE_SIZE", "traffic_bytes", "algorithmic", "ratio")]
        traffic = {}
        for w in pc:
            t = (F[w] * f_scale + W[w] * w_scale) * 1024
            traffic[w] = int(round(t))
            out.append("%-48s %12.1f %12.1f %14d %14d %7.3f" % (w, F[w], W[w], t, pc[w]["bytes"], t / pc[w]["bytes"]))
        with open(prefix + ".hbm_traffic_pmc.txt", "w") as f:
            f.write("\n".join(out) + "\n")
        with open(os.path.join(a.out, "hbm_traffic_per_launch.json"), "w") as f:
            json.dump({"source": os.path.basename(prefix) + ".hbm_traffic_pmc.txt",
                       "unit": "HBM bytes per launch (FETCH_SIZE and WRITE_SIZE, each scaled by the calibration copy)",
                       "fetch_scale": f_scale, "write_scale": w_scale, "bytes_per_launch": traffic}, f, indent=1)
            f.write("\n")

    have = {c: counter_medians(c) for c in COUNTERS}
    if all(have.values()):
        b0 = have[COUNTERS[0]][1]
        pc = b0["roofline"]["per_config"]
        out = ["rocprofv3 --pmc derived counters (VALU, LDS, memory unit, occupancy): every kernel of the library at its benchmark shape", "",
               "commands (one derived metric per run -- each expands to several hardware counters -- from /tmp with TMPDIR=/tmp):"]
        for c in COUNTERS:
            out.append("  rocprofv3 --pmc %s --output-format csv -d RUN/%s -o bench -- python3 bench.py --kernels-only --steps %d --warmup %d"
                       % (c, c, b0["steps"], b0["warmup"]))
        out += ["  python3 -m inferspore_amd.profile_summary RUN --out profiles", "",
                "median per dispatch.  VALUBusy / LDSBankConflict / MemUnitStalled: percent of the kernel's time; VALUUtilization: percent",
                "of lanes active in VALU instructions; MeanOccupancyPerCU: waves resident per CU (32 is the maximum)",
                "%-48s %-50s %9s %9s %9s %9s %9s" % ("workload", "kernel", "VALUBusy", "VALUUtil", "LDSBankCf", "MemStall", "Occupancy")]
        for w in pc:
            if pc[w].get("launches_per_step", 1) != 1:
                continue
            out.append("%-48s %-50s %9.2f %9.2f %9.3f %9.3f %9.2f" % (
                w, pc[w]["kernel"][:50], have["VALUBusy"][0][w], have["VALUUtilization"][0][w],
                have["LDSBankConflict"][0][w], have["MemUnitStalled"][0][w], have["MeanOccupancyPerCU"][0][w]))
        with open(prefix + ".valu_lds_pmc.txt", "w") as f:
            f.write("\n".join(out) + "\n")
    print("profile_summary: wrote summaries under %s" % a.out)


if __name__ == "__main__":
    sys.exit(main())
