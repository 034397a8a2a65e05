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


def summarise_layer(a):
    """Per-layer kernel breakdown of a traced build/bin/bench_context_layer run: RUN/layer/layer.json is the program's
    stdout, the trace CSV lies below RUN/layer.  The layer's kernels repeat with a fixed period; the timed iterations
    are the last `iterations` periods of the trace."""
    import re
    ldir = os.path.join(a.run, "layer")
    with open(os.path.join(ldir, "layer.json")) as f:
        text = f.read()
    rec = json.loads([l for l in text.splitlines() if l.startswith("{")][-1])
    cmd = [l for l in text.splitlines() if l.startswith("command: ")]
    with open(find_one(ldir, "*kernel_trace.csv"), newline="") as f:
        rows = list(csv.DictReader(f))
    rows.sort(key=lambda r: int(r["Start_Timestamp"]))

    def short(n):
        if n.startswith("Cijk_"):
            return "hipBLASLt GEMM kernels (Cijk_*)"
        m = re.search(r"context_attention_f16ILi(\d+)E", n)   # a name the profiler leaves mangled
        if m:
            return "isp_layers::context_attention_f16<%s> (fused attention)" % m.group(1)
        return re.sub(r"^void ", "", n).split("(")[0]

    names = [short(r["Kernel_Name"]) for r in rows]
    iters = int(rec["iterations"])
    per = next(p for p in range(2, 64) if len(names) >= 3 * p and names[-p:] == names[-2 * p:-p] == names[-3 * p:-2 * p])
    tail = rows[-iters * per:]
    agg = {}
    for r in tail:
        k = agg.setdefault(short(r["Kernel_Name"]), [0, 0])
        k[0] += 1
        k[1] += int(r["End_Timestamp"]) - int(r["Start_Timestamp"])
    total = sum(v[1] for v in agg.values())
    span = sum(int(tail[i * per + per - 1]["End_Timestamp"]) - int(tail[i * per]["Start_Timestamp"]) for i in range(iters))
    out = ["rocprofv3 kernel-trace summary: the C++ context-decoder layer (LlamaContextDecoderLayer<half>) at LLaMA-2-7B shape,",
           "batch %d, max_q_len %d, %d valid tokens, %s attention" % (rec["batch"], rec["max_q_len"], rec["valid_tokens"], rec["attention"]), "",
           "command (run from /tmp with TMPDIR=/tmp on the MI355X box; the binary is built by `python -m inferspore_amd.build`):",
           "  " + (cmd[-1][len("command: "):] if cmd else "rocprofv3 --kernel-trace --stats --output-format csv -d RUN/layer -o layer -- build/bin/bench_context_layer ..."),
           "  python3 -m inferspore_amd.profile_summary RUN --layer --out profiles", "",
           "per layer over the %d timed iterations (%d kernels per layer; warm-up iterations, which include the one-off" % (iters, per),
           "algorithm-selection runs of the GEMM plan cache, are left out); the program's own figure for the same run: %.3f ms per layer" % rec["ms_per_layer"]]
    for k, v in sorted(agg.items(), key=lambda kv: -kv[1][1]):
        out.append("%-62s %4.1f calls/layer %8.1f us/layer %5.1f%%" % (k, v[0] / iters, v[1] / iters / 1e3, 100.0 * v[1] / total))
    out.append("sum of kernel time per layer: %.1f us; first kernel start to last kernel end per layer: %.1f us"
               % (total / iters / 1e3, span / iters / 1e3))
    out += ["", "one layer's kernels in call order (last iteration, us):"]
    for r in tail[-per:]:
        out.append("  %-62s %8.2f" % (short(r["Kernel_Name"]), (int(r["End_Timestamp"]) - int(r["Start_Timestamp"])) / 1e3))
    name = "context_decoder_layer_cpp_llama2_7b_b%d_s%d%s.kernel_trace_stats.txt" % (
        rec["batch"], rec["max_q_len"], "" if rec["attention"] == "fused" else "_" + rec["attention"])
    with open(os.path.join(a.out, name), "w") as f:
        f.write("\n".join(out) + "\n")
    print("profile_summary: wrote %s" % os.path.join(a.out, name))
    return 0


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("run", help="directory with trace/ and one sub-directory per counter run")
    ap.add_argument("--out", default="profiles")
    ap.add_argument("--prefix", default="all_kernels_benchmark_shapes", help="file name stem of the summaries")
    ap.add_argument("--title", default="every kernel of the library at its benchmark shape (bench.py, all workloads)")
    ap.add_argument("--bench-args", default="--kernels-only", help="the arguments bench.py was run with")
    ap.add_argument("--layer", action="store_true",
                    help="RUN/layer holds a kernel trace of build/bin/bench_context_layer and its stdout (layer.json): "
                         "write the per-layer kernel breakdown instead")
    a = ap.parse_args()
    os.makedirs(a.out, exist_ok=True)
    if a.layer:
        return summarise_layer(a)
    prefix = os.path.join(a.out, a.prefix)

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

    extra = "" if a.prefix == "all_kernels_benchmark_shapes" else " --prefix %s --bench-args '%s' --title '...'" % (a.prefix, a.bench_args)
    out = ["rocprofv3 kernel-trace summary: " + a.title, "",
           "command (run from /tmp with TMPDIR=/tmp on the MI355X box):",
           "  rocprofv3 --kernel-trace --stats --output-format csv -d RUN/trace -o bench -- python3 bench.py " + a.bench_args,
           "  python3 bench.py " + a.bench_args + " > RUN/plain.json   (optional: the unprofiled table at the end)",
           "  python3 -m inferspore_amd.profile_summary RUN --out profiles" + extra,
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
    plain = os.path.join(a.run, "plain.json")
    if os.path.exists(plain):
        with open(plain) as f:
            pj = json.loads([l for l in f.read().splitlines() if l.startswith("{")][-1])
        out += ["", "the same command without the profiler (python3 bench.py %s): HIP-event time per launch" % a.bench_args,
                "%-48s %10s %8s %8s" % ("workload", "us", "GB/s", "of 8TB/s")]
        for w, rec in pj["roofline"]["per_config"].items():
            out.append("%-48s %10.2f %8.0f %7.1f%%" % (w, rec["us"], rec["GBps"], 100.0 * rec["frac"]))
        if "fit" in pj:
            out.append("least-squares line over %s: time = %.2f us + bytes / %.0f GB/s"
                       % (pj["fit"].get("over", "the points"), pj["fit"]["fixed_us"], pj["fit"]["asymptotic_GBps"]))
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
