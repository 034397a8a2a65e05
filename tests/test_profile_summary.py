"""The profile summariser on a synthetic trace (CPU): dispatches are attributed to workloads through the
benchmark's launch log -- warm-up, gate copies and a discarded pass are skipped, the lead-in launches dropped, and
only the regions in which the host stayed ahead of the device are averaged (when there are at least three, the
benchmark's own rule)."""
import csv
import json
import os
import subprocess
import sys

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def write_trace(path, dispatches):
    """dispatches: list of (kernel name, duration ns, gap before it ns)."""
    t = 1000
    with open(path, "w", newline="") as f:
        w = csv.writer(f)
        w.writerow(["Kind", "Kernel_Name", "Start_Timestamp", "End_Timestamp"])
        for name, dur, gap in dispatches:
            t += gap
            w.writerow(["KERNEL_DISPATCH", name, t, t + dur])
            t += dur


def test_summary_follows_the_launch_log(tmp_path):
    run = tmp_path / "run"
    (run / "trace").mkdir(parents=True)
    norm, copy = "void isp::fused_norm_rows<__half, 2, 4, 1, 512>(__half*, int)", "void isp::copy_vec<1>(char*, char const*, unsigned long)"
    steps, lead_in, regions = 4, 2, 4
    d = []
    d += [(copy, 12000, 0)] * 5                      # device warm-up
    d += [(norm, 50000, 0)] * 3                      # warm-up of the workload: must not count
    d += [(copy, 330000, 0)] * 2                     # gate
    d += [(norm, 99000, 0)] * (lead_in + regions * steps)   # a discarded pass
    d += [(copy, 330000, 0)] * 4                     # a longer gate
    d += [(norm, 70000, 0)] * lead_in                # lead-in of the timed pass: dropped
    d += [(norm, 11000, 0)] * steps                  # region 0: ahead
    d += [(norm, 11200, 0)] * steps                  # region 1: ahead
    d += [(norm, 11100, 0)] * steps                  # region 2: ahead
    d += [(norm, 12400, 2000)] * steps               # region 3: the host fell behind (every launch after a gap)
    d += [(copy, 12000, 0)] * (lead_in + regions * steps)   # the copy workload, all regions ahead
    write_trace(run / "trace" / "bench_kernel_trace.csv", d)
    with open(run / "trace" / "bench_kernel_stats.csv", "w") as f:
        f.write("Name,Calls,TotalDurationNs,AverageNs,Percentage,MinNs,MaxNs,StdDev\n")
        f.write('"%s",10,1,11000.0,1.0,11000,12400,0\n' % norm)
    n_timed = lead_in + regions * steps
    bench = {
        "steps": steps, "warmup": 3, "lead_in": lead_in,
        "dispatch_log": [["device_warmup", "isp::copy_vec<1>", 5],
                         ["warmup:norm_w", "isp::fused_norm_rows<__half, 2, 4, 1, 512>", 3],
                         ["gate", "isp::copy_vec<1>", 2],
                         ["discarded:norm_w", "isp::fused_norm_rows<__half, 2, 4, 1, 512>", n_timed],
                         ["gate", "isp::copy_vec<1>", 4],
                         ["norm_w", "isp::fused_norm_rows<__half, 2, 4, 1, 512>", n_timed],
                         ["copy_w", "isp::copy_vec<1>", n_timed]],
        "regions_ahead": {"norm_w": [True, True, True, False], "copy_w": [True, True, True, True]},
        "roofline": {"per_config": {
            "norm_w": {"kernel": "isp::fused_norm_rows<__half, 2, 4, 1, 512>", "us": 11.1, "GBps": 1.0, "frac": 0.1, "bytes": 11100000},
            "copy_w": {"kernel": "isp::copy_vec<1>", "us": 12.0, "GBps": 1.0, "frac": 0.1, "bytes": 12000000}}},
    }
    with open(run / "trace" / "bench.json", "w") as f:
        f.write("some stderr noise\n" + json.dumps(bench) + "\n")
    out = tmp_path / "out"
    p = subprocess.run([sys.executable, "-m", "inferspore_amd.profile_summary", str(run), "--out", str(out)], cwd=ROOT,
                       stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    assert p.returncode == 0, p.stdout
    text = open(out / "all_kernels_benchmark_shapes.kernel_trace_stats.txt").read()
    rows = {l.split()[0]: l.split() for l in text.splitlines() if l.startswith(("norm_w", "copy_w"))}
    # workload, kernel (5 tokens: "isp::fused_norm_rows<__half," "2," "4," "1," "512>"), regions, calls, avg, med, min, max, GB/s, events, idle, n
    norm_row = rows["norm_w"]
    assert norm_row[6] == "3/4" and norm_row[7] == str(3 * steps)
    assert abs(float(norm_row[8]) - 11.10) < 1e-6 and float(norm_row[10]) == 11.00 and float(norm_row[11]) == 11.20
    assert abs(float(norm_row[12]) - 1000.0) < 1.0          # 11 100 000 bytes / 11.1 us
    assert float(norm_row[14]) == 12.40 and norm_row[15] == str(steps)   # the dispatches that started on an idle device
    copy_row = rows["copy_w"]
    assert copy_row[2] == "4/4" and copy_row[3] == str(regions * steps) and float(copy_row[4]) == 12.00
    assert "99.00" not in text and "70.00" not in text and "50.00" not in text   # discarded pass, lead-in, warm-up
