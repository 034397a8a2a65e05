#!/usr/bin/env python3
"""Benchmark of the fused per-layer kernels on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--only NAME] [--no-cpu] [--warm] [--full]

Prints ONE JSON line.  The headline workload is the fused add-bias + residual + RMSNorm in fp16 at
2048 tokens x 4096 hidden (one step = one launch over one batch); `roofline.per_config` carries the
same measurement for every kernel of the path at its LLaMA-2-7B shape.

Method
  * inputs are synthetic (torch's seeded device RNG), resident in HBM before the timed region;
  * every launch works on the next of R buffer sets, R chosen so the sets together exceed 1 GiB:
    successive launches cannot be served from the 256 MB last-level cache ("cold"; --warm disables
    the rotation and is reported separately, never as `value`);
  * after W warm-up launches and a synchronize, a gate of plain copies keeps the device busy while the
    host enqueues everything behind it: a few untimed lead-in launches and then several regions of
    exactly K launches each, back to back on a private stream, with a HIP event recorded on that stream
    at every region boundary; the reported time per launch is the MEDIAN region's event time / K (it
    includes the gaps between consecutive launches and the cost of the event markers, so it is a lower
    bound on the in-kernel rate); `queued_before_start` says that the host had enqueued every timed launch
    before the device left the gate, i.e. that the launches really ran back to back (under a profiler the
    host needs 10+ us per launch and short kernels would otherwise each start on an idle device);
    ms_per_step is the host wall clock from the first enqueue to the final synchronize, minus the gate's
    event-measured time, over the timed launches;
  * achieved = algorithmic bytes per launch (each operand once: compulsory reads + writes) / time;
  * roofline.traffic = HBM bytes per launch from rocprofv3 counters, read from
    profiles/hbm_traffic_per_launch.json (written by `python -m inferspore_amd.profile_summary`);
  * cpu_baseline: the C oracle (a port of the reference's CPU test functions) timed on the host
    cores of the same machine, on the same workload shapes, single thread plus an OpenMP run.
"""
import argparse
import ctypes
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
HBM_PEAK_GBS = 8000.0  # MI355X HBM3E, published peak
TRAFFIC_FILE = os.path.join(ROOT, "profiles", "hbm_traffic_per_launch.json")
HEADLINE = "fused_add_bias_residual_rmsnorm_f16_2048x4096"


def parse():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=200)
    ap.add_argument("--warmup", type=int, default=20)
    ap.add_argument("--regions", type=int, default=0,
                    help="timed regions of --steps launches per workload (default: enough for 300 launches, at least 5)")
    ap.add_argument("--only", default=None, help="run a single workload by name")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--kernels-only", action="store_true",
                    help="only the per-kernel workloads (no layer, decode-sequence, warm-cache or CPU legs) and a "
                         "`dispatch_log` of every launch in order: the form profile runs use")
    ap.add_argument("--warm", action="store_true",
                    help="report cache-warm (no rotation) rates for every workload, not only the hot-path ones")
    ap.add_argument("--full", action="store_true", help="also print the verbose per-workload records (`kernels`)")
    ap.add_argument("--copy-curve", action="store_true",
                    help="instead of the workloads, time the plain copy at 8 MiB .. 1 GiB of traffic per launch "
                         "(the practical ceiling as a function of launch size) and print it as one JSON line")
    ap.add_argument("--gather-locality", action="store_true",
                    help="instead of the workloads, time the embedding gather with ids in random runs of 1, 2, 4, 8, 32 "
                         "consecutive table rows and with the rows in order, beside a copy of equal bytes: how much of "
                         "the gather's distance to the copy is the randomness of its rows (one JSON line)")
    ap.add_argument("--cpu-seconds", type=float, default=20.0, help="budget of the CPU baseline leg")
    return ap.parse_args()


def measured_traffic():
    """HBM bytes per launch per workload, as the last committed profile run measured them."""
    try:
        with open(TRAFFIC_FILE) as f:
            return json.load(f).get("bytes_per_launch", {})
    except (OSError, ValueError):
        return {}


# --------------------------------------------------------------------------- workloads

class Workload:
    """One kernel at one shape: R rotating buffer sets and a launch(i) closure.

    launch(i) calls the C ABI directly with argument tuples prepared once (raw device pointers and
    ints), so the per-launch host cost is one ctypes call; the small kernels are launch-bound and
    every microsecond of host overhead would otherwise be billed to them."""
    name = ""
    dtype = ""
    tokens = 0
    bytes_per_launch = 0
    kernel = ""
    sets = 1
    keep = None
    launches_per_step = 1

    @staticmethod
    def sets_for(set_bytes, rotate):
        if not rotate:
            return 1
        return max(2, int((1 << 30) // max(set_bytes, 1)) + 1)

    def bind(self, fn, arg_sets):
        n = len(arg_sets)
        self.sets = n

        def launch(i):
            rc = fn(*arg_sets[i % n])
            if rc:
                raise RuntimeError("%s: C ABI returned %d" % (self.name, rc))
        self.launch = launch

    def bind_pair(self, fn_a, args_a, fn_b, args_b):
        """Two dependent launches per step (a fused kernel's unfused counterpart)."""
        n = len(args_a)
        self.sets = n
        self.launches_per_step = 2

        def launch(i):
            rc = fn_a(*args_a[i % n]) or fn_b(*args_b[i % n])
            if rc:
                raise RuntimeError("%s: C ABI returned %d" % (self.name, rc))
        self.launch = launch


def norm_kernel_name(lib, es, tokens, hidden, fused, with_bias=None):
    """The instantiation the launcher picks (`fused`: with a residual; `with_bias` defaults to `fused`)."""
    with_bias = fused if with_bias is None else (fused and with_bias)
    v = [ctypes.c_int() for _ in range(4)]
    rc = lib.isp_norm_launch_config(es, tokens, hidden, int(fused), *[ctypes.byref(x) for x in v])
    if rc:
        return "isp::fused_norm_generic"
    t = "__half" if es == 2 else "float"
    if lib.isp_norm_launch_variant(es, tokens, hidden, int(fused), int(with_bias), 0) == 1:
        return "isp::fused_norm_few_rows<%s, %d, %d, %d, %d>" % (t, v[1].value, v[0].value, v[3].value,
                                                                 (2 if with_bias else 1) if fused else 0)
    return "isp::fused_norm_rows<%s, %d, %d, %d, %d>" % (t, v[1].value, v[0].value, v[3].value, v[2].value)


def make_copy_workload(torch, lib, stream_handle, nbytes, rotate=True):
    """Plain copy of nbytes (traffic 2 x nbytes per launch), rotating over > 1 GiB of buffers."""
    w = Workload()
    w.name, w.dtype, w.tokens = "calibration_copy_%dMiB_traffic" % (2 * nbytes >> 20), "u8", 0
    w.kernel = "isp::copy_vec<1>"
    w.bytes_per_launch = 2 * nbytes
    R = w.sets_for(2 * nbytes, rotate)
    srcs = torch.empty((R, nbytes), device="cuda", dtype=torch.uint8).fill_(7)
    dsts = torch.empty((R, nbytes), device="cuda", dtype=torch.uint8)
    w.keep = (srcs, dsts)
    w.bind(lib.isp_calibration_copy, [(dsts[j].data_ptr(), srcs[j].data_ptr(), nbytes, stream_handle) for j in range(R)])
    w.reset = lambda: None
    w.config = {"bytes_copied": nbytes}
    return w


def make_workloads(torch, lib, stream_handle, rotate):
    dev = "cuda"
    st = stream_handle

    def norm(name, tokens, hidden, tdtype, fused, with_bias=True):
        w = Workload()
        es = 2 if tdtype == torch.float16 else 4
        sfx = "f16" if es == 2 else "f32"
        w.name, w.dtype, w.tokens = name, sfx, tokens
        if fused:
            w.bytes_per_launch = 4 * tokens * hidden * es + (2 if with_bias else 1) * hidden * es
            set_bytes = 2 * tokens * hidden * es
        else:
            w.bytes_per_launch = 2 * tokens * hidden * es + hidden * es
            set_bytes = tokens * hidden * es
        R = w.sets_for(set_bytes, rotate)
        # one allocation per operand, sliced into the R sets: a thousand separate small allocations
        # land on separately mapped pages, and launch-bound kernels then time up to 2x slower
        outs = list(torch.empty((R, tokens, hidden), device=dev, dtype=tdtype).normal_().unbind(0))
        ress = list(torch.empty((R, tokens, hidden), device=dev, dtype=tdtype).normal_().unbind(0)) if fused else None
        bias = (0.02 * torch.randn(hidden, device=dev)).to(tdtype) if fused and with_bias else None
        gamma = (0.5 + torch.rand(hidden, device=dev)).to(tdtype)
        w.keep = (outs, ress, bias, gamma)
        w.kernel = norm_kernel_name(lib, es, tokens, hidden, fused, with_bias)
        if fused:
            fn = getattr(lib, "isp_fused_add_bias_residual_rmsnorm_" + sfx)
            w.bind(fn, [(ress[j].data_ptr(), outs[j].data_ptr(), bias.data_ptr() if with_bias else None, gamma.data_ptr(),
                         1e-5, tokens, hidden, 0, st) for j in range(R)])
        else:
            fn = getattr(lib, "isp_rmsnorm_" + sfx)
            w.bind(fn, [(outs[j].data_ptr(), gamma.data_ptr(), 1e-5, tokens, hidden, st) for j in range(R)])

        def reset():
            # the kernel works in place: refresh the values so repeated launches stay finite
            for t in outs:
                t.normal_()
            if fused:
                for t in ress:
                    t.normal_()

        w.reset = reset
        w.config = {"tokens": tokens, "hidden": hidden}
        return w

    def embedding(tdtype=torch.float16, id_run=1):
        """id_run: 1 = independent random ids (the configuration); n > 1 = random runs of n consecutive table
        rows; 0 = the table rows in order (what a copy reads)."""
        w = Workload()
        tokens, hidden, vocab = 8192, 4096, 32000
        es = 2 if tdtype == torch.float16 else 4
        sfx = "f16" if es == 2 else "f32"
        w.name, w.dtype, w.tokens = "embedding_%s_8192x4096_v32000" % sfx, sfx, tokens
        if id_run != 1:
            w.name += "_runs_of_%d" % id_run
        w.kernel = "isp::gather_chunks_vec<2>"
        w.bytes_per_launch = 2 * tokens * hidden * es + tokens * 4
        table = (0.02 * torch.randn((vocab, hidden), device=dev)).to(tdtype)
        R = w.sets_for(tokens * hidden * es, rotate)
        if id_run == 1:
            ids = [torch.randint(0, vocab, (tokens,), device=dev, dtype=torch.int32) for _ in range(R)]
        elif id_run == 0:
            ids = [((torch.arange(tokens, device=dev) + j * tokens) % vocab).to(torch.int32) for j in range(R)]
        else:
            ids = [(torch.randint(0, vocab - id_run, (tokens // id_run,), device=dev).repeat_interleave(id_run) +
                    torch.arange(tokens, device=dev) % id_run).to(torch.int32) for _ in range(R)]
        outs = [torch.empty((tokens, hidden), device=dev, dtype=tdtype) for _ in range(R)]
        w.keep = (table, ids, outs)
        w.bind(getattr(lib, "isp_embedding_" + sfx), [(ids[j].data_ptr(), outs[j].data_ptr(), table.data_ptr(), tokens, hidden,
                                        vocab, st) for j in range(R)])
        w.reset = lambda: None
        w.config = {"tokens": tokens, "hidden": hidden, "vocab": vocab}
        return w

    def padded_batch():
        batch, seq = 8, 512
        lens = bench_lengths(torch, batch)
        lens_d = lens.to(dev)
        po = torch.zeros((batch, seq), device=dev, dtype=torch.int32)
        cum = torch.zeros((batch + 1,), device=dev, dtype=torch.int32)
        assert lib.isp_cal_padding_offset(po.data_ptr(), cum.data_ptr(), lens_d.data_ptr(), batch, seq, st) == 0
        return batch, seq, int(lens.sum()), lens_d, po

    def qkv(tdtype=torch.float16, hn=32, kvn=32, hs=128, tag="", with_bias=True):
        w = Workload()
        es = 2 if tdtype == torch.float16 else 4
        sfx = "f16" if es == 2 else "f32"
        batch, seq, tokens, lens_d, po = padded_batch()
        w.name, w.dtype, w.tokens = "qkv_bias_rope_transpose_%s_b8_s512%s" % (sfx, tag), sfx, tokens
        flag = "true" if with_bias else "false"
        if es == 2 and hs == 128 and hn % 4 == 0 and kvn % 4 == 0:
            w.kernel = "isp::qkv_rope_lean_f16<2, %s, false, %s>" % (flag, "false" if hn % 32 == 0 and kvn % 32 == 0 else "true")
        elif es == 4 and hs == 128 and hn % 2 == 0 and kvn % 2 == 0:
            w.kernel = "isp::qkv_rope_lean_f32<2, %s, false, %s>" % (flag, "false" if hn % 16 == 0 and kvn % 16 == 0 else "true")
        else:
            w.kernel = "isp::qkv_rope_wave<%s, %d, 2, 4, %s>" % ("__half" if es == 2 else "float", hs, flag)
        w.bytes_per_launch = tokens * (2 * (hn + 2 * kvn) * hs * es + 4) + 2 * batch * 4
        if with_bias:
            w.bytes_per_launch += (hn + 2 * kvn) * hs * es
        hist = torch.zeros(batch, device=dev, dtype=torch.int32)
        bias = (0.02 * torch.randn((hn + 2 * kvn) * hs, device=dev)).to(tdtype) if with_bias else None
        set_bytes = tokens * (hn + 2 * kvn) * hs * es + batch * (hn + 2 * kvn) * seq * hs * es
        R = w.sets_for(set_bytes, rotate)
        ins = [torch.randn((tokens, hn + 2 * kvn, hs), device=dev).to(tdtype) for _ in range(R)]
        outs = [[torch.zeros((batch, n, seq, hs), device=dev, dtype=tdtype) for n in (hn, kvn, kvn)]
                for _ in range(R)]
        w.keep = (lens_d, po, hist, bias, ins, outs)
        w.bind(getattr(lib, "isp_qkv_bias_rope_transpose_" + sfx),
               [(outs[j][0].data_ptr(), outs[j][1].data_ptr(), outs[j][2].data_ptr(), ins[j].data_ptr(),
                 bias.data_ptr() if with_bias else None, po.data_ptr(), hist.data_ptr(), lens_d.data_ptr(), batch, seq,
                 tokens, hn, kvn, hs, hs, 10000.0, 2048, 0, st) for j in range(R)])
        w.reset = lambda: None
        w.config = {"batch": batch, "max_seq": seq, "valid_tokens": tokens, "heads": "%dq/%dkv" % (hn, kvn),
                    "head_dim": hs}
        return w

    def qkv_append(fused, with_bias=True):
        """QKV step + KV-cache append at the benchmark shape: one fused launch (k and v rows written to the
        cache only), or the two launches it replaces.  Both are priced at the bytes the fused form has
        to move (packed qkv read once; q and the cache rows written once).  `with_bias=False` (fused form only)
        is the call a LLaMA layer makes."""
        w = Workload()
        tdtype, es, hn, kvn, hs, max_seq = torch.float16, 2, 32, 32, 128, 1024
        batch, seq, tokens, lens_d, po = padded_batch()
        w.dtype, w.tokens = "f16", tokens
        w.bytes_per_launch = tokens * (2 * (hn + 2 * kvn) * hs * es + 4) + 3 * batch * 4
        if with_bias:
            w.bytes_per_launch += (hn + 2 * kvn) * hs * es
        hist = torch.zeros(batch, device=dev, dtype=torch.int32)
        bias = (0.02 * torch.randn((hn + 2 * kvn) * hs, device=dev)).to(tdtype)
        set_bytes = tokens * (hn + 2 * kvn) * hs * es + batch * hn * seq * hs * es + 2 * batch * kvn * max_seq * hs * es
        if not fused:
            set_bytes += 2 * batch * kvn * seq * hs * es
        R = w.sets_for(set_bytes, rotate)
        ins = [torch.randn((tokens, hn + 2 * kvn, hs), device=dev).to(tdtype) for _ in range(R)]
        qs = [torch.zeros((batch, hn, seq, hs), device=dev, dtype=tdtype) for _ in range(R)]
        caches = [[torch.zeros((1, batch, kvn, max_seq, hs), device=dev, dtype=tdtype) for _ in range(2)] for _ in range(R)]
        w.keep = (lens_d, po, hist, bias, ins, qs, caches)
        if fused:
            w.name = "qkv_bias_rope_transpose_append_f16_b8_s512_S1024" + ("" if with_bias else "_no_bias")
            w.kernel = "isp::qkv_rope_lean_f16<2, %s, true, false>" % ("true" if with_bias else "false")
            w.bind(lib.isp_qkv_bias_rope_transpose_append_f16,
                   [(qs[j].data_ptr(), None, None, caches[j][0].data_ptr(), caches[j][1].data_ptr(), 0, max_seq,
                     ins[j].data_ptr(), bias.data_ptr() if with_bias else None, po.data_ptr(), hist.data_ptr(), lens_d.data_ptr(), batch, seq,
                     tokens, hn, kvn, hs, hs, 10000.0, st) for j in range(R)])
        else:
            w.name = "qkv_bias_rope_transpose_then_concat_kv_f16_b8_s512_S1024"
            w.kernel = "isp::qkv_rope_lean_f16<2, true, false, false> + isp::concat_kv_vec<256>"
            kvs = [[torch.zeros((batch, kvn, seq, hs), device=dev, dtype=tdtype) for _ in range(2)] for _ in range(R)]
            w.keep += (kvs,)
            w.bind_pair(lib.isp_qkv_bias_rope_transpose_f16,
                        [(qs[j].data_ptr(), kvs[j][0].data_ptr(), kvs[j][1].data_ptr(), ins[j].data_ptr(),
                          bias.data_ptr(), po.data_ptr(), hist.data_ptr(), lens_d.data_ptr(), batch, seq, tokens, hn,
                          kvn, hs, hs, 10000.0, 2048, 0, st) for j in range(R)],
                        lib.isp_concat_kv_cache_f16,
                        [(kvs[j][0].data_ptr(), kvs[j][1].data_ptr(), caches[j][0].data_ptr(), caches[j][1].data_ptr(),
                          0, lens_d.data_ptr(), hist.data_ptr(), batch, kvn, seq, max_seq, hs, st) for j in range(R)])
        w.reset = lambda: None
        w.config = {"batch": batch, "max_seq": seq, "valid_tokens": tokens, "max_seq_len": max_seq}
        return w

    def swiglu(tokens, tag, tdtype=torch.float16):
        w = Workload()
        inter = 11008
        es = 2 if tdtype == torch.float16 else 4
        sfx = "f16" if es == 2 else "f32"
        w.name, w.dtype, w.tokens = "swiglu_%s_%s_%dx%d" % (sfx, tag, tokens, inter), sfx, tokens
        w.kernel = "isp::swiglu_vec<%s, 1, 1>" % ("__half" if es == 2 else "float")
        w.bytes_per_launch = tokens * 3 * inter * es
        R = w.sets_for(w.bytes_per_launch, rotate)
        ins = list(torch.empty((R, tokens, 2, inter), device=dev, dtype=tdtype).normal_().unbind(0))
        outs = list(torch.empty((R, tokens, inter), device=dev, dtype=tdtype).unbind(0))
        w.keep = (ins, outs)
        w.bind(getattr(lib, "isp_swiglu_" + sfx),
               [(ins[j].data_ptr(), outs[j].data_ptr(), tokens, inter, st) for j in range(R)])
        w.reset = lambda: None
        w.config = {"tokens": tokens, "inter": inter}
        return w

    def transpose_out():
        w = Workload()
        batch, seq, tokens, lens_d, po = padded_batch()
        hn, hs = 32, 128
        w.name, w.dtype, w.tokens = "transpose_remove_padding_f16_b8_s512", "f16", tokens
        w.kernel = "isp::transpose_remove_padding_vec<64>"
        w.bytes_per_launch = tokens * (2 * hn * hs * 2 + 4)
        R = w.sets_for(batch * hn * seq * hs * 2 + tokens * hn * hs * 2, rotate)
        srcs = [torch.randn((batch, hn, seq, hs), device=dev).to(torch.float16) for _ in range(R)]
        dsts = [torch.empty((tokens, hn, hs), device=dev, dtype=torch.float16) for _ in range(R)]
        w.keep = (lens_d, po, srcs, dsts)
        w.bind(lib.isp_transpose_remove_padding_f16,
               [(srcs[j].data_ptr(), po.data_ptr(), dsts[j].data_ptr(), batch, hn, seq, hs, tokens, st)
                for j in range(R)])
        w.reset = lambda: None
        w.config = {"batch": batch, "max_seq": seq, "valid_tokens": tokens, "heads": hn, "head_dim": hs}
        return w

    def kv_cache(which):
        w = Workload()
        batch, seq, tokens, lens_d, po = padded_batch()
        kvn, hn, hs, max_seq, layers = 32, 32, 128, 1024, 1
        hist = torch.zeros(batch, device=dev, dtype=torch.int32)
        # append: read + write k and v rows of the valid tokens; broadcast: same volume with MHA (rep = 1)
        w.bytes_per_launch = 2 * 2 * tokens * kvn * hs * 2 + 2 * batch * 4
        w.dtype, w.tokens = "f16", tokens
        R = w.sets_for(2 * batch * kvn * (seq + max_seq) * hs * 2, rotate)
        smalls = [[torch.randn((batch, kvn, seq, hs), device=dev).to(torch.float16) for _ in range(2)] for _ in range(R)]
        caches = [[torch.zeros((layers, batch, kvn, max_seq, hs), device=dev, dtype=torch.float16) for _ in range(2)]
                  for _ in range(R)]
        w.keep = (lens_d, po, hist, smalls, caches)
        if which == "append":
            w.name, w.kernel = "concat_kv_cache_f16_b8_q512_S1024", "isp::concat_kv_vec<256>"
            w.bind(lib.isp_concat_kv_cache_f16,
                   [(smalls[j][0].data_ptr(), smalls[j][1].data_ptr(), caches[j][0].data_ptr(),
                     caches[j][1].data_ptr(), 0, lens_d.data_ptr(), hist.data_ptr(), batch, kvn, seq, max_seq, hs, st)
                    for j in range(R)])
        else:
            w.name, w.kernel = "repeat_kv_cache_f16_b8_k512_S1024", "isp::repeat_kv_vec<256>"
            w.bind(lib.isp_repeat_kv_cache_f16,
                   [(caches[j][0].data_ptr(), caches[j][1].data_ptr(), smalls[j][0].data_ptr(),
                     smalls[j][1].data_ptr(), 0, lens_d.data_ptr(), batch, hn, kvn, max_seq, seq, hs, st)
                    for j in range(R)])
        w.reset = lambda: None
        w.config = {"batch": batch, "max_q_len": seq, "max_seq_len": max_seq, "valid_tokens": tokens,
                    "kv_heads": kvn, "head_dim": hs}
        return w

    def rope_decode():
        w = Workload()
        w.name, w.dtype, w.tokens = "rope_decode_f16_1x96x128", "f16", 1
        w.kernel = "isp::rope_decode_wave<__half, 128>"
        w.bytes_per_launch = 2 * 64 * 128 * 2
        R = 64 if rotate else 1
        rows = list(torch.empty((R, 1, 96, 128), device=dev, dtype=torch.float16).normal_().unbind(0))
        w.keep = rows
        w.bind(lib.isp_rope_decode_f16, [(rows[j].data_ptr(), 1, 32, 32, 128, 17, 128, 10000.0, st) for j in range(R)])
        w.reset = lambda: None
        w.config = {"batch": 1, "heads": "32q/32kv", "head_dim": 128}
        return w

    def copy(nbytes):
        return make_copy_workload(torch, lib, st, nbytes, rotate)

    if rotate == "copy-curve":
        return [("calibration_copy_%dMiB_traffic" % mib, (lambda mib=mib: copy((mib << 20) // 2)))
                for mib in (1, 2, 4, 8, 16, 24, 32, 48, 64, 96, 128, 192, 256, 384, 512, 1024)]
    if rotate == "gather-locality":
        return [("embedding_f16_8192x4096_v32000" + ("_runs_of_%d" % n if n != 1 else ""),
                 (lambda n=n: embedding(id_run=n))) for n in (1, 2, 4, 8, 32, 0)] + [("calibration_copy_128MiB_traffic", lambda: copy(64 << 20))]
    table = [
        (HEADLINE, lambda: norm(HEADLINE, 2048, 4096, torch.float16, True)),
        # the same kernel at the row counts a prefill layer hands it (the ragged batch's 2977 valid tokens; 4096)
        ("fused_add_bias_residual_rmsnorm_f16_2977x4096",
         lambda: norm("fused_add_bias_residual_rmsnorm_f16_2977x4096", 2977, 4096, torch.float16, True)),
        ("fused_add_bias_residual_rmsnorm_f16_4096x4096",
         lambda: norm("fused_add_bias_residual_rmsnorm_f16_4096x4096", 4096, 4096, torch.float16, True)),
        # ... and as LLaMA calls it: a residual but no bias (its projections have none, layer_weights.cc:58-62)
        ("fused_add_residual_rmsnorm_f16_2048x4096_no_bias",
         lambda: norm("fused_add_residual_rmsnorm_f16_2048x4096_no_bias", 2048, 4096, torch.float16, True, False)),
        ("fused_add_residual_rmsnorm_f16_2977x4096_no_bias",
         lambda: norm("fused_add_residual_rmsnorm_f16_2977x4096_no_bias", 2977, 4096, torch.float16, True, False)),
        ("rmsnorm_f32_64x4096", lambda: norm("rmsnorm_f32_64x4096", 64, 4096, torch.float32, False)),
        # a decode step's two norms at batch 16 and 256: launch-bound, the kernels with the operand set fixed at compile time
        ("rmsnorm_f16_16x4096", lambda: norm("rmsnorm_f16_16x4096", 16, 4096, torch.float16, False)),
        ("fused_add_residual_rmsnorm_f16_16x4096_no_bias",
         lambda: norm("fused_add_residual_rmsnorm_f16_16x4096_no_bias", 16, 4096, torch.float16, True, False)),
        ("fused_add_residual_rmsnorm_f16_256x4096_no_bias",
         lambda: norm("fused_add_residual_rmsnorm_f16_256x4096_no_bias", 256, 4096, torch.float16, True, False)),
        ("rmsnorm_f32_16384x4096", lambda: norm("rmsnorm_f32_16384x4096", 16384, 4096, torch.float32, False)),
        ("embedding_f16_8192x4096_v32000", embedding),
        ("qkv_bias_rope_transpose_f16_b8_s512", qkv),
        # the same step as LLaMA runs it: its projections have no bias (layer_weights.cc:58-62 sets the pointers to null)
        ("qkv_bias_rope_transpose_f16_b8_s512_no_bias", lambda: qkv(tag="_no_bias", with_bias=False)),
        ("qkv_bias_rope_transpose_append_f16_b8_s512_S1024", lambda: qkv_append(True)),
        ("qkv_bias_rope_transpose_append_f16_b8_s512_S1024_no_bias", lambda: qkv_append(True, with_bias=False)),
        ("qkv_bias_rope_transpose_then_concat_kv_f16_b8_s512_S1024", lambda: qkv_append(False)),
        ("swiglu_f16_prefill_8192x11008", lambda: swiglu(8192, "prefill")),
        ("swiglu_f16_decode_256x11008", lambda: swiglu(256, "decode")),
        ("transpose_remove_padding_f16_b8_s512", transpose_out),
        ("concat_kv_cache_f16_b8_q512_S1024", lambda: kv_cache("append")),
        ("repeat_kv_cache_f16_b8_k512_S1024", lambda: kv_cache("broadcast")),
        ("rope_decode_f16_1x96x128", rope_decode),
        # the reference's own functional precision (its fp16 kernels are incomplete): fp32 storage
        ("fused_add_bias_residual_rmsnorm_f32_2048x4096",
         lambda: norm("fused_add_bias_residual_rmsnorm_f32_2048x4096", 2048, 4096, torch.float32, True)),
        ("embedding_f32_8192x4096_v32000", lambda: embedding(torch.float32)),
        ("qkv_bias_rope_transpose_f32_b8_s512", lambda: qkv(torch.float32)),
        ("qkv_bias_rope_transpose_f32_b8_s512_no_bias", lambda: qkv(torch.float32, tag="_no_bias", with_bias=False)),
        ("swiglu_f32_prefill_8192x11008", lambda: swiglu(8192, "prefill", torch.float32)),
        ("calibration_copy_2MiB_traffic", lambda: copy(1 << 20)),
        ("calibration_copy_16MiB_traffic", lambda: copy(8 << 20)),
        ("calibration_copy_64MiB_traffic", lambda: copy(32 << 20)),
        ("calibration_copy_512MiB_traffic", lambda: copy(256 << 20)),
    ]
    return table


# --------------------------------------------------------------------------- timing

LEAD_IN = 8   # untimed launches in front of the first region, so that it does not start on an empty queue


def region_count(steps, requested):
    if requested > 0:
        return requested
    return max(5, -(-300 // max(steps, 1)))


class QueueGate:
    """Keeps the device busy with plain copies while the host enqueues a workload's timed launches.

    The timed launches are meant to run back to back.  That only happens while the host enqueues faster
    than the device executes: a 3-12 us kernel launched from a Python loop is at that edge already, and
    under a profiler (whose interception costs the host 10+ us per launch) every such kernel starts on
    an idle device -- its duration then includes the start-up that a busy queue hides behind the previous
    kernel's tail (12.1-12.3 us instead of 11.3 us for the 2048 x 4096 fp16 fused norm), and the trace
    and the events disagree.  So each timed pass is preceded by G launches of a large copy (2 GiB of
    traffic, about a third of a millisecond each: few packets, because the launch queue is finite), G
    sized so that the copies outlast the host's enqueuing of every timed launch behind them.  A region
    counts as `queued` when the host had enqueued all of it before the device reached it."""
    BYTES = 1 << 30
    MAX_MS = 200.0

    def __init__(self, torch, lib, stream):
        self.torch, self.lib, self.stream, self.handle = torch, lib, stream, stream.cuda_stream
        with torch.cuda.stream(stream):
            self.src = torch.empty(self.BYTES, dtype=torch.uint8, device="cuda").fill_(3)
            self.dst = torch.empty(self.BYTES, dtype=torch.uint8, device="cuda")
        self.args = (self.dst.data_ptr(), self.src.data_ptr(), self.BYTES, self.handle)
        stream.synchronize()
        n = self.CALIBRATION_LAUNCHES - 2
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        self.launch(2)
        stream.synchronize()
        e0.record(stream)
        t0 = time.perf_counter()
        self.launch(n)
        t1 = time.perf_counter()
        e1.record(stream)
        stream.synchronize()
        self.device_us = e0.elapsed_time(e1) * 1e3 / n    # one gate copy on the device
        self.host_us = (t1 - t0) * 1e6 / n                # one launch's host cost in this process (profiler included)

    CALIBRATION_LAUNCHES = 18

    def launch(self, n):
        fn, args = self.lib.isp_calibration_copy, self.args
        for _ in range(n):
            fn(*args)

    def count(self, timed_launches, host_us):
        """Gate launches that outlast the host's enqueuing of themselves and of `timed_launches` more."""
        host_us = max(host_us, self.host_us)
        need_us = 1.3 * timed_launches * host_us + 200.0
        return min(int(need_us / self.device_us) + 2, int(self.MAX_MS * 1e3 / self.device_us))


PROBE = 16    # untimed launches after the warm-up whose enqueuing is timed on the host (to size the gate)


def time_workload(torch, w, steps, warmup, regions, stream, gate):
    """W warm-up launches, synchronize, the queue gate, then `regions` back-to-back regions of exactly
    `steps` launches with an event at every boundary.  Returns a dict: wall ms per launch over all regions
    (gate excluded), the median region's event ms per launch (over the regions in which the host stayed
    ahead of the device, when there are at least three such), fastest, slowest, and the launches issued in
    order (for the dispatch log)."""
    issued = []
    n_timed = regions * steps + LEAD_IN
    with torch.cuda.stream(stream):
        w.reset()
        for i in range(warmup):
            w.launch(i)
        stream.synchronize()
        # what one launch costs the host in this process, measured on an empty queue once everything
        # lazy has happened (under a profiler this is 10+ us)
        t0 = time.perf_counter()
        for i in range(PROBE):
            w.launch(i)
        host_us = (time.perf_counter() - t0) * 1e6 / PROBE
        stream.synchronize()
        issued.append(("warmup", warmup + PROBE))
        for attempt in range(2):
            w.reset()
            torch.cuda.synchronize()
            g = gate.count(n_timed, host_us)
            ev = [torch.cuda.Event(enable_timing=True) for _ in range(regions + 1)]
            eg = torch.cuda.Event(enable_timing=True)
            host_at = [0.0] * (regions + 1)
            n = 0
            t0 = time.perf_counter()
            eg.record(stream)
            gate.launch(g)
            for _ in range(LEAD_IN):
                w.launch(n)
                n += 1
            for r in range(regions):
                host_at[r] = time.perf_counter()
                ev[r].record(stream)
                for _ in range(steps):
                    w.launch(n)
                    n += 1
            host_at[regions] = time.perf_counter()
            ev[regions].record(stream)
            stream.synchronize()
            torch.cuda.synchronize()
            t1 = time.perf_counter()
            dev_at = [eg.elapsed_time(e) for e in ev]    # ms after the gate began on the device
            gate_ms = dev_at[0]                          # gate copies + lead-in launches
            per_all = [(dev_at[r + 1] - dev_at[r]) / steps for r in range(regions)]
            # The device cannot reach `eg` before t0, so it began region r no earlier than t0 + dev_at[r].
            # The host stayed ahead throughout region r if it began enqueuing the region before the device
            # began it and enqueued its last launch before the device began that one (rates in between are
            # steady, and a host that blocks does so on a full queue).
            ahead = [(host_at[r] - t0) * 1e3 < dev_at[r] and
                     (host_at[r + 1] - t0) * 1e3 < dev_at[r + 1] - per_all[r] for r in range(regions)]
            enqueue_us = (host_at[regions] - t0) * 1e6 / (g + n)
            issued.append(("gate", g))
            if sum(ahead) >= min(3, regions) or attempt == 1:
                issued.append(("timed", n))
                break
            issued.append(("discarded", n))
            host_us = 2.0 * max(host_us, (host_at[regions] - host_at[0]) * 1e6 / (regions * steps))
    good = [t for t, q in zip(per_all, ahead) if q]
    per = sorted(good if len(good) >= min(3, regions) else per_all)
    # the device is busy from the first gate copy to the last timed launch: what the wall clock saw beyond
    # the gate (and the lead-in, a few launches) is the timed launches plus the submit and wake-up latencies
    wall_ms = max((t1 - t0) * 1e3 - gate_ms, 0.0) / (regions * steps)
    return {"wall_ms": wall_ms, "event_ms": per[len(per) // 2], "fastest": per[0], "slowest": per[-1],
            "queued_before_start": (host_at[regions] - t0) * 1e3 < gate_ms, "regions_ahead": ahead,
            "gate_launches": g, "issued": issued, "host_enqueue_us_per_launch": enqueue_us,
            "host_us_per_launch_empty_queue": host_us, "per_region_ms": per_all}


def measure(torch, w, steps, warmup, regions, stream, traffic, gate):
    t = time_workload(torch, w, steps, warmup, regions, stream, gate)
    event_ms = t["event_ms"]
    gbs = w.bytes_per_launch / (event_ms * 1e-3) / 1e9
    return {
        "workload": w.name, "kernel": w.kernel, "dtype": w.dtype, "tokens": w.tokens, "buffer_sets": w.sets,
        "algorithmic_bytes": w.bytes_per_launch, "launches_per_step": w.launches_per_step,
        "ms_per_step_wall": t["wall_ms"], "ms_per_launch_events": event_ms,
        "ms_fastest_region": t["fastest"], "ms_slowest_region": t["slowest"], "regions": regions,
        "GBps": gbs, "frac_of_hbm_peak": gbs / HBM_PEAK_GBS,
        "tokens_per_s": (w.tokens / (event_ms * 1e-3)) if w.tokens else None,
        "traffic": traffic.get(w.name),
        "queued_before_start": t["queued_before_start"], "regions_queued": sum(t["regions_ahead"]),
        "regions_ahead": t["regions_ahead"], "gate_launches": t["gate_launches"],
        "host_enqueue_us_per_launch": t["host_enqueue_us_per_launch"],
        "issued": t["issued"],
    }


# --------------------------------------------------------------------------- one whole layer

def context_layer_record(torch, steps, warmup, stream):
    """One LLaMA-2-7B prefill layer (batch 8, max 512 tokens, ragged) with this library's kernels in model
    order and torch's library GEMMs / attention in between: what the per-kernel rates add up to."""
    from inferspore_amd import ops
    from inferspore_amd.context_layer import BatchState, LayerWeights, context_decoder_layer
    nh, hs, inter, seq, batch = 32, 128, 11008, 512, 8
    hidden = nh * hs
    lens = bench_lengths(torch, batch).tolist()
    with torch.cuda.stream(stream):
        w = LayerWeights(hidden, inter, torch.float16)
        st = BatchState(lens, seq, nh, nh, hs, inter, max_seq_len=seq, layers=1, dtype=torch.float16)
        residual = torch.randn((st.tokens, hidden), device="cuda").half()
        normed = residual.clone()
        ops.rmsnorm(normed, w.attn_norm, 1e-5)

        def step():
            return context_decoder_layer(normed, residual, w, st, 0, w.attn_norm)

        for _ in range(max(3, warmup // 4)):
            step()
            residual.normal_()
        stream.synchronize()
        n = max(10, steps // 10)
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record(stream)
        for _ in range(n):
            step()
        e1.record(stream)
        stream.synchronize()
    ms = e0.elapsed_time(e1) / n
    return {"workload": "llama2_7b_context_decoder_layer_f16_b8_s512", "valid_tokens": st.tokens,
            "ms_per_layer": ms, "tokens_per_s_per_layer": st.tokens / (ms * 1e-3), "iterations": n,
            "note": "library kernels via the C ABI; GEMMs and attention are torch library calls"}


def context_layer_cpp_record(torch, steps, warmup, layers=0, decode=False, attention=False):
    """The same layer through the C++ layer class (launch* kernels + hipBLASLt GEMMs called directly, attention fused
    on the matrix cores): runs build/bin/bench_context_layer in a child process and returns its JSON record.
    With `layers` > 0: the whole stack of that many layers (LlamaContextDecoder, build/bin/bench_context_decoder).
    With `decode`: one new token for each of 16 sequences that already hold 1023 tokens in the KV cache -- the same
    layer call as a decode step.  With `attention`: the layer's fused attention kernel alone (build/bin/bench_context_attention),
    with its rate against the fp16 MFMA peak over the causal flops."""
    import subprocess
    name = "bench_context_attention" if attention else "bench_context_decoder" if layers else "bench_context_layer"
    exe = os.path.join(ROOT, "build", "bin", name)
    if not os.path.exists(exe):
        return {"error": "build/bin/%s is missing (python -m inferspore_amd.build)" % name}
    lens = [str(int(v)) for v in bench_lengths(torch).tolist()]
    counts = [str(layers), "5", "2"] if layers else [str(max(10, steps // 10)), str(max(3, warmup // 4))]
    args = counts + ["512"] + lens
    if attention:
        args = [str(max(50, steps // 2)), "10", "512"] + lens
    if decode:
        args = ["--history", "1023", str(max(50, steps // 2)), "10", "1"] + ["1"] * 16
    try:
        p = subprocess.run([exe] + args, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True, timeout=300)
        lines = [l for l in p.stdout.splitlines() if l.startswith("{")]
        if p.returncode != 0 or not lines:
            return {"error": p.stdout[-400:]}
        return json.loads(lines[-1])
    except (OSError, subprocess.SubprocessError, ValueError) as e:
        return {"error": str(e)}


def norm_in_situ_record(torch, stream, isolated_us):
    """The fused norm where a LLaMA layer runs it: with a residual and no bias, straight behind the GEMM that produced
    its input (the output projection, [tokens, 4096] x [4096, 4096]^T in fp16), on the 2977 valid tokens of the batch.
    Two loops on one stream, each between HIP events: GEMM + norm, and the GEMM alone; the difference per
    iteration is what the norm costs in that place (the GEMMs are long enough for the host to stay ahead).
    `isolated_us` is the same kernel launched back to back on rotating cold buffers (roofline.per_config)."""
    from inferspore_amd import ops
    tokens, hidden, n = 2977, 4096, 200
    with torch.cuda.stream(stream):
        x = torch.randn((tokens, hidden), device="cuda").half()
        w = (torch.randn((hidden, hidden), device="cuda") / 64).half()
        y = torch.empty((tokens, hidden), device="cuda", dtype=torch.float16)
        residual = torch.randn((tokens, hidden), device="cuda").half()
        gamma = (0.5 + torch.rand(hidden, device="cuda")).half()

        def gemm():
            torch.mm(x, w.t(), out=y)

        def both():
            torch.mm(x, w.t(), out=y)
            ops.fused_add_bias_residual_rmsnorm(residual, y, None, gamma, 1e-5)

        def timed(fn):
            for _ in range(10):
                fn()
            stream.synchronize()
            e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            e0.record(stream)
            for _ in range(n):
                fn()
            e1.record(stream)
            stream.synchronize()
            return e0.elapsed_time(e1) * 1e3 / n

        rounds = []
        for _ in range(3):
            residual.normal_()
            g = timed(gemm)
            b = timed(both)
            rounds.append((b - g, g, b))
        rounds.sort()
        diff, g, b = rounds[1]
    bytes_ = 4 * tokens * hidden * 2 + hidden * 2
    return {"workload": "fused_add_residual_rmsnorm_f16_2977x4096_no_bias behind its producer GEMM",
            "gemm_us": g, "gemm_then_norm_us": b, "norm_in_situ_us": diff,
            "norm_in_situ_GBps": bytes_ / (diff * 1e-6) / 1e9 if diff > 0 else None,
            "norm_isolated_cold_us": isolated_us,
            "note": "in situ the norm's input was just written by the GEMM and its residual is reused every iteration, "
                    "so part of both may come from the last-level cache; the isolated figure is cold by construction"}


def decode_sequence_record(torch, stream):
    """The launch-bound side: one decode step's worth of this library's kernels (batch 16: fused norm,
    decode RoPE, KV append, KV broadcast, SwiGLU, RMSNorm) issued eagerly and replayed from a captured
    HIP graph -- the entry points record only kernel nodes, so a caller can amortise launch latency."""
    from inferspore_amd import ops
    batch, kvn, hn, hs, max_seq, inter = 16, 32, 32, 128, 256, 11008
    with torch.cuda.stream(stream):
        h = lambda *sh: torch.randn(sh, device="cuda").half()
        hidden, residual, gamma = h(batch, 4096), h(batch, 4096), h(4096)
        qkv = h(1, 96, 128)
        k_new, v_new = h(batch, kvn, 1, hs), h(batch, kvn, 1, hs)
        ones = torch.ones(batch, dtype=torch.int32, device="cuda")
        hist, ctx = ones * 100, ones * 101
        k_cache, v_cache = h(1, batch, kvn, max_seq, hs), h(1, batch, kvn, max_seq, hs)
        k_rep = torch.zeros((batch, hn, 101, hs), dtype=torch.float16, device="cuda")
        v_rep = torch.zeros_like(k_rep)
        gate_up, act_out = h(batch, 2, inter), torch.zeros((batch, inter), dtype=torch.float16, device="cuda")

        def step():
            ops.fused_add_bias_residual_rmsnorm(residual, hidden, None, gamma, 1e-5)
            ops.rope(qkv, 101, 32, 128, 10000.0)
            ops.concat_kv_cache(k_new, v_new, 0, ones, hist, k_cache, v_cache)
            ops.repeat_kv_cache(k_cache, v_cache, ctx, 0, k_rep, v_rep)
            ops.act(gate_up, act_out)
            ops.rmsnorm(hidden, gamma, 1e-5)

        def timed(fn, n):
            for _ in range(5):
                fn()
            stream.synchronize()
            e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            e0.record(stream)
            for _ in range(n):
                fn()
            e1.record(stream)
            stream.synchronize()
            return e0.elapsed_time(e1) * 1e3 / n

        # the same step with bias + RoPE + append in one launch (the packed buffer then holds the whole batch)
        qkv_b = h(batch, 96, 128)

        def fused_step():
            ops.fused_add_bias_residual_rmsnorm(residual, hidden, None, gamma, 1e-5)
            ops.rope_decode_and_append(qkv_b, None, k_cache, v_cache, 0, hist, 101, 32, 128, 10000.0)
            ops.repeat_kv_cache(k_cache, v_cache, ctx, 0, k_rep, v_rep)
            ops.act(gate_up, act_out)
            ops.rmsnorm(hidden, gamma, 1e-5)

        out = {"workload": "decode_step_sequence_b16"}
        for tag, fn, n_kernels in (("", step, 6), ("fused_", fused_step, 5)):
            eager_us = timed(fn, 200)
            graph = torch.cuda.CUDAGraph()
            graph.capture_begin()
            fn()
            graph.capture_end()
            stream.synchronize()
            out[tag + "eager_us_per_step"] = eager_us
            out[tag + "graph_replay_us_per_step"] = timed(graph.replay, 200)
            out[tag + "kernels_per_step"] = n_kernels
    # the fused step from a C++ caller (no ctypes call per launch)
    import subprocess
    exe = os.path.join(ROOT, "build", "bin", "bench_decode_sequence")
    if os.path.exists(exe):
        try:
            p = subprocess.run([exe, "500"], stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True, timeout=120)
            lines = [l for l in p.stdout.splitlines() if l.startswith("{")]
            if p.returncode == 0 and lines:
                out.update(json.loads(lines[-1]))
            else:
                out["cpp_error"] = p.stdout[-300:]
        except (OSError, subprocess.SubprocessError, ValueError) as e:
            out["cpp_error"] = str(e)
    return out


# --------------------------------------------------------------------------- CPU baseline

def bench_lengths(torch, batch=8, lo=256, hi=512):
    """The ragged batch of the QKV configuration: per-sequence lengths uniform in [256, 512], seed 0."""
    g = torch.Generator(device="cpu").manual_seed(0)
    return torch.randint(lo, hi + 1, (batch,), generator=g, dtype=torch.int32)


def cpu_baseline(budget_s, lens):
    """Times the C oracle (a port of the reference's CPU test functions, tests/unittests/*.cu) on the
    host cores, once per BASELINE configuration at its full size: single thread (as the reference's
    loops are written) and OpenMP over token rows on every core this job may use.  Where one thread
    would take too long for the budget it runs a stated sample of the rows.  The headline entry is the
    fused norm at its full size."""
    import numpy as np
    sys.path.insert(0, ROOT)
    from oracle import load
    o = load()
    L = o.lib
    r = np.random.default_rng(0)
    f16 = np.float16

    def normal(*shape, scale=1.0, dtype=f16):
        a = r.standard_normal(shape, dtype=np.float32)
        if scale != 1.0:
            a *= scale
        return a.astype(dtype)

    def p(a):
        return a.ctypes.data

    # (workload, tokens, bytes, full callable, reset or None, one-thread callable or None, one-thread
    #  tokens, one-thread bytes, sample note, cache note)
    samples = []

    tokens, hidden = 2048, 4096
    out, res = normal(tokens, hidden), normal(tokens, hidden)
    bias, gamma = normal(hidden, scale=0.02), r.uniform(0.5, 1.5, hidden).astype(f16)
    wa, wb = out.copy(), res.copy()

    def norm_reset():
        wa[...] = out
        wb[...] = res
    nb = 4 * tokens * hidden * 2 + 2 * hidden * 2
    samples.append(dict(workload=HEADLINE, tokens=tokens, bytes=nb, reset=norm_reset,
                        fn=lambda: L.isp_oracle_fused_norm_f16(p(wb), p(wa), p(bias), p(gamma), 1e-5, tokens, hidden, 0),
                        sample="full workload", cache="64 MiB working set: exceeds one core's caches, may sit in a "
                                                      "large shared L3 between repetitions"))
    x32 = normal(64, hidden, dtype=np.float32)
    g32 = r.uniform(0.5, 1.5, hidden).astype(np.float32)
    w32 = x32.copy()
    samples.append(dict(workload="rmsnorm_f32_64x4096", tokens=64, bytes=2 * 64 * hidden * 4 + hidden * 4,
                        fn=lambda: L.isp_oracle_fused_norm_f32(None, p(w32), None, p(g32), 1e-5, 64, hidden, 0),
                        reset=lambda: w32.__setitem__(Ellipsis, x32), sample="full workload",
                        cache="1 MiB: cache-resident"))
    # embedding: a random table, and different random ids on every repetition (the same ids again would
    # turn the gather into a replay of 64 MiB of rows that a large L3 still holds)
    et, vocab = 8192, 32000
    table = r.integers(0, 0x3000, (vocab, hidden), dtype=np.uint16).view(f16)   # random finite bit patterns
    id_sets = [r.integers(0, vocab, et, dtype=np.int32) for _ in range(8)]
    eo = np.empty((et, hidden), f16)
    turn = [0]

    def gather():
        ids = id_sets[turn[0] % len(id_sets)]
        turn[0] += 1
        L.isp_oracle_embedding(p(ids), p(eo), p(table), et, hidden, 2)
    samples.append(dict(workload="embedding_f16_8192x4096_v32000", tokens=et, bytes=2 * et * hidden * 2 + et * 4,
                        fn=gather, reset=None, sample="full workload, fresh random ids per repetition",
                        cache="rows come from a 262 MB table (DRAM); the 64 MiB output is rewritten in place"))
    # QKV + RoPE: the whole ragged batch
    batch, seq, heads, hs = 8, 512, 96, 128
    lens = np.ascontiguousarray(lens, dtype=np.int32)
    qt = int(lens.sum())
    qkv, qb = normal(qt, heads, hs), normal(heads * hs, scale=0.02)
    qo = [np.zeros((batch, 32, seq, hs), f16) for _ in range(3)]
    po = np.repeat(np.concatenate([[0], np.cumsum(seq - lens)[:-1]]), lens).astype(np.int32)
    hist = np.zeros(batch, np.int32)
    samples.append(dict(workload="qkv_bias_rope_transpose_f16_b8_s512", tokens=qt,
                        bytes=qt * (2 * heads * hs * 2 + 4) + heads * hs * 2 + 2 * batch * 4,
                        fn=lambda: L.isp_oracle_qkv_rope_f16(p(qo[0]), p(qo[1]), p(qo[2]), p(qkv), p(qb), p(po), p(hist),
                                                             p(lens), batch, seq, qt, 32, 32, hs, 128, 10000.0),
                        reset=None, sample="full workload (8 sequences, %d tokens)" % qt,
                        cache="compute-bound on the CPU (powf, cos, sin per element, as the reference's loop)"))
    # SwiGLU prefill: all 8192 rows under OpenMP; one thread runs the first 1024 rows
    inter, st_full, st_one = 11008, 8192, 1024
    sx = np.empty((st_full, 2, inter), f16)
    for i in range(0, st_full, 1024):
        sx[i:i + 1024] = normal(1024, 2, inter)
    so = np.empty((st_full, inter), f16)
    samples.append(dict(workload="swiglu_f16_prefill_8192x11008", tokens=st_full, bytes=st_full * 3 * inter * 2,
                        fn=lambda: L.isp_oracle_swiglu_f16(p(sx), p(so), st_full, inter), reset=None,
                        one_fn=lambda: L.isp_oracle_swiglu_f16(p(sx), p(so), st_one, inter), one_tokens=st_one,
                        one_bytes=st_one * 3 * inter * 2,
                        sample="OpenMP: full workload; one thread: the first %d of %d rows" % (st_one, st_full),
                        cache="541 MB: DRAM"))
    sd = 256
    samples.append(dict(workload="swiglu_f16_decode_256x11008", tokens=sd, bytes=sd * 3 * inter * 2,
                        fn=lambda: L.isp_oracle_swiglu_f16(p(sx), p(so), sd, inter), reset=None,
                        sample="full workload", cache="17 MB: cache-resident between repetitions"))
    # padding offsets: the reference's serial loop (one thread by construction)
    ppo, pcum = np.zeros((batch, seq), np.int32), np.zeros(batch + 1, np.int32)
    samples.append(dict(workload="cal_padding_offset_b8_s512", tokens=qt, bytes=qt * 4 + (2 * batch + 1) * 4,
                        fn=lambda: L.isp_oracle_cal_padding_offset(p(ppo), p(pcum), p(lens), batch, seq), reset=None,
                        serial_only=True, sample="full workload", cache="12 KB: cache-resident"))

    def timed(fn, reset, threads, budget):
        o.set_threads(threads)
        times = []
        t_end = time.perf_counter() + budget
        while len(times) < 2 or (time.perf_counter() < t_end and len(times) < 30):
            if reset:
                reset()
            t0 = time.perf_counter()
            fn()
            times.append(time.perf_counter() - t0)
        o.set_threads(1)
        times.sort()
        return times[len(times) // 2], len(times)

    cores = o.max_threads()   # OMP_NUM_THREADS if set (the GPU box sets it to this job's CPU share), else all cores
    per = budget_s / (2.0 * len(samples))
    records = []
    for s in samples:
        one_fn = s.get("one_fn", s["fn"])
        t1, n1 = timed(one_fn, s["reset"], 1, per * 1.4)
        b1, k1 = s.get("one_bytes", s["bytes"]), s.get("one_tokens", s["tokens"])
        rec = {"workload": s["workload"], "sample": s["sample"], "kind": "port", "memory": s["cache"],
               "one_thread": {"GBps": b1 / t1 / 1e9, "tokens_per_s": k1 / t1, "us": t1 * 1e6, "cores": 1, "runs": n1}}
        if not s.get("serial_only"):
            tn, nn = timed(s["fn"], s["reset"], cores, per * 0.6)
            rec["openmp"] = {"GBps": s["bytes"] / tn / 1e9, "tokens_per_s": s["tokens"] / tn, "us": tn * 1e6,
                             "cores": cores, "runs": nn}
        records.append(rec)
    head = records[0]
    return {
        "value": head["one_thread"]["GBps"], "unit": "GB/s", "cores": 1, "kind": "port",
        "sample": "full workload (2048x4096 fp16 fused add-bias+residual+RMSNorm), median of %d runs"
                  % head["one_thread"]["runs"],
        "tokens_per_s": head["one_thread"]["tokens_per_s"],
        "openmp": {"value": head["openmp"]["GBps"], "unit": "GB/s", "cores": cores,
                   "tokens_per_s": head["openmp"]["tokens_per_s"]},
        "host_cpus": os.cpu_count(), "openmp_threads": cores,
        "per_kernel": records,
    }


# --------------------------------------------------------------------------- main

def compact(r):
    """The per-workload record that travels inside `roofline.per_config`."""
    out = {"kernel": r["kernel"], "us": round(r["ms_per_launch_events"] * 1e3, 3), "GBps": round(r["GBps"], 1),
           "frac": round(r["frac_of_hbm_peak"], 4), "bytes": r["algorithmic_bytes"], "traffic": r["traffic"]}
    if r.get("vs_copy") is not None:
        out["vs_copy"] = round(r["vs_copy"], 3)
    if r["tokens_per_s"]:
        out["tokens_per_s"] = round(r["tokens_per_s"])
    if r["launches_per_step"] != 1:
        out["launches_per_step"] = r["launches_per_step"]
    if r.get("regions_queued", r["regions"]) < r["regions"]:
        out["regions_queued"] = r["regions_queued"]   # of r["regions"]: the host fell behind the device in the others
    return out


def main():
    a = parse()
    if a.gpus != 1:
        print("bench.py: this build measures one GPU only; --gpus %d is not supported (use --gpus 1)" % a.gpus,
              file=sys.stderr)
        sys.exit(2)
    import torch
    if not torch.cuda.is_available():
        print("bench.py: no GPU available; the kernels have no CPU path", file=sys.stderr)
        sys.exit(3)
    from inferspore_amd import capi
    lib = capi.lib()
    capi.check(lib.isp_init(), "isp_init")
    torch.manual_seed(0)
    stream = torch.cuda.Stream()
    handle = stream.cuda_stream
    regions = region_count(a.steps, a.regions)
    traffic = measured_traffic()
    dispatch_log = []

    def log_issued(name, w, issued):
        """Every launch of a workload's measurement in order: warm-up, gate copies, timed launches (the first
        LEAD_IN of them untimed); a pass that was repeated with a longer gate is logged as discarded."""
        for kind, count in issued:
            if kind == "gate":
                dispatch_log.append(["gate", "isp::copy_vec<1>", count])
            else:
                dispatch_log.append([name if kind == "timed" else kind + ":" + name, w.kernel,
                                     count * w.launches_per_step])

    def run_all(rotate, names=None):
        out = []
        for name, make in make_workloads(torch, lib, handle, rotate):
            if a.only and a.only != name:
                continue
            if names is not None and name not in names:
                continue
            with torch.cuda.stream(stream):
                w = make()
            torch.cuda.synchronize()
            r = measure(torch, w, a.steps, a.warmup, regions, stream, traffic, gate)
            out.append(r)
            log_issued(name, w, r.pop("issued"))
            # the buffers go back to torch's caching allocator, not to the driver: kernels that run
            # on freshly mapped device memory measured up to 2x slower at launch-bound sizes
            del w
        return out

    # bring the device out of its idle clocks before the first timed region (the headline workload is
    # measured first): ~50 ms of streaming copies, untimed
    with torch.cuda.stream(stream):
        a_buf = torch.empty(64 << 20, dtype=torch.uint8, device="cuda")
        b_buf = torch.empty(64 << 20, dtype=torch.uint8, device="cuda")
        for _ in range(2000):
            lib.isp_calibration_copy(b_buf.data_ptr(), a_buf.data_ptr(), 64 << 20, handle)
        stream.synchronize()
        del a_buf, b_buf
    dispatch_log.append(["device_warmup", "isp::copy_vec<1>", 2000])
    gate = QueueGate(torch, lib, stream)
    dispatch_log.append(["gate_calibration", "isp::copy_vec<1>", QueueGate.CALIBRATION_LAUNCHES])

    def side_study(line, results):
        """The special modes print the same per-workload records and launch log as --kernels-only, so that
        `python -m inferspore_amd.profile_summary` can summarise a rocprofv3 trace of them too."""
        line.update({"steps": a.steps, "warmup": a.warmup, "lead_in": LEAD_IN, "dispatch_log": dispatch_log,
                     "regions_ahead": {r["workload"]: r["regions_ahead"] for r in results},
                     "roofline": {"per_config": {r["workload"]: compact(r) for r in results}}})
        print(json.dumps(line))

    if a.copy_curve:
        results = run_all("copy-curve")
        points = [{"traffic_MiB": r["algorithmic_bytes"] >> 20, "us_per_launch": r["ms_per_launch_events"] * 1e3,
                   "GBps": r["GBps"], "frac_of_hbm_peak": r["frac_of_hbm_peak"]} for r in results]
        # least-squares line  time = fixed + bytes / rate  over the points from 16 MiB up
        fit = [p for p in points if p["traffic_MiB"] >= 16]
        xs = [p["traffic_MiB"] * 2.0 ** 20 for p in fit]
        ys = [p["us_per_launch"] for p in fit]
        n = len(xs)
        mx, my = sum(xs) / n, sum(ys) / n
        slope = sum((x - mx) * (y - my) for x, y in zip(xs, ys)) / sum((x - mx) ** 2 for x in xs)
        side_study({"metric": "plain copy (isp_calibration_copy) vs traffic per launch", "unit": "GB/s", "points": points,
                    "fit": {"fixed_us": my - slope * mx, "asymptotic_GBps": 1e-3 / slope, "over": "16 MiB .. 1 GiB"}},
                   results)
        return

    if a.gather_locality:
        results = run_all("gather-locality")
        side_study({"metric": "embedding gather vs locality of the token ids (8192 ids, 32000 x 4096 fp16 table)",
                    "unit": "us per launch",
                    "points": {r["workload"]: {"us": round(r["ms_per_launch_events"] * 1e3, 3),
                                               "GBps": round(r["GBps"], 1)} for r in results}}, results)
        return

    results = run_all(True)
    head = results[0]
    # The practical ceiling of this device for a read+write stream, from the two plain copies of
    # this very run: time = fixed + bytes / rate.  Each kernel is also priced against the copy of
    # equal algorithmic bytes ("vs_copy" = copy-model time / kernel time; 1.0 = at the ceiling).
    by_name = {r["workload"]: r for r in results}
    c_small, c_big = by_name.get("calibration_copy_64MiB_traffic"), by_name.get("calibration_copy_512MiB_traffic")
    copy_model = None
    if c_small and c_big:
        rate = (c_big["algorithmic_bytes"] - c_small["algorithmic_bytes"]) / (
            c_big["ms_per_launch_events"] - c_small["ms_per_launch_events"])          # bytes per ms
        fixed = c_small["ms_per_launch_events"] - c_small["algorithmic_bytes"] / rate  # ms
        copy_model = {"fixed_us": round(fixed * 1e3, 3), "asymptotic_GBps": round(rate / 1e6, 1),
                      "form": "copy_time = fixed_us + bytes / asymptotic rate from 64 MiB of traffic up; below that, "
                              "interpolated between the copies measured at 2, 16 and 64 MiB of traffic (a launch "
                              "of a few MiB does not ramp up to the asymptotic rate)"}
        # measured copy points (bytes, ms), ascending: the model passes through every one of them
        points = sorted((r["algorithmic_bytes"], r["ms_per_launch_events"]) for r in results
                        if r["workload"].startswith("calibration_copy_"))
        copy_model["measured_us"] = {"%dMiB" % (b >> 20): round(t * 1e3, 3) for b, t in points}

        def copy_time(nbytes):
            if nbytes >= points[-2][0] or len(points) < 3:
                return fixed + nbytes / rate
            if nbytes <= points[0][0]:
                return points[0][1]   # the floor: a smaller launch is not faster
            for (b0, t0), (b1, t1) in zip(points, points[1:]):
                if nbytes <= b1:
                    return t0 + (t1 - t0) * (nbytes - b0) / (b1 - b0)
            return fixed + nbytes / rate

        for r in results:
            t = copy_time(r["algorithmic_bytes"])
            r["copy_model_ms"] = t
            r["vs_copy"] = t / r["ms_per_launch_events"]
    config = {"workload": head["workload"], "storage_dtype": "f16", "tokens_per_s": head["tokens_per_s"],
              "cache": "cold: launches rotate over %d buffer sets (> 1 GiB)" % head["buffer_sets"],
              "timing": "median of %d back-to-back regions of %d launches, HIP events on the launch stream"
                        % (regions, a.steps)}
    if copy_model:
        config["copy_ceiling"] = copy_model
    line = {}
    if a.full:
        line["kernels"] = results
    if a.kernels_only:
        line["dispatch_log"] = dispatch_log
        line["lead_in"] = LEAD_IN
        line["regions_ahead"] = {r["workload"]: r["regions_ahead"] for r in results}
    if not a.only and not a.kernels_only:
        layer = context_layer_record(torch, a.steps, a.warmup, stream)
        own = {"qkv_bias_rope_transpose_f16_b8_s512": 1, "concat_kv_cache_f16_b8_q512_S1024": 1,
               "repeat_kv_cache_f16_b8_k512_S1024": 1, "transpose_remove_padding_f16_b8_s512": 1}
        tokens = layer["valid_tokens"]
        # fused norm (x2) and SwiGLU run on `tokens` rows here; scale their measured per-token cost
        est = sum(by_name[k]["ms_per_launch_events"] for k in own if k in by_name)
        est += 2 * by_name[HEADLINE]["ms_per_launch_events"] * tokens / 2048
        est += by_name["swiglu_f16_prefill_8192x11008"]["ms_per_launch_events"] * tokens / 8192
        layer["library_kernels_ms_estimate"] = est
        layer["library_kernels_share"] = est / layer["ms_per_layer"]
        config["context_layer"] = layer
        config["context_layer_cpp"] = context_layer_cpp_record(torch, a.steps, a.warmup)
        config["context_decoder_cpp"] = context_layer_cpp_record(torch, a.steps, a.warmup, layers=32)
        config["context_layer_cpp_decode_step"] = context_layer_cpp_record(torch, a.steps, a.warmup, decode=True)
        config["context_attention_cpp"] = context_layer_cpp_record(torch, a.steps, a.warmup, attention=True)
        config["decode_sequence"] = decode_sequence_record(torch, stream)
        iso = by_name.get("fused_add_residual_rmsnorm_f16_2977x4096_no_bias")
        config["norm_in_situ"] = norm_in_situ_record(torch, stream, iso["ms_per_launch_events"] * 1e3 if iso else None)
    if not a.kernels_only:
        # cache-resident rates (one buffer set, no rotation): the hot-path configurations by default, every
        # workload with --warm.  These are not HBM rates: the 256 MB last-level cache serves part of them.
        hot = None if a.warm else {
            HEADLINE, "rmsnorm_f32_64x4096", "embedding_f16_8192x4096_v32000",
            "qkv_bias_rope_transpose_f16_b8_s512", "swiglu_f16_prefill_8192x11008", "swiglu_f16_decode_256x11008"}
        config["warm_cache_GBps"] = {r["workload"]: round(r["GBps"], 1) for r in run_all(False, hot)}
    line.update({
        "metric": "HBM GB/s & % of peak per fused kernel at LLaMA-2-7B shapes; tokens/sec",
        "value": head["GBps"], "unit": "GB/s", "n_gpus": 1, "steps": a.steps, "warmup": a.warmup,
        "ms_per_step": head["ms_per_step_wall"], "higher_is_better": True, "scaling": "weak",
        "vs_baseline": None, "dtype": "f32", "data": "synthetic",
        "config": config,
        "roofline": {"bound": "hbm", "achieved": head["GBps"], "peak": HBM_PEAK_GBS, "unit": "GB/s",
                     "frac": head["GBps"] / HBM_PEAK_GBS, "traffic": head["traffic"], "kernel": head["kernel"],
                     "algorithmic_bytes_per_launch": head["algorithmic_bytes"],
                     "avg_launch_ms": head["ms_per_launch_events"],
                     "fastest_region_ms": head["ms_fastest_region"], "slowest_region_ms": head["ms_slowest_region"],
                     "vs_copy": head.get("vs_copy"),
                     "queued_before_start": head["queued_before_start"], "regions_queued": head["regions_queued"],
                     "regions": head["regions"], "gate_launches": head["gate_launches"],
                     "host_enqueue_us_per_launch": round(head["host_enqueue_us_per_launch"], 2),
                     "per_config": {r["workload"]: compact(r) for r in results}},
    })
    if not a.no_cpu and not a.kernels_only:
        line["cpu_baseline"] = cpu_baseline(a.cpu_seconds, bench_lengths(torch).numpy())
    print(json.dumps(line))


if __name__ == "__main__":
    main()
