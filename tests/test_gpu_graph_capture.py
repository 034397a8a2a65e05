"""The entry points allocate nothing, synchronise nothing and record only kernel nodes, so a caller
can capture a launch-bound sequence of them into a HIP graph.  A decode-step-like sequence is captured
once and replayed several times, with eager work and synchronisation between replays; every replay
must reproduce the eager results bit for bit."""
import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu


def _sequence(isp, t):
    """One decode step's worth of the memory-bound kernels on pre-allocated tensors (batch of 16)."""
    isp.fused_add_bias_residual_rmsnorm(t["residual"], t["hidden"], None, t["gamma"], 1e-5)
    isp.rope(t["qkv"], t["step"], 32, 128, 10000.0)
    isp.concat_kv_cache(t["k_new"], t["v_new"], 0, t["cur"], t["hist"], t["k_cache"], t["v_cache"])
    isp.repeat_kv_cache(t["k_cache"], t["v_cache"], t["ctx"], 0, t["k_rep"], t["v_rep"])
    isp.act(t["gate_up"], t["act_out"])
    isp.rmsnorm(t["hidden"], t["gamma"], 1e-5)


def _tensors(seed):
    g = torch.Generator(device="cuda").manual_seed(seed)
    r = lambda *s: torch.randn(s, device="cuda", generator=g).half()
    batch, kvn, hn, hs, max_seq = 16, 8, 32, 128, 64
    return {
        "hidden": r(batch, 4096), "residual": r(batch, 4096), "gamma": r(4096),
        "qkv": r(1, 96, 128), "step": 9,
        "k_new": r(batch, kvn, 1, hs), "v_new": r(batch, kvn, 1, hs),
        "cur": torch.ones(batch, dtype=torch.int32, device="cuda"),
        "hist": torch.full((batch,), 8, dtype=torch.int32, device="cuda"),
        "ctx": torch.full((batch,), 9, dtype=torch.int32, device="cuda"),
        "k_cache": r(1, batch, kvn, max_seq, hs), "v_cache": r(1, batch, kvn, max_seq, hs),
        "k_rep": torch.zeros((batch, hn, 9, hs), dtype=torch.float16, device="cuda"),
        "v_rep": torch.zeros((batch, hn, 9, hs), dtype=torch.float16, device="cuda"),
        "gate_up": r(batch, 2, 11008), "act_out": torch.zeros((batch, 11008), dtype=torch.float16, device="cuda"),
    }


def _snapshot(t):
    return {k: v.clone() for k, v in t.items() if torch.is_tensor(v)}


def test_capture_and_replay_matches_eager(isp):
    print("[case] graph capture of a decode-step sequence", flush=True)
    t = _tensors(1)
    initial = _snapshot(t)
    # eager reference: three steps in a row (the in-place kernels make each step depend on the last)
    eager = []
    for _ in range(3):
        _sequence(isp, t)
        torch.cuda.synchronize()
        eager.append(_snapshot(t))
    # restore, capture one step
    for k, v in initial.items():
        t[k].copy_(v)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    side = torch.cuda.Stream()
    with torch.cuda.stream(side):
        # warm-up on the capture stream (outside the capture), then restore the state
        _sequence(isp, t)
        for k, v in initial.items():
            t[k].copy_(v)
        side.synchronize()
        graph.capture_begin()
        _sequence(isp, t)      # ops.* launch on torch's current stream, which is the capturing one
        graph.capture_end()
    torch.cuda.synchronize()
    for k, v in initial.items():   # capture does not execute: the state is still the initial one
        assert torch.equal(t[k], v), k
    scratch = torch.zeros(1 << 20, device="cuda")
    for step in range(3):
        graph.replay()
        torch.cuda.synchronize()
        for k, v in eager[step].items():
            assert torch.equal(t[k], v), "replay %d differs from eager in %s" % (step, k)
        # unrelated eager work and a synchronisation between replays
        scratch.add_(1.0)
        isp.rmsnorm(torch.randn((4, 4096), device="cuda").half(), t["gamma"], 1e-5)
        torch.cuda.synchronize()


def test_capture_of_the_prefill_kernels(isp):
    """The prefill-side entry points under capture: the gather, the padding-offset builder, the LLaMA-shape
    QKV kernel (which reads its divisor table straight out of the kernel-argument block, so the block
    the graph node holds must serve it on every replay), transpose-out and the fused norm."""
    print("[case] graph capture of the prefill kernels", flush=True)
    g = torch.Generator(device="cuda").manual_seed(3)
    batch, seq, hn, hs, vocab, hidden = 4, 48, 32, 128, 500, 4096
    lens = torch.tensor([48, 17, 30, 5], dtype=torch.int32, device="cuda")
    tokens = int(lens.sum())
    t = {
        "ids": torch.randint(0, vocab, (tokens,), dtype=torch.int32, device="cuda", generator=g),
        "table": torch.randn((vocab, hidden), device="cuda", generator=g).half(),
        "emb": torch.zeros((tokens, hidden), dtype=torch.float16, device="cuda"),
        "po": torch.zeros((batch, seq), dtype=torch.int32, device="cuda"),
        "cum": torch.zeros((batch + 1,), dtype=torch.int32, device="cuda"),
        "hist": torch.tensor([0, 100, 7, 2000], dtype=torch.int32, device="cuda"),
        "qkv": torch.randn((tokens, 3 * hn, hs), device="cuda", generator=g).half(),
        "bias": (0.02 * torch.randn((3 * hn * hs,), device="cuda", generator=g)).half(),
        "q": torch.zeros((batch, hn, seq, hs), dtype=torch.float16, device="cuda"),
        "k": torch.zeros((batch, hn, seq, hs), dtype=torch.float16, device="cuda"),
        "v": torch.zeros((batch, hn, seq, hs), dtype=torch.float16, device="cuda"),
        "packed": torch.zeros((tokens, hn, hs), dtype=torch.float16, device="cuda"),
        "residual": torch.randn((tokens, hidden), device="cuda", generator=g).half(),
        "gamma": torch.rand((hidden,), device="cuda", generator=g).half(),
    }

    def sequence():
        isp.input_embedding(t["ids"], t["emb"], t["table"])
        isp.cal_padding_offset(t["po"], t["cum"], lens)
        isp.add_fused_qkv_bias_transpose_and_rope(t["q"], t["k"], t["v"], t["qkv"], t["bias"], t["po"], t["hist"],
                                                  lens, 128, 10000.0)
        isp.transpose_out_remove_padding(t["q"], t["po"], t["packed"])
        isp.fused_add_bias_residual_rmsnorm(t["residual"], t["emb"], None, t["gamma"], 1e-5)

    initial = _snapshot(t)
    eager = []
    for _ in range(2):
        sequence()
        torch.cuda.synchronize()
        eager.append(_snapshot(t))
    for k, v in initial.items():
        t[k].copy_(v)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    side = torch.cuda.Stream()
    with torch.cuda.stream(side):
        sequence()
        for k, v in initial.items():
            t[k].copy_(v)
        side.synchronize()
        graph.capture_begin()
        sequence()
        graph.capture_end()
    torch.cuda.synchronize()
    for step in range(2):
        graph.replay()
        torch.cuda.synchronize()
        for k, v in eager[step].items():
            assert torch.equal(t[k], v), "replay %d differs from eager in %s" % (step, k)
        # a launch of the same kernel with other arguments between the replays
        other = torch.zeros_like(t["q"])
        isp.add_fused_qkv_bias_transpose_and_rope(other, other.clone(), other.clone(), t["qkv"], None, t["po"],
                                                  t["hist"], lens, 128, 500000.0)
        torch.cuda.synchronize()


def test_capture_of_the_fused_entry_points(isp):
    """The fused forms under capture: the prefill step with the KV append (fp16 with 64-element heads, whose
    kernel reads its divisors out of the argument block, and fp32 through the general kernel, which does the
    same) and the decode step (bias + RoPE + append in one launch).  Each replay continues where the last one
    stopped: the decode step rotates its buffer in place, so three replays must equal three eager steps."""
    print("[case] graph capture of the fused entry points", flush=True)
    g = torch.Generator(device="cuda").manual_seed(5)
    batch, seq, max_seq = 3, 20, 64
    lens = torch.tensor([20, 7, 13], dtype=torch.int32, device="cuda")
    tokens = int(lens.sum())
    hist = torch.tensor([0, 30, 5], dtype=torch.int32, device="cuda")
    t = {"po": torch.zeros((batch, seq), dtype=torch.int32, device="cuda"),
         "cum": torch.zeros((batch + 1,), dtype=torch.int32, device="cuda")}
    shapes = {"h": (torch.float16, 16, 8, 64), "f": (torch.float32, 8, 2, 128)}
    for tag, (dt, hn, kvn, hs) in shapes.items():
        r = lambda *s: torch.randn(s, device="cuda", generator=g).to(dt)
        t.update({
            tag + "qkv": r(tokens, hn + 2 * kvn, hs), tag + "bias": r((hn + 2 * kvn) * hs) * 0.1,
            tag + "q": torch.zeros((batch, hn, seq, hs), dtype=dt, device="cuda"),
            tag + "kc": torch.zeros((2, batch, kvn, max_seq, hs), dtype=dt, device="cuda"),
            tag + "vc": torch.zeros((2, batch, kvn, max_seq, hs), dtype=dt, device="cuda"),
            tag + "step_qkv": r(batch, hn + 2 * kvn, hs),
        })

    ctx = hist + lens          # allocated before the capture: the sequence itself must not allocate

    def sequence():
        isp.cal_padding_offset(t["po"], t["cum"], lens)
        for tag, (dt, hn, kvn, hs) in shapes.items():
            isp.add_fused_qkv_bias_transpose_rope_and_append(t[tag + "q"], None, None, t[tag + "kc"], t[tag + "vc"], 1,
                                                             t[tag + "qkv"], t[tag + "bias"], t["po"], hist, lens, hs,
                                                             10000.0)
            isp.rope_decode_and_append(t[tag + "step_qkv"], t[tag + "bias"], t[tag + "kc"], t[tag + "vc"], 0, ctx,
                                       41, hn, hs, 10000.0)

    initial = _snapshot(t)
    eager = []
    for _ in range(3):
        sequence()
        torch.cuda.synchronize()
        eager.append(_snapshot(t))
    assert not torch.equal(eager[0]["hstep_qkv"], eager[1]["hstep_qkv"]), "the decode step must work in place"
    for k, v in initial.items():
        t[k].copy_(v)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    side = torch.cuda.Stream()
    with torch.cuda.stream(side):
        sequence()
        for k, v in initial.items():
            t[k].copy_(v)
        side.synchronize()
        graph.capture_begin()
        sequence()
        graph.capture_end()
    torch.cuda.synchronize()
    for step in range(3):
        graph.replay()
        torch.cuda.synchronize()
        for k, v in eager[step].items():
            assert torch.equal(t[k], v), "replay %d differs from eager in %s" % (step, k)
        # the same kernels with other arguments between the replays
        other = torch.zeros_like(t["hq"])
        isp.add_fused_qkv_bias_transpose_rope_and_append(other, None, None, torch.zeros_like(t["hkc"]),
                                                         torch.zeros_like(t["hvc"]), 0, t["hqkv"], None, t["po"], hist,
                                                         lens, 64, 500000.0)
        torch.cuda.synchronize()
