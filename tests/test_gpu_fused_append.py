"""The fused forms against what they fuse: QKV bias + RoPE + transpose with the KV-cache append in one
launch, and the decode step's bias + RoPE + append in one launch.  Each must reproduce, bit for bit,
the launches it replaces (which the other GPU tests pin against the oracle), and is also compared
with the oracle's own composition (bit-exact for v and for every index, stated tolerance for the
rotated rows)."""
import numpy as np
import pytest
import torch

from helpers import assert_f16_close, assert_f32_close, qkv_inputs, rope_pair_radius

pytestmark = pytest.mark.gpu
NP2T = {np.float16: torch.float16, np.float32: torch.float32}
SENTINEL = -55.0


def dev(a):
    return None if a is None else torch.from_numpy(np.ascontiguousarray(a)).cuda()


def say(msg):
    print("[case] " + msg, flush=True)


def _run_pair(isp, dtype, batch, seq, hn, kvn, hs, rot, max_seq, layers, layer, hist, with_bias, seed, keep_kv):
    lens, qkv, bias, po, _ = qkv_inputs(batch, seq, hn, kvn, hs, dtype, seed=seed, min_len=0, with_bias=with_bias)
    hist = np.asarray(hist, np.int32)
    td = NP2T[dtype]
    tokens = qkv.shape[0]
    po_dev = torch.zeros((batch, seq), dtype=torch.int32, device="cuda")
    po_dev.view(-1)[:tokens] = dev(po)
    d_qkv, d_bias, d_hist, d_lens = dev(qkv), dev(bias), dev(hist), dev(lens)
    full = lambda *shape: torch.full(shape, SENTINEL, dtype=td, device="cuda")
    # two launches
    q1, k1, v1 = full(batch, hn, seq, hs), full(batch, kvn, seq, hs), full(batch, kvn, seq, hs)
    kc1, vc1 = full(layers, batch, kvn, max_seq, hs), full(layers, batch, kvn, max_seq, hs)
    isp.add_fused_qkv_bias_transpose_and_rope(q1, k1, v1, d_qkv, d_bias, po_dev, d_hist, d_lens, rot, 10000.0)
    isp.concat_kv_cache(k1, v1, layer, d_lens, d_hist, kc1, vc1)
    # one launch
    q2 = full(batch, hn, seq, hs)
    k2, v2 = (full(batch, kvn, seq, hs), full(batch, kvn, seq, hs)) if keep_kv else (None, None)
    kc2, vc2 = full(layers, batch, kvn, max_seq, hs), full(layers, batch, kvn, max_seq, hs)
    isp.add_fused_qkv_bias_transpose_rope_and_append(q2, k2, v2, kc2, vc2, layer, d_qkv, d_bias, po_dev, d_hist,
                                                     d_lens, rot, 10000.0)
    torch.cuda.synchronize()
    assert torch.equal(q1, q2), "q differs from the unfused launch"
    if keep_kv:
        assert torch.equal(k1, k2) and torch.equal(v1, v2), "padded k / v differ from the unfused launch"
    assert torch.equal(kc1, kc2) and torch.equal(vc1, vc2), "cache differs from the two-launch result"
    return lens, qkv, bias, po, hist, kc2.cpu().numpy(), vc2.cpu().numpy()


@pytest.mark.parametrize("dtype", [np.float16, np.float32])
@pytest.mark.parametrize("keep_kv", [True, False])
@pytest.mark.parametrize("batch,seq,hn,kvn,hs,rot,max_seq", [
    (8, 512, 32, 32, 128, 128, 1024),   # the benchmark configuration: the one-vector-per-lane kernel in fp16
    (3, 12, 64, 32, 128, 128, 40),      # same kernel, two q groups
    (2, 9, 8, 2, 128, 128, 16),         # GQA: every wave places its own heads
    (2, 9, 6, 3, 128, 128, 16),         # head counts that fit no vector layout of whole waves: the general kernel
    (2, 9, 5, 1, 128, 64, 16),          # MQA, partial rotary
    (3, 7, 4, 2, 64, 64, 12),           # 64-element heads
    (3, 7, 16, 8, 64, 64, 12),          # 64-element heads in groups of 8: two tokens per workgroup in fp16
    (2, 6, 3, 3, 16, 16, 9),            # scalar kernel
    (2, 6, 2, 1, 96, 32, 6),            # scalar kernel, partial rotary, cache too short for the longest row
])
def test_qkv_append_equals_two_launches_and_the_oracle(isp, oracle, dtype, keep_kv, batch, seq, hn, kvn, hs, rot,
                                                      max_seq):
    say("qkv+append %s keep_kv=%s b=%d s=%d hn=%d kvn=%d hs=%d rot=%d S=%d" % (
        dtype.__name__, keep_kv, batch, seq, hn, kvn, hs, rot, max_seq))
    layers, layer = 2, 1
    hist = [(3 * b) % max(1, max_seq - seq + 2) for b in range(batch)] if max_seq > seq else list(range(batch))
    for with_bias in (True, False):
        lens, qkv, bias, po, hist_a, kc, vc = _run_pair(isp, dtype, batch, seq, hn, kvn, hs, rot, max_seq, layers,
                                                         layer, hist, with_bias, seed=hs + batch, keep_kv=keep_kv)
        # the oracle's composition: qkv step, then append
        ek_pad, ev_pad = oracle.qkv_rope(qkv, bias, po, hist_a, lens, batch, seq, hn, kvn, rot, 10000.0,
                                         fill=SENTINEL)[1:]
        assert np.all(kc[0] == SENTINEL) and np.all(vc[0] == SENTINEL), "the other layer must stay untouched"
        written = np.zeros((batch, max_seq), bool)
        rad = rope_pair_radius(qkv, bias)
        starts = np.concatenate([[0], np.cumsum(lens)[:-1]])
        for b in range(batch):
            for s in range(int(lens[b])):
                row = int(hist_a[b]) + s
                if row >= max_seq:
                    continue
                written[b, row] = True
                assert np.array_equal(vc[layer, b, :, row], ev_pad[b, :, s]), "v rows are copies: bit-exact"
                mag = rad[starts[b] + s, hn:hn + kvn]
                if dtype == np.float32:
                    assert_f32_close(kc[layer, b, :, row], ek_pad[b, :, s], "appended k", scale=mag + 1e-30)
                else:
                    assert_f16_close(kc[layer, b, :, row], ek_pad[b, :, s], "appended k", magnitude=mag,
                                     max_mismatch_fraction=0.2)
        untouched = ~np.broadcast_to(written[:, None, :, None], kc[layer].shape)
        assert np.all(kc[layer][untouched] == SENTINEL) and np.all(vc[layer][untouched] == SENTINEL)


def test_qkv_append_respects_input_length(isp):
    """A token whose position is not below input_length[b] is scattered but not appended, exactly as the
    two launches behave when the lengths and the padding offsets disagree."""
    hn = kvn = 32
    hs, seq, max_seq = 128, 8, 16
    qkv = torch.randn((8, 96, hs), device="cuda").half()
    z = torch.zeros(8, dtype=torch.int32, device="cuda")
    lens = torch.tensor([5], dtype=torch.int32, device="cuda")     # shorter than the 8 packed tokens
    hist = torch.tensor([2], dtype=torch.int32, device="cuda")
    q = torch.zeros((1, hn, seq, hs), dtype=torch.float16, device="cuda")
    kc = torch.full((1, 1, kvn, max_seq, hs), SENTINEL, dtype=torch.float16, device="cuda")
    vc = kc.clone()
    isp.add_fused_qkv_bias_transpose_rope_and_append(q, None, None, kc, vc, 0, qkv, None, z, hist, lens, 128, 10000.0)
    assert torch.all(kc[0, 0, :, 7:] == SENTINEL) and torch.all(kc[0, 0, :, :2] == SENTINEL)
    assert torch.equal(vc[0, 0, :, 2:7], qkv[:5, 64:].permute(1, 0, 2))


@pytest.mark.parametrize("dtype", [np.float16, np.float32])
@pytest.mark.parametrize("batch,hn,kvn,hs,rot,step,max_seq", [
    (1, 32, 32, 128, 128, 57, 128), (16, 32, 32, 128, 128, 101, 256), (3, 8, 2, 128, 64, 700, 1024),
    (2, 4, 4, 64, 64, 13, 16), (2, 3, 1, 16, 16, 5, 8), (1, 2, 2, 96, 32, 9, 9)])
def test_decode_step_equals_rope_then_append(isp, oracle, dtype, batch, hn, kvn, hs, rot, step, max_seq):
    say("decode step %s b=%d hn=%d kvn=%d hs=%d rot=%d step=%d" % (dtype.__name__, batch, hn, kvn, hs, rot, step))
    r = np.random.default_rng(step)
    td = NP2T[dtype]
    x = r.standard_normal((batch, hn + 2 * kvn, hs), dtype=np.float32).astype(dtype)
    hist_np = np.array([min(step - 1, max_seq - 1) - (b % 2) for b in range(batch)], np.int32)
    hist_np[-1] = max_seq + 3 if batch > 1 else hist_np[-1]       # one sequence whose row falls outside
    hist = dev(hist_np)
    ones = torch.ones(batch, dtype=torch.int32, device="cuda")
    full = lambda *shape: torch.full(shape, SENTINEL, dtype=td, device="cuda")
    # three launches: rope in place, split k / v rows out of the packed buffer, append
    a = dev(x)
    isp.rope(a, step, hn, rot, 10000.0)
    k_src = a[:, hn:hn + kvn].reshape(batch, kvn, 1, hs).contiguous()
    v_src = a[:, hn + kvn:].reshape(batch, kvn, 1, hs).contiguous()
    kc1, vc1 = full(2, batch, kvn, max_seq, hs), full(2, batch, kvn, max_seq, hs)
    isp.concat_kv_cache(k_src, v_src, 1, ones, hist, kc1, vc1)
    # one launch
    b_ = dev(x)
    kc2, vc2 = full(2, batch, kvn, max_seq, hs), full(2, batch, kvn, max_seq, hs)
    isp.rope_decode_and_append(b_, None, kc2, vc2, 1, hist, step, hn, rot, 10000.0)
    torch.cuda.synchronize()
    assert torch.equal(a, b_) and torch.equal(kc1, kc2) and torch.equal(vc1, vc2)
    # and the oracle: rotation within tolerance, v and the indices exact
    exp = oracle.rope_decode(x, hn, kvn, step, rot, 10000.0)
    got = b_.cpu().numpy()
    rad = rope_pair_radius(x, None)[:, :hn + kvn]
    if dtype == np.float32:
        assert_f32_close(got[:, :hn + kvn], exp[:, :hn + kvn], "decode rope", scale=rad + 1e-30)
    else:
        assert_f16_close(got[:, :hn + kvn], exp[:, :hn + kvn], "decode rope", magnitude=rad)
    vc = vc2.cpu().numpy()
    for b in range(batch):
        if 0 <= hist_np[b] < max_seq:
            assert np.array_equal(vc[1, b, :, hist_np[b]], x[b, hn + kvn:])
            vc[1, b, :, hist_np[b]] = SENTINEL
    assert np.all(vc == SENTINEL), "no other cache row may be written"


@pytest.mark.parametrize("dtype", [np.float16, np.float32])
@pytest.mark.parametrize("hn,kvn,hs,rot", [(32, 32, 128, 128), (8, 2, 128, 64), (4, 4, 64, 64), (3, 1, 16, 16)])
def test_decode_step_with_bias_equals_the_prefill_kernel(isp, oracle, dtype, hn, kvn, hs, rot):
    """With a bias the decode step is the prefill step of one-token sequences at history = step - 1: same bits
    as that kernel, and the oracle's prefill function within the stated tolerance."""
    batch, step, max_seq = 5, 77, 128
    r = np.random.default_rng(hs + hn)
    td = NP2T[dtype]
    x = r.standard_normal((batch, hn + 2 * kvn, hs), dtype=np.float32).astype(dtype)
    bias = (0.02 * r.standard_normal((hn + 2 * kvn) * hs)).astype(dtype)
    hist = torch.full((batch,), step - 1, dtype=torch.int32, device="cuda")
    ones = torch.ones(batch, dtype=torch.int32, device="cuda")
    zeros = torch.zeros(batch, dtype=torch.int32, device="cuda")
    q, k, v = (torch.zeros((batch, n, 1, hs), dtype=td, device="cuda") for n in (hn, kvn, kvn))
    isp.add_fused_qkv_bias_transpose_and_rope(q, k, v, dev(x), dev(bias), zeros, hist, ones, rot, 10000.0)
    y = dev(x)
    kc = torch.full((1, batch, kvn, max_seq, hs), SENTINEL, dtype=td, device="cuda")
    vc = kc.clone()
    isp.rope_decode_and_append(y, dev(bias), kc, vc, 0, hist, step, hn, rot, 10000.0)
    torch.cuda.synchronize()
    assert torch.equal(y[:, :hn], q[:, :, 0]) and torch.equal(y[:, hn:hn + kvn], k[:, :, 0])
    assert torch.equal(y[:, hn + kvn:], v[:, :, 0])
    assert torch.equal(kc[0, :, :, step - 1], k[:, :, 0]) and torch.equal(vc[0, :, :, step - 1], v[:, :, 0])
    eq, ek, ev = oracle.qkv_rope(x, bias, np.zeros(batch, np.int32), np.full(batch, step - 1, np.int32),
                                 np.ones(batch, np.int32), batch, 1, hn, kvn, rot, 10000.0)
    assert np.array_equal(v.cpu().numpy(), ev)
    rad = rope_pair_radius(x, bias)
    for got, exp, sl in ((q, eq, slice(0, hn)), (k, ek, slice(hn, hn + kvn))):
        if dtype == np.float32:
            assert_f32_close(got.cpu().numpy()[:, :, 0], exp[:, :, 0], "decode with bias", scale=rad[:, sl] + 1e-30)
        else:
            assert_f16_close(got.cpu().numpy()[:, :, 0], exp[:, :, 0], "decode with bias", magnitude=rad[:, sl])


@pytest.mark.parametrize("dtype", [np.float16, np.float32])
@pytest.mark.parametrize("hn,kvn,hs,rot,with_bias", [(32, 32, 128, 128, False), (8, 2, 128, 64, True), (4, 4, 64, 64, True),
                                                     (3, 1, 16, 16, False)])
def test_decode_step_with_ragged_histories_rotates_each_sequence_at_its_own_position(isp, dtype, hn, kvn, hs, rot, with_bias):
    """step = 0: sequence b is rotated at history_length[b], where its row is appended -- the prefill kernel on
    one-token sequences with those histories, bit for bit.  (With one step for the whole batch the rotation and the
    cache row only agree where history_length[b] == step - 1.)"""
    say("ragged decode step %s hn=%d kvn=%d hs=%d rot=%d bias=%s" % (dtype.__name__, hn, kvn, hs, rot, with_bias))
    batch, max_seq = 6, 256
    r = np.random.default_rng(hs * 3 + hn)
    td = NP2T[dtype]
    x = r.standard_normal((batch, hn + 2 * kvn, hs), dtype=np.float32).astype(dtype)
    bias = (0.02 * r.standard_normal((hn + 2 * kvn) * hs)).astype(dtype) if with_bias else None
    hist = torch.tensor([0, 5, 200, 17, 255, 63], dtype=torch.int32, device="cuda")
    ones = torch.ones(batch, dtype=torch.int32, device="cuda")
    zeros = torch.zeros(batch, dtype=torch.int32, device="cuda")
    q = torch.zeros((batch, hn, 1, hs), dtype=td, device="cuda")
    kc1 = torch.full((1, batch, kvn, max_seq, hs), SENTINEL, dtype=td, device="cuda")
    vc1 = kc1.clone()
    isp.add_fused_qkv_bias_transpose_rope_and_append(q, None, None, kc1, vc1, 0, dev(x), dev(bias), zeros, hist, ones, rot,
                                                     10000.0)
    y = dev(x)
    kc2, vc2 = torch.full_like(kc1, SENTINEL), torch.full_like(kc1, SENTINEL)
    isp.rope_decode_and_append(y, dev(bias), kc2, vc2, 0, hist, 0, hn, rot, 10000.0)
    torch.cuda.synchronize()
    assert torch.equal(y[:, :hn], q[:, :, 0])
    assert torch.equal(kc1, kc2) and torch.equal(vc1, vc2)
    for b, h in enumerate(hist.tolist()):
        assert torch.equal(y[b, hn:hn + kvn], kc2[0, b, :, h])
    # one step for everybody is a different operation on this batch: it must not give the same rows
    y1 = dev(x)
    kc3, vc3 = torch.full_like(kc1, SENTINEL), torch.full_like(kc1, SENTINEL)
    isp.rope_decode_and_append(y1, dev(bias), kc3, vc3, 0, hist, 6, hn, rot, 10000.0)
    torch.cuda.synchronize()
    assert torch.equal(y1[1], y[1]) and not torch.equal(y1[2, :hn + kvn], y[2, :hn + kvn])
    # the plain decode RoPE has no per-sequence positions: step 0 is rejected there
    with pytest.raises(RuntimeError):
        isp.rope(dev(x), 0, hn, rot, 10000.0)
