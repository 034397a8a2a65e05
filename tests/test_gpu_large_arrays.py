"""Arrays beyond 2^31 elements / 4 GiB: every kernel's index arithmetic must be 64-bit where it matters.

Each case runs the kernel once on a multi-gigabyte tensor generated on the device, then checks
  * the whole result on the device against an independent torch expression (exact for the byte movers,
    the residual sum and the v heads; a loose float tolerance for the rest), and
  * row windows at the start, around the 2^31-element boundary and at the very end against the CPU
    oracle, to the same bar as the small parity tests.
"""
import numpy as np
import pytest
import torch

from helpers import assert_f16_close

pytestmark = pytest.mark.gpu

F16 = torch.float16


def say(msg):
    print("[case] " + msg, flush=True)


def host(t):
    return t.cpu().numpy()


def windows(rows, row_elems, width=24):
    """Row ranges at the start, straddling element index 2^31 (= byte offset 2^32 in fp16) and at the end."""
    cross = (1 << 31) // row_elems
    assert cross + width < rows, "array does not reach 2^31 elements"
    return [(0, width), (cross - width // 2, cross + width // 2), (rows - width, rows)]


def normal_f16(*shape, scale=1.0):
    t = torch.empty(shape, dtype=F16, device="cuda")
    t.normal_(0.0, scale)
    return t


def test_swiglu_beyond_4gib(isp, oracle):
    tokens, inter = 100000, 11008
    say("swiglu %dx%d fp16 (input %.1f GiB)" % (tokens, inter, tokens * 2 * inter * 2 / 2 ** 30))
    x = normal_f16(tokens, 2, inter)
    out = torch.full((tokens, inter), -3.0, dtype=F16, device="cuda")
    isp.act(x, out)
    torch.cuda.synchronize()
    step = 20000
    for r0 in range(0, tokens, step):
        g, u = x[r0:r0 + step, 0].float(), x[r0:r0 + step, 1].float()
        ref = torch.nn.functional.silu(g) * u
        err = (out[r0:r0 + step].float() - ref).abs() / (ref.abs() + 1e-3)
        assert float(err.max()) < 2e-3, "rows %d..: worst relative error %g" % (r0, float(err.max()))
    for a, b in windows(tokens, 2 * inter):
        assert_f16_close(host(out[a:b]), oracle.swiglu(host(x[a:b])), "swiglu rows %d..%d" % (a, b))


def test_fused_norm_beyond_4gib(isp, oracle):
    tokens, hidden = 540000, 4096
    say("fused norm %dx%d fp16 (%.1f GiB per operand)" % (tokens, hidden, tokens * hidden * 2 / 2 ** 30))
    out = normal_f16(tokens, hidden)
    res = normal_f16(tokens, hidden)
    bias = normal_f16(hidden, scale=0.02)
    gamma = (0.5 + torch.rand(hidden, device="cuda")).to(F16)
    wins = windows(tokens, hidden)
    before = [(host(res[a:b]), host(out[a:b])) for a, b in wins]
    step = 60000
    expect_res = []  # the expected residual per chunk, taken before the in-place update
    for r0 in range(0, tokens, step):
        s = ((out[r0:r0 + step].float() + res[r0:r0 + step].float()) + bias.float()).to(F16)
        expect_res.append(s)
    isp.fused_add_bias_residual_rmsnorm(res, out, bias, gamma, 1e-5)
    torch.cuda.synchronize()
    for i, r0 in enumerate(range(0, tokens, step)):
        s = expect_res[i]
        assert torch.equal(res[r0:r0 + step], s), "residual rows %d.. differ from the once-rounded fp32 sum" % r0
        x32 = s.float()  # not the fp32 sum itself, so only a loose check here; the oracle windows are exact
        ref = x32 * torch.rsqrt((x32 * x32).mean(1, keepdim=True) + 1e-5) * gamma.float()
        err = (out[r0:r0 + step].float() - ref).abs()
        assert float(err.max()) < 0.05, "rows %d..: worst absolute error %g" % (r0, float(err.max()))
    del expect_res
    for (a, b), (r_in, o_in) in zip(wins, before):
        e_res, e_out = oracle.fused_norm(r_in, o_in, host(bias), host(gamma), 1e-5)
        assert np.array_equal(host(res[a:b]), e_res), "residual rows %d..%d" % (a, b)
        assert_f16_close(host(out[a:b]), e_out, "normalised rows %d..%d" % (a, b))


def test_embedding_beyond_4gib(isp, oracle):
    tokens, hidden, vocab = 540000, 4096, 5000
    say("embedding %d ids x %d fp16" % (tokens, hidden))
    table = normal_f16(vocab, hidden, scale=0.02)
    ids = torch.randint(0, vocab, (tokens,), dtype=torch.int32, device="cuda")
    out = torch.full((tokens, hidden), -3.0, dtype=F16, device="cuda")
    isp.input_embedding(ids, out, table)
    torch.cuda.synchronize()
    step = 90000
    for r0 in range(0, tokens, step):
        assert torch.equal(out[r0:r0 + step], table[ids[r0:r0 + step].long()]), "rows %d.." % r0
    a, b = tokens - 16, tokens
    assert np.array_equal(host(out[a:b]), oracle.embedding(host(ids[a:b]), host(table)))


def _padded_batch(lens, seq):
    lens_t = torch.tensor(lens, dtype=torch.int32, device="cuda")
    batch = len(lens)
    po = torch.zeros((batch, seq), dtype=torch.int32, device="cuda")
    cum = torch.zeros((batch + 1,), dtype=torch.int32, device="cuda")
    return lens_t, po, cum


def test_qkv_rope_beyond_4gib(isp, oracle):
    batch, seq, hn, kvn, hs = 2, 90000, 32, 32, 128
    lens = [90000, 88000]
    tokens = sum(lens)
    say("qkv+rope %d tokens x 96 heads x 128 fp16 (input %.1f GiB)" % (tokens, tokens * 96 * 128 * 2 / 2 ** 30))
    lens_t, po, cum = _padded_batch(lens, seq)
    isp.cal_padding_offset(po, cum, lens_t)
    hist = torch.tensor([0, 500], dtype=torch.int32, device="cuda")
    qkv = normal_f16(tokens, hn + 2 * kvn, hs)
    bias = normal_f16((hn + 2 * kvn) * hs, scale=0.02)
    q = torch.full((batch, hn, seq, hs), -7.0, dtype=F16, device="cuda")
    k = torch.full((batch, kvn, seq, hs), -7.0, dtype=F16, device="cuda")
    v = torch.full((batch, kvn, seq, hs), -7.0, dtype=F16, device="cuda")
    isp.add_fused_qkv_bias_transpose_and_rope(q, k, v, qkv, bias, po, hist, lens_t, 128, 10000.0)
    torch.cuda.synchronize()
    # v heads are a copy (+ bias, added in fp32 and rounded once): exact on the whole array
    vb = bias.view(hn + 2 * kvn, hs)[hn + kvn:].float()
    start = 0
    for b in range(batch):
        n = lens[b]
        exp = (qkv[start:start + n, hn + kvn:].float() + vb).to(F16)          # [n, kvn, hs]
        assert torch.equal(v[b, :, :n], exp.permute(1, 0, 2)), "v of sequence %d" % b
        assert bool((v[b, :, n:] == -7.0).all()) and bool((q[b, :, n:] == -7.0).all()), "padded slots were written"
        # rotation preserves the norm of every (d, d + 64) pair: whole-array check on q
        xq = qkv[start:start + n, :hn].float() + bias.view(hn + 2 * kvn, hs)[:hn].float()
        r_in = xq[..., :64] ** 2 + xq[..., 64:] ** 2                           # [n, hn, 64]
        qo = q[b, :, :n].float()
        r_out = (qo[..., :64] ** 2 + qo[..., 64:] ** 2).permute(1, 0, 2)
        assert float(((r_in - r_out).abs() / (r_in + 1e-2)).max()) < 2e-2, "pair norms of sequence %d" % b
        del xq, r_in, qo, r_out, exp
        start += n
    # windows against the oracle: a window of one sequence is a small problem with history = first position
    n = 24
    for b, s0 in ((0, 0), (0, lens[0] - n), (1, 0), (1, (1 << 31) // (96 * 128) - lens[0] - n // 2), (1, lens[1] - n)):
        t0 = (0 if b == 0 else lens[0]) + s0
        sub = host(qkv[t0:t0 + n])
        h0 = int(hist[b]) + s0
        eq, ek, ev = oracle.qkv_rope(sub, host(bias), np.zeros(n, np.int32), np.array([h0], np.int32),
                                     np.array([n], np.int32), 1, n, hn, kvn, 128, 10000.0)
        xs = sub.astype(np.float32) + host(bias).reshape(96, 128).astype(np.float32)
        rad = np.sqrt(xs[..., :64] ** 2 + xs[..., 64:] ** 2)                   # [n, 96, 64]
        rad = np.concatenate([rad, rad], axis=-1).transpose(1, 0, 2)           # [96, n, 128]
        what = "sequence %d positions %d..%d" % (b, s0, s0 + n)
        assert_f16_close(host(q[b, :, s0:s0 + n]), eq[0], "q " + what, magnitude=rad[:hn])
        assert_f16_close(host(k[b, :, s0:s0 + n]), ek[0], "k " + what, magnitude=rad[hn:hn + kvn])
        assert np.array_equal(host(v[b, :, s0:s0 + n]), ev[0]), "v " + what


def test_kv_movers_beyond_4gib(isp, oracle):
    batch, heads, hs = 4, 32, 128
    max_seq, max_q = 140000, 70000
    say("KV cache [1, %d, %d, %d, %d] fp16 (%.1f GiB each)" % (batch, heads, max_seq, hs,
                                                              batch * heads * max_seq * hs * 2 / 2 ** 30))
    cur = [70000, 69999, 1, 65000]
    hist = [70000, 1, 139999, 70000]
    cur_t = torch.tensor(cur, dtype=torch.int32, device="cuda")
    hist_t = torch.tensor(hist, dtype=torch.int32, device="cuda")
    k_src, v_src = normal_f16(batch, heads, max_q, hs), normal_f16(batch, heads, max_q, hs)
    k_cache = torch.full((1, batch, heads, max_seq, hs), -5.0, dtype=F16, device="cuda")
    v_cache = torch.full((1, batch, heads, max_seq, hs), -5.0, dtype=F16, device="cuda")
    isp.concat_kv_cache(k_src, v_src, 0, cur_t, hist_t, k_cache, v_cache)
    torch.cuda.synchronize()
    for src, cache in ((k_src, k_cache), (v_src, v_cache)):
        for b in range(batch):
            h0, n = hist[b], cur[b]
            assert torch.equal(cache[0, b, :, h0:h0 + n], src[b, :, :n]), "appended rows of sequence %d" % b
            assert bool((cache[0, b, :, :h0] == -5.0).all()) and bool((cache[0, b, :, h0 + n:] == -5.0).all())

    say("broadcast out of the same cache")
    ctx = [140000, 70000, 140000, 135000]
    ctx_t = torch.tensor(ctx, dtype=torch.int32, device="cuda")
    k_all = torch.full((batch, heads, max_seq, hs), -9.0, dtype=F16, device="cuda")
    v_all = torch.full((batch, heads, max_seq, hs), -9.0, dtype=F16, device="cuda")
    isp.repeat_kv_cache(k_cache, v_cache, ctx_t, 0, k_all, v_all)
    torch.cuda.synchronize()
    for cache, dst in ((k_cache, k_all), (v_cache, v_all)):
        for b in range(batch):
            assert torch.equal(dst[b, :, :ctx[b]], cache[0, b, :, :ctx[b]]), "sequence %d" % b
            assert bool((dst[b, :, ctx[b]:] == -9.0).all()), "rows past the context were written"
    del k_all, v_all, k_src, v_src

    say("transpose-out + remove padding of the same array")
    src = k_cache[0]                                    # [batch, heads, max_seq, hs], 4.3 GiB
    lens = [140000, 139000, 1, 138000]
    tokens = sum(lens)
    lens_t, po, cum = _padded_batch(lens, max_seq)
    isp.cal_padding_offset(po, cum, lens_t)
    dst = torch.full((tokens, heads, hs), -1.0, dtype=F16, device="cuda")
    isp.transpose_out_remove_padding(src, po, dst)
    torch.cuda.synchronize()
    start = 0
    for b in range(batch):
        n = lens[b]
        assert torch.equal(dst[start:start + n], src[b, :, :n].permute(1, 0, 2)), "sequence %d" % b
        start += n
    # last tokens against the oracle on a window of the last sequence
    n = 8
    win = host(src[3:4, :, lens[3] - n:lens[3]])        # [1, heads, n, hs]
    exp = oracle.transpose_remove_padding(win, np.zeros(n, np.int32), n)
    assert np.array_equal(host(dst[tokens - n:]), exp)
