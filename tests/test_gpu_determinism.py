"""Every kernel, launched repeatedly on the same inputs at its benchmark shape, must give the same bits
every time.  Summation order is fixed by design, so any difference is a defect; the check also catches
corruption that shows only once in millions of elements (for example a hardware hazard between two
stores that only bites when register allocation lines up), which a single parity run can miss."""
import pytest
import torch

pytestmark = pytest.mark.gpu

REPEATS = 40


def say(msg):
    print("[case] " + msg, flush=True)


def _padded_batch(isp, batch, seq, seed):
    g = torch.Generator(device="cpu").manual_seed(seed)
    lens = torch.randint(seq // 2, seq + 1, (batch,), generator=g, dtype=torch.int32)
    lens_d = lens.cuda()
    po = torch.zeros((batch, seq), dtype=torch.int32, device="cuda")
    cum = torch.zeros((batch + 1,), dtype=torch.int32, device="cuda")
    isp.cal_padding_offset(po, cum, lens_d)
    return lens_d, po, int(lens.sum())


def _same_every_time(run, what):
    first = run()
    torch.cuda.synchronize()
    for i in range(REPEATS):
        again = run()
        for a, b in zip(first, again):
            assert torch.equal(a, b), "%s: launch %d differs from the first" % (what, i + 1)


@pytest.mark.parametrize("dtype", [torch.float16, torch.float32])
def test_qkv_rope_repeats(isp, dtype):
    for hn, kvn, with_bias in ((32, 32, True), (32, 32, False), (32, 8, True), (40, 40, True)):
        say("qkv %s %dq/%dkv bias=%s x%d" % (dtype, hn, kvn, with_bias, REPEATS))
        batch, seq, hs = 8, 512, 128
        lens_d, po, tokens = _padded_batch(isp, batch, seq, seed=hn + kvn)
        hist = torch.arange(batch, dtype=torch.int32, device="cuda") * 7
        qkv = torch.randn((tokens, hn + 2 * kvn, hs), device="cuda").to(dtype)
        bias = (0.02 * torch.randn((hn + 2 * kvn) * hs, device="cuda")).to(dtype) if with_bias else None

        def run():
            q = torch.full((batch, hn, seq, hs), -5.0, dtype=dtype, device="cuda")
            k = torch.full((batch, kvn, seq, hs), -5.0, dtype=dtype, device="cuda")
            v = torch.full((batch, kvn, seq, hs), -5.0, dtype=dtype, device="cuda")
            isp.add_fused_qkv_bias_transpose_and_rope(q, k, v, qkv, bias, po, hist, lens_d, 128, 10000.0)
            return q, k, v

        _same_every_time(run, "qkv")


@pytest.mark.parametrize("dtype", [torch.float16, torch.float32])
def test_norm_swiglu_embedding_repeats(isp, dtype):
    tokens, hidden, inter, vocab = 2048, 4096, 11008, 32000
    out0 = torch.randn((tokens, hidden), device="cuda").to(dtype)
    res0 = torch.randn((tokens, hidden), device="cuda").to(dtype)
    bias = (0.02 * torch.randn(hidden, device="cuda")).to(dtype)
    gamma = (0.5 + torch.rand(hidden, device="cuda")).to(dtype)

    def run_norm():
        out, res = out0.clone(), res0.clone()
        isp.fused_add_bias_residual_rmsnorm(res, out, bias, gamma, 1e-5)
        return out, res

    say("fused norm %s x%d" % (dtype, REPEATS))
    _same_every_time(run_norm, "fused norm")

    x = torch.randn((tokens, 2, inter), device="cuda").to(dtype)

    def run_act():
        out = torch.empty((tokens, inter), dtype=dtype, device="cuda")
        isp.act(x, out)
        return (out,)

    say("swiglu %s x%d" % (dtype, REPEATS))
    _same_every_time(run_act, "swiglu")

    table = (0.02 * torch.randn((vocab, hidden), device="cuda")).to(dtype)
    ids = torch.randint(0, vocab, (8192,), dtype=torch.int32, device="cuda")

    def run_embed():
        out = torch.empty((8192, hidden), dtype=dtype, device="cuda")
        isp.input_embedding(ids, out, table)
        return (out,)

    say("embedding %s x%d" % (dtype, REPEATS))
    _same_every_time(run_embed, "embedding")
    assert torch.equal(run_embed()[0], table[ids.long()])


def test_movers_repeat(isp):
    dtype = torch.float16
    batch, seq, heads, hs, max_seq = 8, 512, 32, 128, 1024
    lens_d, po, tokens = _padded_batch(isp, batch, seq, seed=5)
    hist = torch.arange(batch, dtype=torch.int32, device="cuda") * 3
    ctx = lens_d + hist
    k_src = torch.randn((batch, heads, seq, hs), device="cuda").to(dtype)
    v_src = torch.randn((batch, heads, seq, hs), device="cuda").to(dtype)

    def run():
        kc = torch.zeros((1, batch, heads, max_seq, hs), dtype=dtype, device="cuda")
        vc = torch.zeros((1, batch, heads, max_seq, hs), dtype=dtype, device="cuda")
        isp.concat_kv_cache(k_src, v_src, 0, lens_d, hist, kc, vc)
        k_all = torch.zeros((batch, heads, int(ctx.max()), hs), dtype=dtype, device="cuda")
        v_all = torch.zeros_like(k_all)
        isp.repeat_kv_cache(kc, vc, ctx, 0, k_all, v_all)
        packed = torch.zeros((tokens, heads, hs), dtype=dtype, device="cuda")
        isp.transpose_out_remove_padding(k_src, po, packed)
        return kc, vc, k_all, v_all, packed

    say("KV append, broadcast, transpose-out x%d" % REPEATS)
    _same_every_time(run, "movers")
