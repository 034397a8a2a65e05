"""Parity of the kernels either side of the fused QKV step -- decode-phase RoPE, transpose-out +
remove padding, KV-cache append and broadcast -- against the CPU oracle (bit-exact for the copies)."""
import numpy as np
import pytest
import torch

from helpers import (assert_f16_close, assert_f32_close, padding_offsets_np, reference_mover_configurations,
                     rope_pair_radius)

pytestmark = pytest.mark.gpu
NP2T = {np.float16: torch.float16, np.float32: torch.float32}


def dev(a):
    return None if a is None else torch.from_numpy(np.ascontiguousarray(a)).cuda()


def say(msg):
    print("[case] " + msg, flush=True)


@pytest.mark.parametrize("dtype", [np.float16, np.float32])
@pytest.mark.parametrize("batch,hn,kvn,hs,rot,step", [(1, 32, 32, 128, 128, 1), (1, 32, 32, 128, 128, 57),
                                                      (3, 8, 2, 128, 64, 700), (2, 4, 4, 64, 64, 13),
                                                      (2, 3, 1, 16, 16, 5), (1, 2, 2, 96, 32, 9)])
def test_rope_decode(isp, oracle, dtype, batch, hn, kvn, hs, rot, step):
    say("rope decode %s b=%d hn=%d kvn=%d hs=%d rot=%d step=%d" % (dtype.__name__, batch, hn, kvn, hs, rot, step))
    x = np.random.default_rng(step).standard_normal((batch, hn + 2 * kvn, hs), dtype=np.float32).astype(dtype)
    d = dev(x)
    isp.rope(d, step, hn, rot, 10000.0)
    got = d.cpu().numpy()
    exp = oracle.rope_decode(x, hn, kvn, step, rot, 10000.0)
    assert np.array_equal(got[:, hn + kvn:], x[:, hn + kvn:]), "v heads must stay untouched"
    rad = rope_pair_radius(x, None)[:, :hn + kvn]
    if dtype == np.float32:
        assert_f32_close(got[:, :hn + kvn], exp[:, :hn + kvn], "decode rope", scale=rad + 1e-30)
    else:
        assert_f16_close(got[:, :hn + kvn], exp[:, :hn + kvn], "decode rope", magnitude=rad)


def test_rope_decode_matches_prefill_kernel(isp):
    # one token at history = step - 1 through the prefill kernel gives the same q and k bits
    hn, kvn, hs, step = 32, 32, 128, 41
    x = dev(np.random.default_rng(41).standard_normal((1, hn + 2 * kvn, hs), dtype=np.float32).astype(np.float16))
    q, k, v = (torch.zeros((1, n, 1, hs), dtype=torch.float16, device="cuda") for n in (hn, kvn, kvn))
    z = torch.zeros(1, dtype=torch.int32, device="cuda")
    isp.add_fused_qkv_bias_transpose_and_rope(q, k, v, x.clone(), None, z, z + (step - 1), z + 1, 128, 10000.0)
    y = x.clone()
    isp.rope(y, step, hn, 128, 10000.0)
    assert torch.equal(y[0, :hn], q[0, :, 0]) and torch.equal(y[0, hn:hn + kvn], k[0, :, 0])


@pytest.mark.parametrize("dtype", [np.float16, np.float32])
@pytest.mark.parametrize("batch,heads,seq,hs", [(8, 32, 512, 128), (2, 2, 4, 2), (3, 5, 9, 24), (1, 1, 1, 8)])
def test_transpose_remove_padding(isp, oracle, dtype, batch, heads, seq, hs):
    say("transpose-remove-padding %s b=%d h=%d s=%d hs=%d" % (dtype.__name__, batch, heads, seq, hs))
    r = np.random.default_rng(batch * seq)
    lens = r.integers(max(1, seq // 2), seq + 1, batch, dtype=np.int32)
    po, _ = padding_offsets_np(lens, seq)
    tokens = int(lens.sum())
    src = r.standard_normal((batch, heads, seq, hs), dtype=np.float32).astype(dtype)
    out = torch.full((tokens, heads, hs), -5, dtype=NP2T[dtype], device="cuda")
    isp.transpose_out_remove_padding(dev(src), dev(po), out)
    assert np.array_equal(out.cpu().numpy(), oracle.transpose_remove_padding(src, po, tokens))


def test_transpose_remove_padding_known_answer_and_inverse(isp):
    # the reference's example: [2, 2, 4, 2] iota, offsets 0 0 2 2 2
    src = torch.arange(32, dtype=torch.float32, device="cuda").view(2, 2, 4, 2)
    po = torch.tensor([0, 0, 2, 2, 2], dtype=torch.int32, device="cuda")
    out = torch.empty((5, 2, 2), device="cuda")
    isp.transpose_out_remove_padding(src, po, out)
    assert out.cpu().tolist() == [[[0, 1], [8, 9]], [[2, 3], [10, 11]], [[16, 17], [24, 25]],
                                  [[18, 19], [26, 27]], [[20, 21], [28, 29]]]
    # inverse of the QKV scatter: v goes out padded and comes back packed
    batch, seq, hn, hs = 4, 64, 32, 128
    lens = np.array([64, 1, 33, 17], np.int32)
    po_np, _ = padding_offsets_np(lens, seq)
    tokens = int(lens.sum())
    qkv = dev(np.random.default_rng(7).standard_normal((tokens, 3 * hn, hs), dtype=np.float32).astype(np.float16))
    q, k, v = (torch.zeros((batch, hn, seq, hs), dtype=torch.float16, device="cuda") for _ in range(3))
    z = torch.zeros(batch, dtype=torch.int32, device="cuda")
    isp.add_fused_qkv_bias_transpose_and_rope(q, k, v, qkv, None, dev(po_np), z, dev(lens), 128, 10000.0)
    back = torch.empty((tokens, hn, hs), dtype=torch.float16, device="cuda")
    isp.transpose_out_remove_padding(v, dev(po_np), back)
    assert torch.equal(back, qkv[:, 2 * hn:])


@pytest.mark.parametrize("dtype", [np.float16, np.float32])
@pytest.mark.parametrize("layers,batch,kvn,hn,max_q,max_seq,hs", [(2, 8, 32, 32, 512, 1024, 128), (3, 2, 2, 6, 5, 16, 8),
                                                                   (1, 3, 1, 4, 7, 9, 20), (2, 1, 4, 4, 1, 64, 128)])
def test_kv_cache_movers(isp, oracle, dtype, layers, batch, kvn, hn, max_q, max_seq, hs):
    say("kv movers %s L=%d b=%d kvn=%d hn=%d q=%d S=%d hs=%d" % (dtype.__name__, layers, batch, kvn, hn, max_q, max_seq, hs))
    r = np.random.default_rng(max_seq)
    k_src = r.standard_normal((batch, kvn, max_q, hs), dtype=np.float32).astype(dtype)
    v_src = r.standard_normal((batch, kvn, max_q, hs), dtype=np.float32).astype(dtype)
    k_cache = r.standard_normal((layers, batch, kvn, max_seq, hs), dtype=np.float32).astype(dtype)
    v_cache = r.standard_normal((layers, batch, kvn, max_seq, hs), dtype=np.float32).astype(dtype)
    cur = r.integers(0, max_q + 1, batch, dtype=np.int32)
    hist = np.array([r.integers(0, max_seq - c + 1) for c in cur], np.int32)
    layer = layers - 1
    dk, dv = dev(k_cache), dev(v_cache)
    isp.concat_kv_cache(dev(k_src), dev(v_src), layer, dev(cur), dev(hist), dk, dv)
    ek = oracle.concat_kv(k_src, k_cache, layer, cur, hist)
    ev = oracle.concat_kv(v_src, v_cache, layer, cur, hist)
    assert np.array_equal(dk.cpu().numpy(), ek) and np.array_equal(dv.cpu().numpy(), ev)
    ctx = (hist + cur).astype(np.int32)
    max_k = int(max(1, ctx.max()))
    ok = torch.full((batch, hn, max_k, hs), -3, dtype=NP2T[dtype], device="cuda")
    ov = torch.full((batch, hn, max_k, hs), -3, dtype=NP2T[dtype], device="cuda")
    isp.repeat_kv_cache(dk, dv, dev(ctx), layer, ok, ov)
    assert np.array_equal(ok.cpu().numpy(), oracle.repeat_kv(ek, layer, ctx, hn, max_k, fill=-3.0))
    assert np.array_equal(ov.cpu().numpy(), oracle.repeat_kv(ev, layer, ctx, hn, max_k, fill=-3.0))


def test_kv_cache_append_skips_rows_past_the_cache_end(isp):
    k_src = torch.ones((1, 2, 4, 128), dtype=torch.float16, device="cuda")
    cache_k = torch.zeros((1, 1, 2, 6, 128), dtype=torch.float16, device="cuda")
    cache_v = torch.zeros_like(cache_k)
    cur = torch.tensor([4], dtype=torch.int32, device="cuda")
    hist = torch.tensor([4], dtype=torch.int32, device="cuda")  # rows 4..7, the cache holds 6
    isp.concat_kv_cache(k_src, k_src, 0, cur, hist, cache_k, cache_v)
    torch.cuda.synchronize()
    assert torch.all(cache_k[0, 0, :, 4:6] == 1) and torch.all(cache_k[0, 0, :, :4] == 0)


# ------------------------------------------------------------------ fallback copy widths (4, 2, 1 bytes)
@pytest.mark.parametrize("shift", [0, 4, 2, 1])
def test_fallback_copy_units_through_raw_pointers(isp, shift):
    """Rows that are not whole aligned 16-byte vectors are copied in the widest unit the addresses allow.
    `shift` moves every buffer off its 16-byte alignment by that many bytes (0: only the row size is odd),
    so the 4-, 2- and 1-byte kernels all run; the data are bytes, checked against numpy indexing."""
    from inferspore_amd import capi
    lib = capi.lib()
    st = torch.cuda.current_stream().cuda_stream
    rng = np.random.default_rng(90 + shift)

    def on_device(a):
        """Copies a byte array to the device at `shift` bytes past an aligned address."""
        buf = torch.zeros(a.size + 64, dtype=torch.uint8, device="cuda")
        view = buf[shift:shift + a.size]
        view.copy_(torch.from_numpy(a.reshape(-1)))
        assert view.data_ptr() % 16 == shift % 16
        return buf, view

    # gather: rows of 10 fp16 elements = 20 bytes (4-byte units at shift 0 and 4, 2 at 2, 1 at 1)
    tokens, vocab, hidden = 29, 17, 10
    table = rng.integers(0, 256, (vocab, hidden * 2), dtype=np.uint8)
    ids = rng.integers(0, vocab, tokens).astype(np.int32)
    _, d_table = on_device(table)
    _, d_out = on_device(np.zeros((tokens, hidden * 2), np.uint8))
    d_ids = torch.from_numpy(ids).cuda()
    say("gather through raw pointers, shift %d" % shift)
    capi.check(lib.isp_embedding_f16(d_ids.data_ptr(), d_out.data_ptr(), d_table.data_ptr(), tokens, hidden, vocab, st),
               "isp_embedding_f16")
    assert np.array_equal(d_out.cpu().numpy().reshape(tokens, hidden * 2), table[ids])

    # movers: head rows of 6 fp16 elements = 12 bytes
    batch, heads, seq, hs = 3, 2, 6, 6
    seg = hs * 2
    lens = np.array([6, 2, 4], np.int32)
    src = rng.integers(0, 256, (batch, heads, seq, seg), dtype=np.uint8)
    tokens = int(lens.sum())
    po = np.concatenate([np.full(n, b * seq - lens[:b].sum(), np.int32) for b, n in enumerate(lens)])
    _, d_src = on_device(src)
    _, d_dst = on_device(np.zeros((tokens, heads, seg), np.uint8))
    d_po = torch.from_numpy(po).cuda()
    say("transpose-out through raw pointers, shift %d" % shift)
    capi.check(lib.isp_transpose_remove_padding_f16(d_src.data_ptr(), d_po.data_ptr(), d_dst.data_ptr(), batch, heads,
                                                    seq, hs, tokens, st), "isp_transpose_remove_padding_f16")
    p = np.arange(tokens) + po
    exp = src[p // seq, :, p % seq, :]
    assert np.array_equal(d_dst.cpu().numpy().reshape(tokens, heads, seg), exp)

    max_seq = 9
    hist = np.array([1, 7, 0], np.int32)
    ksrc, vsrc = src, src[::-1].copy()
    kc0 = rng.integers(0, 256, (batch, heads, max_seq, seg), dtype=np.uint8)
    vc0 = rng.integers(0, 256, (batch, heads, max_seq, seg), dtype=np.uint8)
    _, d_ks = on_device(ksrc)
    _, d_vs = on_device(vsrc)
    _, d_kc = on_device(kc0)
    _, d_vc = on_device(vc0)
    d_lens, d_hist = torch.from_numpy(lens).cuda(), torch.from_numpy(hist).cuda()
    say("KV append through raw pointers, shift %d" % shift)
    capi.check(lib.isp_concat_kv_cache_f16(d_ks.data_ptr(), d_vs.data_ptr(), d_kc.data_ptr(), d_vc.data_ptr(), 0,
                                           d_lens.data_ptr(), d_hist.data_ptr(), batch, heads, seq, max_seq, hs, st),
               "isp_concat_kv_cache_f16")
    for got, s_, c0 in ((d_kc, ksrc, kc0), (d_vc, vsrc, vc0)):
        exp = c0.copy()
        for b in range(batch):
            n = min(int(lens[b]), max_seq - int(hist[b]))
            exp[b, :, hist[b]:hist[b] + n] = s_[b, :, :n]
        assert np.array_equal(got.cpu().numpy().reshape(exp.shape), exp)

    ctx = np.array([9, 3, 5], np.int32)
    max_k = 9
    _, d_kd = on_device(np.full((batch, heads, max_k, seg), 7, np.uint8))
    _, d_vd = on_device(np.full((batch, heads, max_k, seg), 7, np.uint8))
    d_ctx = torch.from_numpy(ctx).cuda()
    say("KV broadcast through raw pointers, shift %d" % shift)
    capi.check(lib.isp_repeat_kv_cache_f16(d_kc.data_ptr(), d_vc.data_ptr(), d_kd.data_ptr(), d_vd.data_ptr(), 0,
                                           d_ctx.data_ptr(), batch, heads, heads, max_seq, max_k, hs, st),
               "isp_repeat_kv_cache_f16")
    kc_now = d_kc.cpu().numpy().reshape(batch, heads, max_seq, seg)
    got = d_kd.cpu().numpy().reshape(batch, heads, max_k, seg)
    for b in range(batch):
        assert np.array_equal(got[b, :, :ctx[b]], kc_now[b, :, :ctx[b]])
        assert (got[b, :, ctx[b]:] == 7).all()


def test_kv_cache_movers_on_the_reference_configurations(isp):
    print("[case] kv movers on the reference programs' configurations", flush=True)
    k_src, cache, expect_cache, src_cache, expect_rep = reference_mover_configurations()
    d = lambda a: torch.from_numpy(a).cuda()
    i32 = lambda v: torch.tensor(v, dtype=torch.int32, device="cuda")
    kc, vc = d(cache.copy()), d(cache.copy())
    isp.concat_kv_cache(d(k_src), d(k_src.copy()), 0, i32([16]), i32([1]), kc, vc)
    assert np.array_equal(kc.cpu().numpy(), expect_cache) and np.array_equal(vc.cpu().numpy(), expect_cache)
    kd = torch.full((1, 2, 2, 2), -3.0, device="cuda")
    vd = kd.clone()
    isp.repeat_kv_cache(d(src_cache), d(src_cache.copy()), i32([2]), 0, kd, vd)
    assert np.array_equal(kd.cpu().numpy(), expect_rep) and np.array_equal(vd.cpu().numpy(), expect_rep)
