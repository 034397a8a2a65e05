"""Seeded sweep over random shapes, alignments and operand combinations: every kernel against the
oracle on configurations nobody hand-picked (odd extents, unaligned bases, empty sequences, GQA ratios),
plus re-entrancy of the C ABI from several host threads on their own streams."""
import threading

import numpy as np
import pytest
import torch

from helpers import (assert_f16_close, assert_f32_close, embedding_inputs, norm_inputs, padding_offsets_np,
                     rope_pair_radius, swiglu_inputs)

pytestmark = pytest.mark.gpu
NP2T = {np.float16: torch.float16, np.float32: torch.float32}


def dev(a, offset_elems=0):
    """Upload; with offset_elems the tensor starts that many elements into a larger buffer (misaligned)."""
    if a is None:
        return None
    a = np.ascontiguousarray(a)
    if offset_elems == 0:
        return torch.from_numpy(a).cuda()
    big = torch.zeros(a.size + offset_elems + 8, dtype=NP2T.get(a.dtype.type, torch.int32), device="cuda")
    view = big[offset_elems:offset_elems + a.size].view(a.shape)
    view.copy_(torch.from_numpy(a))
    return view


def test_random_norm_shapes(isp, oracle):
    r = np.random.default_rng(101)
    for case in range(40):
        dtype = [np.float16, np.float32][case % 2]
        tokens = int(r.integers(1, 70))
        hidden = int(r.choice([int(r.integers(1, 300)), 8 * int(r.integers(1, 1200)), 4096, 5120]))
        with_res, with_bias = bool(r.integers(2)), bool(r.integers(2))
        flags = int(r.integers(2))
        off = int(r.choice([0, 0, 1, 3]))
        print("[case] norm #%d %s %dx%d res=%d bias=%d flags=%d off=%d" % (case, dtype.__name__, tokens, hidden,
                                                                          with_res, with_bias, flags, off), flush=True)
        res, out, bias, gamma = norm_inputs(tokens, hidden, dtype, seed=1000 + case, with_residual=with_res,
                                            with_bias=with_bias)
        d_res, d_out = dev(res, off), dev(out, off)
        isp.fused_add_bias_residual_rmsnorm(d_res, d_out, dev(bias), dev(gamma), 1e-5, flags=flags)
        e_res, e_out = oracle.fused_norm(res, out, bias, gamma, 1e-5, flags=flags)
        got = d_out.cpu().numpy()
        if dtype == np.float32:
            assert_f32_close(got, e_out, "norm")
        else:
            assert_f16_close(got, e_out, "norm", max_mismatch_fraction=0.05)
        if with_res:
            assert np.array_equal(d_res.cpu().numpy(), e_res)


def test_random_swiglu_and_embedding_shapes(isp, oracle):
    r = np.random.default_rng(102)
    for case in range(30):
        dtype = [np.float16, np.float32][case % 2]
        tokens = int(r.integers(1, 50))
        inter = int(r.choice([int(r.integers(1, 200)), 8 * int(r.integers(1, 1500))]))
        off = int(r.choice([0, 0, 1]))
        print("[case] swiglu #%d %s %dx%d off=%d" % (case, dtype.__name__, tokens, inter, off), flush=True)
        x = swiglu_inputs(tokens, inter, dtype, seed=2000 + case) * dtype(2)
        out = torch.zeros((tokens, inter), dtype=NP2T[dtype], device="cuda")
        isp.act(dev(x, off), out)
        e = oracle.swiglu(x)
        if dtype == np.float32:
            assert_f32_close(out.cpu().numpy(), e, "swiglu", scale=np.abs(e) + 1e-2 * np.abs(x[:, 1]))
        else:
            assert_f16_close(out.cpu().numpy(), e, "swiglu", max_mismatch_fraction=0.05)
        hidden = int(r.choice([int(r.integers(1, 100)), 8 * int(r.integers(1, 700))]))
        vocab = int(r.integers(1, 500))
        ids, table = embedding_inputs(tokens, hidden, vocab, dtype, seed=3000 + case)
        out = torch.zeros((tokens, hidden), dtype=NP2T[dtype], device="cuda")
        isp.input_embedding(dev(ids), out, dev(table, off))
        assert np.array_equal(out.cpu().numpy(), oracle.embedding(ids, table))


def test_random_qkv_and_neighbour_shapes(isp, oracle):
    r = np.random.default_rng(103)
    for case in range(30):
        dtype = [np.float16, np.float32][case % 2]
        batch, seq = int(r.integers(1, 5)), int(r.integers(1, 40))
        kvn = int(r.choice([1, 2, 3, 8]))
        hn = kvn * int(r.choice([1, 2, 4]))
        hs = int(r.choice([128, 128, 64, 32, 6]))
        rot = int(r.choice([hs, hs, hs // 2 if (hs // 2) % 2 == 0 else hs]))
        lens = r.integers(0, seq + 1, batch).astype(np.int32)
        hist = r.integers(0, 50, batch).astype(np.int32)
        tokens = int(lens.sum())
        print("[case] qkv #%d %s b=%d s=%d hn=%d kvn=%d hs=%d rot=%d tokens=%d" % (case, dtype.__name__, batch, seq, hn,
                                                                                   kvn, hs, rot, tokens), flush=True)
        rr = np.random.default_rng(4000 + case)
        qkv = rr.standard_normal((tokens, hn + 2 * kvn, hs), dtype=np.float32).astype(dtype)
        bias = (0.05 * rr.standard_normal((hn + 2 * kvn) * hs)).astype(dtype) if case % 3 else None
        po, _ = padding_offsets_np(lens, seq)
        td = NP2T[dtype]
        q = torch.full((batch, hn, seq, hs), -9, dtype=td, device="cuda")
        k = torch.full((batch, kvn, seq, hs), -9, dtype=td, device="cuda")
        v = torch.full((batch, kvn, seq, hs), -9, dtype=td, device="cuda")
        d_po = torch.zeros((batch, seq), dtype=torch.int32, device="cuda")
        d_cum = torch.zeros(batch + 1, dtype=torch.int32, device="cuda")
        isp.cal_padding_offset(d_po, d_cum, dev(lens))
        assert np.array_equal(d_po.cpu().numpy().reshape(-1)[:tokens], po)
        if tokens:
            isp.add_fused_qkv_bias_transpose_and_rope(q, k, v, dev(qkv), dev(bias), d_po, dev(hist), dev(lens), rot, 10000.0)
        eq, ek, ev = oracle.qkv_rope(qkv, bias, po, hist, lens, batch, seq, hn, kvn, rot, 10000.0, fill=-9.0)
        assert np.array_equal(v.cpu().numpy(), ev)
        rad = rope_pair_radius(qkv, bias)
        p = np.arange(tokens) + po
        b, s = p // seq, p % seq
        for got, exp, sl in ((q.cpu().numpy(), eq, slice(0, hn)), (k.cpu().numpy(), ek, slice(hn, hn + kvn))):
            valid = np.arange(seq)[None, :] < lens[:, None]
            pad = ~np.broadcast_to(valid[:, None, :, None], exp.shape)
            assert np.array_equal(got[pad], exp[pad])
            if dtype == np.float32:
                assert_f32_close(got[b, :, s, :], exp[b, :, s, :], "rope", scale=rad[:, sl] + 1e-30)
            else:
                assert_f16_close(got[b, :, s, :], exp[b, :, s, :], "rope", magnitude=rad[:, sl], max_mismatch_fraction=0.05)
        # the way back: transpose-out + remove padding recovers the packed v rows (times the GQA broadcast)
        back = torch.zeros((tokens, kvn, hs), dtype=td, device="cuda")
        isp.transpose_out_remove_padding(v, d_po, back)
        assert np.array_equal(back.cpu().numpy(), oracle.transpose_remove_padding(ev, po, tokens))
        # cache append at history, then broadcast to the query heads
        max_seq = int(seq + hist.max() + 1)
        cache_k = torch.zeros((2, batch, kvn, max_seq, hs), dtype=td, device="cuda")
        cache_v = torch.zeros_like(cache_k)
        isp.concat_kv_cache(k, v, 1, dev(lens), dev(hist), cache_k, cache_v)
        e_ck = oracle.concat_kv(k.cpu().numpy(), np.zeros(cache_k.shape, dtype), 1, lens, hist)  # same source bits
        assert np.array_equal(cache_k.cpu().numpy(), e_ck)
        ctx = (lens + hist).astype(np.int32)
        max_k = int(max(1, ctx.max()))
        rep_k = torch.full((batch, hn, max_k, hs), -2, dtype=td, device="cuda")
        rep_v = torch.full((batch, hn, max_k, hs), -2, dtype=td, device="cuda")
        isp.repeat_kv_cache(cache_k, cache_v, dev(ctx), 1, rep_k, rep_v)
        assert np.array_equal(rep_k.cpu().numpy(), oracle.repeat_kv(e_ck, 1, ctx, hn, max_k, fill=-2.0))


def test_c_abi_is_reentrant_across_host_threads(isp, oracle):
    """Four host threads launch different kernels on their own streams at the same time."""
    results, errors = {}, []
    res, out, bias, gamma = norm_inputs(512, 4096, np.float16, seed=7)
    x = swiglu_inputs(256, 11008, np.float16, seed=8)
    ids, table = embedding_inputs(1024, 4096, 2000, np.float16, seed=9)
    d = {"res": dev(res), "out": dev(out), "bias": dev(bias), "gamma": dev(gamma), "x": dev(x), "ids": dev(ids),
         "table": dev(table)}
    torch.cuda.synchronize()

    def worker(name):
        try:
            stream = torch.cuda.Stream()
            with torch.cuda.stream(stream):
                for _ in range(20):
                    if name == "norm":
                        r_, o_ = d["res"].clone(), d["out"].clone()
                        isp.fused_add_bias_residual_rmsnorm(r_, o_, d["bias"], d["gamma"], 1e-5)
                        results[name] = (r_, o_)
                    elif name == "swiglu":
                        o_ = torch.empty((256, 11008), dtype=torch.float16, device="cuda")
                        isp.act(d["x"], o_)
                        results[name] = o_
                    else:
                        o_ = torch.empty((1024, 4096), dtype=torch.float16, device="cuda")
                        isp.input_embedding(d["ids"], o_, d["table"])
                        results[name] = o_
                stream.synchronize()
        except Exception as e:  # noqa: BLE001
            errors.append((name, e))

    threads = [threading.Thread(target=worker, args=(n,)) for n in ("norm", "swiglu", "embed", "embed2")]
    for t in threads:
        t.start()
    for t in threads:
        t.join()
    assert not errors, errors
    torch.cuda.synchronize()
    e_res, e_out = oracle.fused_norm(res, out, bias, gamma, 1e-5)
    assert np.array_equal(results["norm"][0].cpu().numpy(), e_res)
    assert_f16_close(results["norm"][1].cpu().numpy(), e_out, "norm under concurrency")
    assert_f16_close(results["swiglu"].cpu().numpy(), oracle.swiglu(x), "swiglu under concurrency")
    assert np.array_equal(results["embed"].cpu().numpy(), oracle.embedding(ids, table))
    assert np.array_equal(results["embed2"].cpu().numpy(), oracle.embedding(ids, table))
