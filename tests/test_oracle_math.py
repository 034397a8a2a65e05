"""Pins the oracle by what the mathematics fixes: library routines (torch / scipy on the CPU),
invariants and brute force on small inputs.  Each check is chosen so that a plausible mistake (a
dropped term, a wrong sign or index, a swapped operand) fails it."""
import numpy as np
import pytest
import torch

import npref
from helpers import (assert_f16_close, assert_f32_close, embedding_inputs, norm_inputs, padding_offsets_np,
                     qkv_inputs, swiglu_inputs)


# ------------------------------------------------------------------ embedding
@pytest.mark.parametrize("dtype", [np.float16, np.float32])
def test_embedding_equals_library_gather(oracle, dtype):
    ids, table = embedding_inputs(97, 136, 513, dtype, seed=5)
    out = oracle.embedding(ids, table)
    assert np.array_equal(out.view(np.uint8), np.take(table, ids, axis=0).view(np.uint8))
    t = torch.nn.functional.embedding(torch.from_numpy(ids.astype(np.int64)), torch.from_numpy(table))
    assert np.array_equal(out.view(np.uint8), t.numpy().view(np.uint8))


def test_embedding_empty(oracle):
    ids, table = embedding_inputs(0, 8, 4, np.float16)
    assert oracle.embedding(ids, table).shape == (0, 8)


# ------------------------------------------------------------------ padding offset
@pytest.mark.parametrize("lens,max_q", [([3, 2, 5], 5), ([1], 1), ([0, 4, 0, 2], 4), ([7] * 9, 7), ([], 3)])
def test_padding_offset_equals_cumsum(oracle, lens, max_q):
    po, cum = oracle.cal_padding_offset(np.array(lens, np.int32), max_q, fill=-1)
    epo, ecum = padding_offsets_np(lens, max_q)
    n = int(np.sum(lens)) if len(lens) else 0
    assert np.array_equal(po.reshape(-1)[:n], epo)
    assert np.all(po.reshape(-1)[n:] == -1)
    assert np.array_equal(cum, ecum)


def test_padding_offset_places_tokens_inside_their_sequence(oracle):
    r = np.random.default_rng(2)
    lens = r.integers(0, 33, 17).astype(np.int32)
    po, cum = oracle.cal_padding_offset(lens, 32)
    n = int(lens.sum())
    p = np.arange(n) + po.reshape(-1)[:n]
    b, s = p // 32, p % 32
    assert np.array_equal(b, np.repeat(np.arange(17), lens))
    assert np.array_equal(s, np.concatenate([np.arange(l) for l in lens]))


# ------------------------------------------------------------------ norm
def test_rmsnorm_equals_torch_rms_norm(oracle):
    _, x, _, gamma = norm_inputs(19, 320, np.float32, seed=7, with_residual=False, with_bias=False)
    y = oracle.rmsnorm(x, gamma, 1e-5)
    t = torch.nn.functional.rms_norm(torch.from_numpy(x).double(), (320,), torch.from_numpy(gamma).double(), 1e-5)
    assert_f32_close(y, t.numpy(), "rmsnorm vs torch")


@pytest.mark.parametrize("dtype", [np.float32, np.float16])
@pytest.mark.parametrize("with_res,with_bias", [(True, True), (True, False), (False, True), (False, False)])
def test_fused_norm_equals_float64_closed_form(oracle, dtype, with_res, with_bias):
    res, out, bias, gamma = norm_inputs(11, 200, dtype, seed=11, with_residual=with_res, with_bias=with_bias)
    for flags in (0, 1):
        rs, y = oracle.fused_norm(res, out, bias, gamma, 1e-5, flags=flags)
        ers, ey = npref.fused_norm64(res, out, bias, gamma, 1e-5, residual_excludes_bias=bool(flags))
        if dtype == np.float32:
            assert_f32_close(y, ey, "y")
            if with_res:
                assert_f32_close(rs, ers, "residual", rtol=2e-7, scale=np.abs(ers) + 4)
        else:
            assert_f16_close(y, ey.astype(np.float16), "y f16")
            if with_res:
                assert_f16_close(rs, ers.astype(np.float16), "residual f16")
        if not with_res:
            assert rs is None


def test_fused_norm_invariants(oracle):
    res, out, bias, gamma = norm_inputs(8, 256, np.float32, seed=13)
    rs, y = oracle.fused_norm(res, out, bias, gamma, 1e-5)
    x = rs.astype(np.float64)
    # stored residual is exactly the fp32 sum
    assert np.array_equal(rs, (out + res) + bias)
    # mean((y/gamma)^2) * (1 + eps/mean(x^2)) == 1
    ms = (x * x).mean(axis=1)
    lhs = ((y / gamma).astype(np.float64) ** 2).mean(axis=1) * (1 + 1e-5 / ms)
    assert np.allclose(lhs, 1.0, rtol=0, atol=5e-6)
    # scale equivariance (eps scaled with the square): norm(2x) == norm(x)
    _, y2 = oracle.fused_norm(2 * res, 2 * out, 2 * bias, gamma, 4e-5)
    assert_f32_close(y2, y, "scale equivariance", rtol=1e-6)
    # null bias == zero bias ; null residual == zero residual in the output
    _, y0 = oracle.fused_norm(res, out, np.zeros_like(bias), gamma, 1e-5)
    _, yn = oracle.fused_norm(res, out, None, gamma, 1e-5)
    assert np.array_equal(y0, yn)
    _, yz = oracle.fused_norm(np.zeros_like(res), out, None, gamma, 1e-5)
    assert np.array_equal(yz, oracle.rmsnorm(out, gamma, 1e-5))
    # the literal-reference flag only changes the stored residual
    rs1, y1 = oracle.fused_norm(res, out, bias, gamma, 1e-5, flags=1)
    assert np.array_equal(y1, y)
    assert np.array_equal(rs1, out + res)


# ------------------------------------------------------------------ swiglu
@pytest.mark.parametrize("dtype", [np.float32, np.float16])
def test_swiglu_equals_torch_silu(oracle, dtype):
    x = swiglu_inputs(13, 72, dtype, seed=17) * dtype(3)
    y = oracle.swiglu(x)
    t = torch.from_numpy(x.astype(np.float64))
    e = (torch.nn.functional.silu(t[:, 0]) * t[:, 1]).numpy()
    if dtype == np.float32:
        assert_f32_close(y, e, "swiglu vs torch silu", scale=np.abs(e) + 1e-3 * np.abs(x[:, 1]))
    else:
        assert_f16_close(y, e.astype(np.float16), "swiglu f16 vs torch silu")


def test_swiglu_special_values(oracle):
    g = np.array([0.0, -0.0, 1.0, -1.0, 20.0, -20.0, 65504.0, -65504.0, 1e-4], np.float32)
    x = np.stack([g, np.ones_like(g)])[None]
    y = oracle.swiglu(x)[0]
    assert y[0] == 0 and y[1] == 0
    assert np.isfinite(y).all()
    assert y[6] == 65504.0 and y[7] == 0.0
    # silu(x) - silu(-x) == x
    assert abs((y[2] - y[3]) - 1.0) < 1e-6 and abs((y[4] - y[5]) - 20.0) < 1e-5
    y16 = oracle.swiglu(x.astype(np.float16))[0]
    assert np.isfinite(y16.astype(np.float32)).all() and y16[6] == np.float16(65504)


# ------------------------------------------------------------------ qkv + rope + re-pad
@pytest.mark.parametrize("dtype", [np.float32, np.float16])
@pytest.mark.parametrize("hn,kvn,hs,rot", [(4, 4, 16, 16), (8, 2, 32, 32), (4, 1, 16, 8), (2, 2, 128, 128)])
def test_qkv_rope_equals_complex_rotation_and_scatter(oracle, dtype, hn, kvn, hs, rot):
    batch, seq = 3, 12
    lens, qkv, bias, po, _ = qkv_inputs(batch, seq, hn, kvn, hs, dtype, seed=19, min_len=0)
    hist = np.array([0, 5, 17], np.int32)
    q, k, v = oracle.qkv_rope(qkv, bias, po, hist, lens, batch, seq, hn, kvn, rot, 10000.0, fill=-9.0)
    eq, ek, ev, written = npref.qkv_rope64(qkv, bias, po, hist, batch, seq, hn, kvn, rot, 10000.0, fill=-9.0)
    x = qkv.astype(np.float64) + bias.astype(np.float64).reshape(1, -1, hs)
    radius = np.sqrt(2.0) * np.abs(x).max()
    if dtype == np.float32:
        # fp32 angle (t <= 28): half an ulp is 1e-6 rad, inside the 1e-5 band relative to the radius
        assert_f32_close(q, eq, "q", scale=np.full(q.shape, radius))
        assert_f32_close(k, ek, "k", scale=np.full(k.shape, radius))
        assert_f32_close(v, ev, "v", rtol=2e-7, scale=np.abs(ev) + 1)
    else:
        assert_f16_close(q, eq.astype(np.float16), "q f16")
        assert_f16_close(k, ek.astype(np.float16), "k f16")
        assert_f16_close(v, ev.astype(np.float16), "v f16")
    # every valid (b, s) written exactly where the lengths say, nothing else touched
    valid = np.arange(seq)[None, :] < lens[:, None]
    assert np.array_equal(written, valid)
    assert np.all(q[~valid[:, None, :].repeat(hn, 1)] == dtype(-9))
    assert np.all(k[~valid[:, None, :].repeat(kvn, 1)] == dtype(-9))


def test_qkv_rope_invariants(oracle):
    batch, seq, hn, kvn, hs = 2, 8, 4, 4, 32
    lens, qkv, _, po, hist = qkv_inputs(batch, seq, hn, kvn, hs, np.float32, seed=23, with_bias=False)
    q, k, v = oracle.qkv_rope(qkv, None, po, hist, lens, batch, seq, hn, kvn, hs, 10000.0)
    n = int(lens.sum())
    p = np.arange(n) + po[:n]
    b, s = p // seq, p % seq
    src_q = qkv[:, :hn]
    got_q = q[b, :, s, :]
    # rotation preserves x_d^2 + x_{d+half}^2
    r_in = src_q[..., :hs // 2] ** 2 + src_q[..., hs // 2:] ** 2
    r_out = got_q[..., :hs // 2] ** 2 + got_q[..., hs // 2:] ** 2
    assert np.allclose(r_in, r_out, rtol=1e-5, atol=1e-6)
    # timestep 0 is the identity
    first = s == 0
    assert np.array_equal(got_q[first], src_q[first])
    # pair d = 0 rotates by exactly t radians
    t = s.astype(np.float64)[:, None]
    assert np.allclose(got_q[..., 0], np.cos(t) * src_q[..., 0] - np.sin(t) * src_q[..., hs // 2], atol=1e-5)
    assert np.allclose(got_q[..., hs // 2], np.cos(t) * src_q[..., hs // 2] + np.sin(t) * src_q[..., 0], atol=1e-5)
    # history h at position s == history 0 at position h + s (same sequence shifted inside a longer pad)
    hist2 = np.array([3, 1], np.int32)
    q2, _, _ = oracle.qkv_rope(qkv, None, po, hist2, lens, batch, seq, hn, kvn, hs, 10000.0)
    ang = npref.rope_angles64(hist2[b] + s, hs, hs, 10000.0)[:, None, :]
    assert_f32_close(q2[b, :, s, :], npref.rotate_half64(src_q, ang), "history shift",
                     scale=np.full(src_q.shape, np.abs(src_q).max() * 1.5))
    # v is a pure copy
    assert np.array_equal(v[b, :, s, :], qkv[:, hn + kvn:])


# ------------------------------------------------------------------ decode rope, transpose, kv movers
@pytest.mark.parametrize("dtype", [np.float32, np.float16])
def test_rope_decode_equals_prefill_rotation(oracle, dtype):
    hn, kvn, hs, step = 4, 4, 32, 9
    x = np.random.default_rng(29).standard_normal((1, hn + 2 * kvn, hs)).astype(dtype)
    y = oracle.rope_decode(x, hn, kvn, step, hs, 10000.0)
    # the prefill step with one token at history = step - 1 must give the same q and k
    q, k, v = oracle.qkv_rope(x, None, np.zeros(1, np.int32), np.array([step - 1], np.int32),
                              np.ones(1, np.int32), 1, 1, hn, kvn, hs, 10000.0)
    assert np.array_equal(y[0, :hn], q[0, :, 0, :])
    assert np.array_equal(y[0, hn:hn + kvn], k[0, :, 0, :])
    assert np.array_equal(y[0, hn + kvn:], x[0, hn + kvn:])  # v untouched
    ang = npref.rope_angles64([step - 1], hs, hs, 10000.0)[None]
    e = npref.rotate_half64(x[:, :hn + kvn].astype(np.float64), ang)
    if dtype == np.float32:
        assert_f32_close(y[:, :hn + kvn], e, "decode rope", scale=np.full(e.shape, 8.0))
    else:
        assert_f16_close(y[:, :hn + kvn], e.astype(np.float16), "decode rope f16")


def test_transpose_remove_padding_inverts_the_scatter(oracle):
    batch, seq, hn, kvn, hs = 3, 10, 4, 4, 16
    lens, qkv, _, po, hist = qkv_inputs(batch, seq, hn, kvn, hs, np.float32, seed=31, with_bias=False, min_len=1)
    _, _, v = oracle.qkv_rope(qkv, None, po, hist, lens, batch, seq, hn, kvn, hs, 10000.0)
    back = oracle.transpose_remove_padding(v, po, int(lens.sum()))
    assert np.array_equal(back, qkv[:, hn + kvn:])


def test_kv_movers_equal_numpy_slicing(oracle):
    r = np.random.default_rng(37)
    layers, batch, kvn, hn, max_q, max_seq, hs = 3, 2, 2, 6, 5, 16, 8
    src = r.standard_normal((batch, kvn, max_q, hs)).astype(np.float16)
    cache = r.standard_normal((layers, batch, kvn, max_seq, hs)).astype(np.float16)
    cur = np.array([5, 3], np.int32)
    hist = np.array([4, 0], np.int32)
    got = oracle.concat_kv(src, cache, 1, cur, hist)
    exp = cache.copy()
    for b in range(batch):
        exp[1, b, :, hist[b]:hist[b] + cur[b]] = src[b, :, :cur[b]]
    assert np.array_equal(got, exp)
    ctx = hist + cur
    rep = oracle.repeat_kv(got, 1, ctx, hn, 12, fill=-3.0)
    exp_rep = np.full((batch, hn, 12, hs), -3.0, np.float16)
    for b in range(batch):
        exp_rep[b, :, :ctx[b]] = np.repeat(got[1, b], hn // kvn, axis=0)[:, :ctx[b]]
    assert np.array_equal(rep, exp_rep)
