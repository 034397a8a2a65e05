"""The oracle against every known answer the reference's unit tests hold for this path, and against
the committed float64 fixtures (tests/golden/)."""
import json
import os

import numpy as np
import pytest

from helpers import assert_f16_close, assert_f32_close

GOLD = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")


@pytest.fixture(scope="module")
def known():
    with open(os.path.join(GOLD, "reference_known_answers.json")) as f:
        return json.load(f)


@pytest.fixture(scope="module")
def f64():
    return np.load(os.path.join(GOLD, "float64_cases.npz"))


def test_padding_offset_known_answer(oracle, known):
    k = known["cal_padding_offset"]
    po, cum = oracle.cal_padding_offset(k["input_lengths"], k["max_q_len"], fill=-7)
    n = len(k["padding_offset_prefix"])
    assert po.reshape(-1)[:n].tolist() == k["padding_offset_prefix"]
    assert np.all(po.reshape(-1)[n:] == -7)  # entries past the token count stay untouched
    assert cum.tolist() == k["cum_seqlens"]


@pytest.mark.parametrize("dtype", [np.float32, np.float16])
def test_fused_norm_known_answer(oracle, known, dtype):
    k = known["fused_norm"]
    out = np.full((k["tokens"], k["hidden"]), k["decoder_out"], dtype)
    res = np.full((k["tokens"], k["hidden"]), k["residual"], dtype)
    gamma = np.full(k["hidden"], k["gamma"], dtype)
    rs, y = oracle.fused_norm(res, out, None, gamma, k["eps"])
    exp = np.full_like(out, k["expected_out"])
    if dtype == np.float32:
        assert_f32_close(y, exp, "fused norm known answer")
    else:
        assert np.array_equal(y, exp)  # 1/sqrt(1.5) rounds to a single fp16 value
    assert np.all(rs == k["expected_residual"])


def test_swiglu_known_answer(oracle, known):
    k = known["swiglu"]
    x32 = np.full((k["batch"], 2, k["inter"]), k["input"], np.float32)
    assert_f32_close(oracle.swiglu(x32), np.full((k["batch"], k["inter"]), k["expected_f32"]), "swiglu f32")
    y16 = oracle.swiglu(x32.astype(np.float16))
    assert np.all(y16 == np.float16(k["expected_f16"]))


@pytest.mark.parametrize("dtype", [np.float32, np.float16])
def test_embedding_known_answer(oracle, known, dtype):
    k = known["embedding"]
    table = np.repeat(np.arange(k["vocab"], dtype=np.float32).astype(dtype)[:, None], k["hidden"], axis=1)
    ids = np.random.default_rng(3).integers(0, k["vocab"], k["tokens"], dtype=np.int32)
    out = oracle.embedding(ids, table)
    assert np.array_equal(out[:, 0], ids.astype(np.float32).astype(dtype))
    assert np.all(out == out[:, :1])


def test_qkv_rope_known_answer(oracle, known):
    k = known["qkv_rope"]
    B, S, hn, kvn, hs = k["batch"], k["seq_len"], k["head_num"], k["kv_head_num"], k["head_size"]
    qkv = np.full((B * S, hn + 2 * kvn, hs), k["qkv"], np.float32)
    po = np.full(B * S, k["padding_offset"], np.int32)
    hist = np.full(B, k["history_length"], np.int32)
    ilen = np.full(B, k["input_length"], np.int32)
    s = np.arange(S, dtype=np.float64)[:, None]
    d = np.arange(hs // 2, dtype=np.float64)[None, :]
    a = s / 10000.0 ** (d / 64.0)
    for bias, amp in ((None, 32.0), (np.full((hn + 2 * kvn) * hs, k["bias"], np.float32), 34.0)):
        q, kk, v = oracle.qkv_rope(qkv, bias, po, hist, ilen, B, S, hn, kvn, k["rotary_dim"], k["rotary_base"])
        exp = np.concatenate([amp * (np.cos(a) - np.sin(a)), amp * (np.cos(a) + np.sin(a))], axis=1)
        exp = np.broadcast_to(exp[None, None], q.shape)
        # the angle is formed in fp32 (half an ulp of up to 31 rad), so allow ulp32(angle) on top
        scale = amp * np.sqrt(2.0) * (1.0 + np.broadcast_to(np.concatenate([a, a], 1)[None, None], q.shape) * 0.02)
        assert_f32_close(q, exp, "q known answer", scale=scale)
        assert_f32_close(kk, exp, "k known answer", scale=scale)
        assert np.all(v == amp)


def test_transpose_remove_padding_known_answer(oracle, known):
    k = known["transpose_remove_padding"]
    src = np.arange(k["batch"] * k["head_num"] * k["max_seq_len"] * k["head_size"], dtype=np.float32)
    src = src.reshape(k["batch"], k["head_num"], k["max_seq_len"], k["head_size"])
    out = oracle.transpose_remove_padding(src, k["padding_offset"], k["num_tokens"])
    assert out.tolist() == k["expected"]


# ---------------------------------------------------------------- committed float64 fixtures

@pytest.mark.parametrize("excl", [False, True])
def test_fused_norm_float64_fixture(oracle, f64, excl):
    tag = "excl" if excl else "incl"
    rs, y = oracle.fused_norm(f64["norm_residual"], f64["norm_out"], f64["norm_bias"], f64["norm_gamma"],
                              1e-5, flags=1 if excl else 0)
    assert_f32_close(y, f64["norm_y_" + tag], "fused norm y")
    assert_f32_close(rs, f64["norm_res_" + tag], "fused norm residual", rtol=2e-7,
                     scale=np.abs(f64["norm_out"]) + np.abs(f64["norm_residual"]) + 1)
    y16 = oracle.fused_norm(f64["norm_residual"].astype(np.float16), f64["norm_out"].astype(np.float16),
                            f64["norm_bias"].astype(np.float16), f64["norm_gamma"].astype(np.float16),
                            1e-5, flags=1 if excl else 0)
    import npref
    e_rs, e_y = npref.fused_norm64(f64["norm_residual"].astype(np.float16), f64["norm_out"].astype(np.float16),
                                   f64["norm_bias"].astype(np.float16), f64["norm_gamma"].astype(np.float16),
                                   1e-5, residual_excludes_bias=excl)
    assert_f16_close(y16[1], e_y.astype(np.float16), "fused norm f16 y")
    assert_f16_close(y16[0], e_rs.astype(np.float16), "fused norm f16 residual")


def test_rmsnorm_float64_fixture(oracle, f64):
    assert_f32_close(oracle.rmsnorm(f64["norm_out"], f64["norm_gamma"], 1e-5), f64["rmsnorm_y"], "rmsnorm")


def test_swiglu_float64_fixture(oracle, f64):
    x = f64["swiglu_in"]
    assert_f32_close(oracle.swiglu(x), f64["swiglu_out"], "swiglu f32",
                     scale=np.abs(f64["swiglu_out"]) + 1e-3 * np.abs(x[:, 1]))
    import npref
    x16 = x.astype(np.float16)
    assert_f16_close(oracle.swiglu(x16), npref.swiglu64(x16).astype(np.float16), "swiglu f16")


def test_qkv_rope_float64_fixture(oracle, f64):
    batch, seq, hn, kvn, hs, rot = [int(t) for t in f64["qkv_dims"]]
    q, k, v = oracle.qkv_rope(f64["qkv_in"], f64["qkv_bias"], f64["qkv_po"], f64["qkv_hist"], f64["qkv_lens"],
                              batch, seq, hn, kvn, rot, float(f64["qkv_base"]), fill=0.0)
    x = f64["qkv_in"].astype(np.float64) + f64["qkv_bias"].reshape(1, -1, hs)
    radius = float(np.abs(x).max()) * np.sqrt(2.0)
    # angle formed in fp32: allow ulp32 of the largest angle (t <= 20) on top of 1e-5
    for got, exp, name in ((q, f64["qkv_q"], "q"), (k, f64["qkv_k"], "k")):
        assert_f32_close(got, exp, name, scale=np.full(exp.shape, radius * 1.3))
    assert_f32_close(v, f64["qkv_v"], "v", rtol=2e-7, scale=np.abs(f64["qkv_v"]) + 1)
    # padded positions untouched, bit-exact
    w = f64["qkv_written"]
    assert np.all(q[~w[:, None, :].repeat(hn, 1)] == 0.0)
    assert np.all(v[~w[:, None, :].repeat(kvn, 1)] == 0.0)


def test_reference_mover_configurations(oracle):
    """The configurations of the reference's own programs for the KV-cache append and broadcast."""
    from helpers import reference_mover_configurations
    k_src, cache, expect_cache, src_cache, expect_rep = reference_mover_configurations()
    assert np.array_equal(oracle.concat_kv(k_src, cache, 0, [16], [1]), expect_cache)
    assert np.array_equal(oracle.repeat_kv(src_cache, 0, [2], 2, 2), expect_rep)
