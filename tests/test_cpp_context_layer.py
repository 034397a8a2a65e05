"""The C++ context-decoder layer (include/src/layers/decoder/context_decoder_layer.h: launch* kernels +
hipBLASLt GEMMs over TensorMap / LlamaLayerWeight / BaseAllocator) against an independent float64
implementation of the same layer, written the Hugging Face way (rotate_half with cos/sin tables, dense
causal attention, weights applied as x @ W.T).  build/bin/test_context_layer runs the layer and dumps
every operand and result; this file recomputes the results in float64 from the dumped operands."""
import math
import os
import subprocess

import numpy as np
import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
EXE = os.path.join(ROOT, "build", "bin", "test_context_layer")
LAYER_LIB = os.path.join(ROOT, "inferspore_amd", "lib", "libinferspore_layers.so")


def rms(x, g, eps=1e-5):
    return x / np.sqrt((x * x).mean(-1, keepdims=True) + eps) * g


def rotate_half(x):
    h = x.shape[-1] // 2
    return np.concatenate([-x[..., h:], x[..., :h]], -1)


def reference_layer(residual_rows, lens, w, nh, kvh, hs, base=10000.0):
    """residual_rows: list of [len_b, H] float64 arrays (positions 0 .. len-1, no history).
    Returns (new residual rows, next layer's normalised input rows, k rows, v rows)."""
    H = nh * hs
    rep = nh // kvh
    res_out, next_out, ks, vs = [], [], [], []
    for x in residual_rows:
        S = x.shape[0]
        normed = rms(x, w["attn_norm"])
        qkv = normed @ w["qkv_weight"].T + w["qkv_bias"]
        q = qkv[:, :H].reshape(S, nh, hs).transpose(1, 0, 2)
        k = qkv[:, H:H + kvh * hs].reshape(S, kvh, hs).transpose(1, 0, 2)
        v = qkv[:, H + kvh * hs:].reshape(S, kvh, hs).transpose(1, 0, 2)
        pos = np.arange(S, dtype=np.float64)
        inv_freq = 1.0 / base ** (np.arange(0, hs, 2, dtype=np.float64) / hs)
        ang = np.outer(pos, inv_freq)
        cos, sin = np.concatenate([np.cos(ang)] * 2, -1), np.concatenate([np.sin(ang)] * 2, -1)
        q = q * cos + rotate_half(q) * sin
        k = k * cos + rotate_half(k) * sin
        ks.append(k)
        vs.append(v)
        kk, vv = np.repeat(k, rep, axis=0), np.repeat(v, rep, axis=0)
        scores = q @ kk.transpose(0, 2, 1) / math.sqrt(hs)
        scores = np.where(np.tril(np.ones((S, S), bool))[None], scores, -np.inf)
        p = np.exp(scores - scores.max(-1, keepdims=True))
        p /= p.sum(-1, keepdims=True)
        ctx = (p @ vv).transpose(1, 0, 2).reshape(S, H)
        r = x + ctx @ w["o_weight"].T + w["o_bias"]
        n2 = rms(r, w["ffn_norm"])
        gu = n2 @ w["gate_up_weight"].T
        inter = gu.shape[-1] // 2
        g = gu[:, :inter]
        ffn = (g / (1.0 + np.exp(-g)) * gu[:, inter:]) @ w["down_weight"].T
        r = r + ffn
        res_out.append(r)
        next_out.append(rms(r, w["next_norm"]))
    return res_out, next_out, ks, vs


@pytest.mark.gpu
@pytest.mark.parametrize("dtype,tol", [("f32", 2e-4), ("f16", 3e-2)])
@pytest.mark.parametrize("nh,kvh,hs,inter,attention", [(2, 2, 128, 512, "fused"), (4, 2, 128, 512, "fused"),
                                                        (2, 2, 128, 512, "padded"), (4, 2, 64, 384, "fused"), (4, 2, 64, 384, "padded")])
def test_cpp_context_layer_matches_float64(tmp_path, dtype, tol, nh, kvh, hs, inter, attention):
    """fp16 layers with 128- or 64-element heads run the fused attention kernel unless the environment asks for the padded
    batched form; fp32 layers and other head sizes always run the padded form."""
    assert os.path.exists(EXE), "build/bin/test_context_layer is missing: run python -m inferspore_amd.build"
    print("[case] test_context_layer %s %d/%d heads x %d, inter %d, %s attention" % (dtype, nh, kvh, hs, inter, attention),
          flush=True)
    env = dict(os.environ)
    env.pop("ISP_LAYERS_ATTENTION", None)
    if attention == "padded":
        env["ISP_LAYERS_ATTENTION"] = "padded"
    p = subprocess.run([EXE, dtype, str(tmp_path), str(nh), str(kvh), str(hs), str(inter)], stdout=subprocess.PIPE,
                       stderr=subprocess.STDOUT, text=True, timeout=200, env=env)
    assert p.returncode == 0 and "passed" in p.stdout, p.stdout[-3000:]
    H, lens, layers, max_seq = nh * hs, [16, 5, 11], 2, 32
    load = lambda name: np.fromfile(os.path.join(str(tmp_path), name + ".bin"), np.float32).astype(np.float64)
    qkv_out = (nh + 2 * kvh) * hs
    w = {"attn_norm": load("attn_norm"), "ffn_norm": load("ffn_norm"), "next_norm": load("next_norm"),
         "qkv_weight": load("qkv_weight").reshape(qkv_out, H), "qkv_bias": load("qkv_bias"),
         "o_weight": load("o_weight").reshape(H, H), "o_bias": load("o_bias"),
         "gate_up_weight": load("gate_up_weight").reshape(2 * inter, H), "down_weight": load("down_weight").reshape(H, inter)}
    x = load("residual_in").reshape(-1, H)
    starts = np.concatenate([[0], np.cumsum(lens)])
    rows = [x[starts[b]:starts[b + 1]] for b in range(len(lens))]
    e_res, e_next, e_k, e_v = reference_layer(rows, lens, w, nh, kvh, hs)
    for name, exp in (("residual_out", np.concatenate(e_res)), ("decoder_output", np.concatenate(e_next))):
        got = load(name).reshape(-1, H)
        err, scale = np.abs(got - exp).max(), np.abs(exp).max()
        assert err <= tol * scale, "%s: max error %g vs scale %g" % (name, err, scale)
    # the KV cache of layer 1 holds the rotated keys and the values at rows 0 .. len-1; layer 0 is untouched
    for name, exp_rows in (("k_cache", e_k), ("v_cache", e_v)):
        cache = load(name).reshape(layers, len(lens), kvh, max_seq, hs)
        assert not cache[0].any(), "the other layer's cache must stay untouched"
        for b, l in enumerate(lens):
            err, scale = np.abs(cache[1, b, :, :l] - exp_rows[b]).max(), np.abs(exp_rows[b]).max()
            assert err <= tol * scale, "%s row block %d: max error %g vs scale %g" % (name, b, err, scale)
            assert not cache[1, b, :, l:].any(), "rows past the sequence must stay untouched"


@pytest.mark.gpu
def test_cpp_fused_context_attention_matches_float64():
    exe = os.path.join(ROOT, "build", "bin", "test_context_attention")
    assert os.path.exists(exe), "build/bin/test_context_attention is missing: run python -m inferspore_amd.build"
    print("[case] test_context_attention", flush=True)
    p = subprocess.run([exe], stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True, timeout=200)
    assert p.returncode == 0 and "context attention: passed" in p.stdout, p.stdout[-3000:]


def test_layers_library_exports_the_layer_classes():
    assert os.path.exists(LAYER_LIB), "libinferspore_layers.so is missing: run python -m inferspore_amd.build"
    syms = subprocess.run(["nm", "-D", "--defined-only", "-C", LAYER_LIB], stdout=subprocess.PIPE, text=True,
                          check=True).stdout
    for t in ("float", "__half"):
        assert "LlamaContextDecoderLayer<%s>::forward(" % t in syms
        assert "LlamaContextDecoderLayer<%s>::allocForForward(" % t in syms
        assert "LlamaLayerWeight<%s>::loadWeights()" % t in syms
        assert "isp_layers::launch_masked_scaled_softmax<%s>(" % t in syms
    assert "isp_layers::launch_fused_context_attention(" in syms
    assert "isp_layers::fused_context_attention_supports(" in syms
