"""End-to-end check of the kernels composed in model order: one LLaMA prefill layer assembled from this
library's kernels (inferspore_amd.context_layer) against an independent float64 implementation of the
same layer written the Hugging Face way (rotate_half with cos/sin tables, dense causal attention).
This pins the cross-kernel contracts -- head layout of the packed QKV row, rotate-half pairing, padded
[b, h, s, d] scatter and its inverse, KV-cache rows at history + s, gate/up packing -- in one place."""
import math

import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu


def rms64(x, g, eps):
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps) * g


def rotate_half(x):
    h = x.shape[-1] // 2
    return torch.cat([-x[..., h:], x[..., :h]], dim=-1)


def reference_layer64(residual_pad, lens, w, nh, hs, next_gamma, eps=1e-5, base=10000.0):
    """residual_pad [B, S, H] float64 (one contiguous sequence per row, positions 0 .. len-1).
    Returns (new residual, next layer's normalised input), both [B, S, H]."""
    B, S, H = residual_pad.shape
    f = lambda t: t.double()
    normed = rms64(residual_pad, f(w.attn_norm), eps)
    qkv = normed @ f(w.qkv)
    q, k, v = [t.view(B, S, nh, hs).transpose(1, 2) for t in qkv.split(H, dim=-1)]       # [B, nh, S, hs]
    pos = torch.arange(S, dtype=torch.float64, device=residual_pad.device)
    inv_freq = 1.0 / (base ** (torch.arange(0, hs, 2, dtype=torch.float64, device=pos.device) / hs))
    ang = torch.outer(pos, inv_freq)
    cos, sin = torch.cat([ang.cos(), ang.cos()], -1), torch.cat([ang.sin(), ang.sin()], -1)
    q = q * cos + rotate_half(q) * sin
    k = k * cos + rotate_half(k) * sin
    scores = q @ k.transpose(-1, -2) / math.sqrt(hs)
    i = torch.arange(S, device=pos.device)
    allowed = (i[None, :] <= i[:, None])[None] & (i[None, None, :] < lens[:, None, None])     # causal & key valid
    scores = scores.masked_fill(~allowed[:, None], float("-inf"))
    ctx = torch.softmax(scores, -1) @ v
    attn = ctx.transpose(1, 2).reshape(B, S, H) @ f(w.o)
    residual = residual_pad + attn
    n2 = rms64(residual, f(w.ffn_norm), eps)
    gu = n2 @ f(w.gate_up)
    inter = gu.shape[-1] // 2
    ffn = (torch.nn.functional.silu(gu[..., :inter]) * gu[..., inter:]) @ f(w.down)
    residual = residual + ffn
    return residual, rms64(residual, f(next_gamma), eps)


def pack(x_pad, lens):
    return torch.cat([x_pad[b, :int(l)] for b, l in enumerate(lens)], 0)


@pytest.mark.parametrize("dtype,tol", [(torch.float32, 2e-4), (torch.float16, 3e-2)])
def test_prefill_layer_matches_float64_reference(isp, dtype, tol):
    from inferspore_amd.context_layer import BatchState, LayerWeights, context_decoder_layer
    print("[case] context layer %s" % dtype, flush=True)
    g = torch.Generator(device="cuda").manual_seed(3)
    nh, hs, inter, S = 2, 128, 512, 16
    H = nh * hs
    lens = [16, 5, 11]
    w = LayerWeights(H, inter, dtype, generator=g)
    next_gamma = (0.5 + torch.rand(H, device="cuda", generator=g)).to(dtype)
    st = BatchState(lens, S, nh, nh, hs, inter, max_seq_len=32, layers=2, dtype=dtype)
    res_pad = torch.randn((len(lens), S, H), device="cuda", generator=g).to(dtype)
    lens_t = torch.tensor(lens, device="cuda")
    residual = pack(res_pad, lens).contiguous()
    normed = residual.clone()
    isp.rmsnorm(normed, w.attn_norm, 1e-5)
    out = context_decoder_layer(normed, residual, w, st, 1, next_gamma)
    torch.cuda.synchronize()
    e_res, e_next = reference_layer64(res_pad.double(), lens_t, w, nh, hs, next_gamma)
    e_res, e_next = pack(e_res, lens), pack(e_next, lens)
    for got, exp, name in ((residual, e_res, "residual"), (out, e_next, "next input")):
        err = (got.double() - exp).abs().max().item()
        scale = exp.abs().max().item()
        assert err <= tol * scale, "%s: max error %g vs scale %g" % (name, err, scale)


def test_second_turn_uses_the_cached_keys(isp):
    """Prefill 9 tokens, then 7 more with history = 9: must equal one 16-token prefill."""
    from inferspore_amd.context_layer import BatchState, LayerWeights, context_decoder_layer
    g = torch.Generator(device="cuda").manual_seed(5)
    nh, hs, inter = 2, 128, 256
    H = nh * hs
    dtype = torch.float32
    w = LayerWeights(H, inter, dtype, generator=g)
    next_gamma = torch.ones(H, device="cuda", dtype=dtype)
    x = torch.randn((16, H), device="cuda", generator=g)

    def run(st, rows):
        residual = rows.clone()
        normed = rows.clone()
        isp.rmsnorm(normed, w.attn_norm, 1e-5)
        out = context_decoder_layer(normed, residual, w, st, 0, next_gamma)
        return residual, out

    whole = BatchState([16], 16, nh, nh, hs, inter, max_seq_len=32, layers=1, dtype=dtype)
    r_all, o_all = run(whole, x)
    first = BatchState([9], 16, nh, nh, hs, inter, max_seq_len=32, layers=1, dtype=dtype)
    r1, o1 = run(first, x[:9])
    second = BatchState([7], 16, nh, nh, hs, inter, max_seq_len=32, layers=1, dtype=dtype, history=[9])
    second.k_cache, second.v_cache = first.k_cache, first.v_cache     # the cache carries over
    r2, o2 = run(second, x[9:])
    torch.cuda.synchronize()
    for got, exp in ((torch.cat([r1, r2]), r_all), (torch.cat([o1, o2]), o_all)):
        assert (got - exp).abs().max().item() <= 2e-4 * exp.abs().max().item()
