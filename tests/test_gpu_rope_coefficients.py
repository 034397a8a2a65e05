"""Every rotation coefficient of the QKV kernels, checked one pair at a time through the public ABI.

The one-vector-per-lane fp16 kernel fetches its divisor base^(2d/rot) from word d of the kernel's
argument block instead of through the parameter's name, so a change of the argument layout (or an
off-by-one in the word index) would hand lane d the divisor of another pair while still compiling.
The inputs here make that visible directly: with x[d] = 1 and x[d + rot/2] = 0 the rotated pair IS
(cos, sin) of position / divisor[d], so each output element names the divisor its lane used.  The
expected divisors come from the closed form in float64, not from the oracle, and neighbouring pairs'
divisors differ by 14 % at rot = 128 -- hundreds of fp16 ulp at the positions used."""
import numpy as np
import pytest
import torch

from inferspore_amd import capi


def say(msg):
    print("[case] " + msg, flush=True)


def expected_cos_sin(positions, rot, base):
    """[positions, rot/2] cos and sin of p / base^(2d/rot); the divisor and the quotient rounded to
    float32 as the kernels hold them (src/kernels/qkv_bias_and_RoPE.cu:7-13: inv_freq = t / powf(...))."""
    d = np.arange(rot // 2, dtype=np.float64)
    div = np.power(np.float64(base), 2.0 * d / rot).astype(np.float32)
    ang = (positions[:, None].astype(np.float32) / div[None, :]).astype(np.float32).astype(np.float64)
    return np.cos(ang), np.sin(ang), div


def fp16_bound(ref, positions, div):
    """Half an fp16 ulp of the value plus the effect of one float32 ulp of the divisor and of the
    quotient on the angle (the derivative of cos and sin is at most 1)."""
    ang = positions[:, None] / div[None, :].astype(np.float64)
    return 2.0 ** -11 * np.maximum(np.abs(ref), 2.0 ** -14) + 3 * ang * 2.0 ** -23 + 1e-6


@pytest.mark.gpu
@pytest.mark.parametrize("base", [10000.0, 500000.0])
@pytest.mark.parametrize("store", [1, 2, 3])
@pytest.mark.parametrize("with_bias", [False, True])
@pytest.mark.parametrize("append", [False, True])
@pytest.mark.parametrize("hs", [128, 64])
def test_lean_fp16_kernel_uses_divisor_d_for_pair_d(isp, base, store, with_bias, append, hs):
    say("coefficients hs=%d base=%g store=%d bias=%s append=%s" % (hs, base, store, with_bias, append))
    # 128-element heads in groups of 32, 64-element heads in groups of 8 with an odd token count: the shapes
    # that select the two kernels reading their divisors from the argument block
    batch, seq, hn, rot = (2, 40, 32, 128) if hs == 128 else (2, 39, 8, 64)
    hist = np.array([0, 977], np.int32)
    lens = np.array([seq, seq - (hs == 64)], np.int32)
    tokens = int(lens.sum())
    row = np.zeros(hs, np.float16)
    row[:rot // 2] = 1.0
    qkv = np.tile(row, (tokens, 3 * hn, 1))
    bias = None
    if with_bias:
        # the ones arrive through the bias: the kernel must add it before rotating
        bias = np.tile(row, (3 * hn, 1))
        qkv = np.zeros_like(qkv)
    d_qkv = torch.from_numpy(qkv).cuda()
    d_bias = None if bias is None else torch.from_numpy(bias).cuda()
    q = torch.full((batch, hn, seq, hs), -3.0, dtype=torch.float16, device="cuda")
    k = torch.full_like(q, -3.0)
    v = torch.full_like(q, -3.0)
    po = torch.zeros((batch, seq), dtype=torch.int32, device="cuda")
    po.view(-1)[lens[0]:tokens] = int(seq - lens[0])   # the second sequence starts at padded position seq
    d_hist, d_lens = torch.from_numpy(hist).cuda(), torch.from_numpy(lens).cuda()
    assert capi.lib().isp_tuning_set(capi.TUNE_QKV_STORE, store) >= 0
    try:
        if append:
            max_seq = 1024
            kc = torch.full((1, batch, hn, max_seq, hs), -3.0, dtype=torch.float16, device="cuda")
            vc = torch.full_like(kc, -3.0)
            isp.add_fused_qkv_bias_transpose_rope_and_append(q, k, v, kc, vc, 0, d_qkv, d_bias, po, d_hist, d_lens,
                                                             rot, base)
        else:
            isp.add_fused_qkv_bias_transpose_and_rope(q, k, v, d_qkv, d_bias, po, d_hist, d_lens, rot, base)
        torch.cuda.synchronize()
    finally:
        capi.lib().isp_tuning_set(capi.TUNE_QKV_STORE, 0)
    for b in range(batch):
        n = int(lens[b])
        positions = hist[b] + np.arange(n, dtype=np.int64)
        cos, sin, div = expected_cos_sin(positions, rot, base)
        outs = [("q", q[b, :, :n]), ("k", k[b, :, :n])]
        if append:
            outs.append(("k_cache", kc[0, b, :, hist[b]:hist[b] + n, :]))
        for what, t in outs:
            got = t.cpu().numpy().astype(np.float64)                      # [heads, seq, hs]
            for half, ref in ((got[:, :, :rot // 2], cos), (got[:, :, rot // 2:], sin)):
                err = np.abs(half - ref[None])
                bound = fp16_bound(ref, positions, div)[None]
                if (err > bound).any():
                    h, s, d = np.unravel_index(np.argmax(err - bound), err.shape)
                    raise AssertionError("%s batch %d head %d position %d pair %d: got %r, closed form %r" % (
                        what, b, h, positions[s], d, half[h, s, d], ref[s, d]))
        # v is copied, not rotated
        assert torch.equal(v[b, :, :n].cpu(), torch.from_numpy(np.tile(row, (hn, n, 1)))), "v must pass through unrotated"


def test_neighbouring_divisors_are_far_apart_in_this_test():
    """The premise of the test above: with pair d's divisor replaced by pair d+1's (or d-1's), some
    position in the tested range moves the result by far more than the bound allows."""
    positions = 977 + np.arange(40, dtype=np.int64)
    for base in (10000.0, 500000.0):
        cos, sin, div = expected_cos_sin(positions, 128, base)
        for shift in (1, -1):
            wrong = np.roll(div, shift)
            ang = (positions[:, None].astype(np.float32) / wrong[None, :]).astype(np.float64)
            excess = np.maximum(np.abs(np.cos(ang) - cos) / fp16_bound(cos, positions, div),
                                np.abs(np.sin(ang) - sin) / fp16_bound(sin, positions, div))
            inner = slice(1, -1)  # np.roll wraps the two end pairs; they are covered by the other shift
            assert (excess[:, inner].max(axis=0) > 20).all(), excess[:, inner].max(axis=0).min()
