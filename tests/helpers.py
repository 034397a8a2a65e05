"""Shared test helpers: seeded inputs of the benchmark configurations and the stated tolerances."""
import numpy as np

# Tolerances stated for this path:
#   bit-exact      : embedding gather, padding offsets, every scatter index
#   fp32 outputs   : |err| <= 1e-5 relative
#   fp16 outputs   : |err| <= 1e-2 absolute and <= 2 fp16 ulp (fp32 accumulation)
F32_RTOL = 1e-5
F16_ATOL = 1e-2
F16_MAX_ULP = 2


def f16_ordered(a):
    """Map float16 bit patterns to integers that are monotonic in the represented value."""
    u = np.ascontiguousarray(a, dtype=np.float16).view(np.uint16).astype(np.int32)
    return np.where(u & 0x8000, -(u & 0x7FFF), u)


def f16_ulp_distance(a, b):
    return np.abs(f16_ordered(a) - f16_ordered(b))


def f16_ulp_size(x):
    """Spacing of binary16 at magnitude |x| (2^-24 in the subnormal range)."""
    x = np.abs(np.asarray(x, dtype=np.float64))
    e = np.floor(np.log2(np.maximum(x, 2.0 ** -14)))
    return 2.0 ** (e - 10)


def assert_f16_close(got, ref, what, magnitude=None, max_mismatch_fraction=0.02):
    """fp16 criterion: every element within 2 fp16 ulp of the oracle and within 1e-2 absolute.

    Where one fp16 ulp is itself larger than 1e-2 (|value| >= 16) a single last-bit rounding
    difference cannot meet the absolute bound, so there the bound is one ulp.
    `magnitude` (broadcastable to the outputs) is the size of the operands a result was formed
    from when the result can cancel (a rotation: the radius of the rotated pair).  The fp32
    arithmetic behind both implementations is only accurate to ~2^-23 of that size, so the ulp is
    taken at max(|ref|, magnitude / 4096) -- i.e. the bound stays 2 ulp of the value itself unless the
    value is more than 4096 times smaller than what it was computed from.
    The share of elements that differ at all is bounded too, so a systematic error cannot hide in
    the tolerance."""
    got = np.asarray(got)
    ref = np.asarray(ref)
    assert got.dtype == np.float16 and ref.dtype == np.float16, (got.dtype, ref.dtype)
    assert got.shape == ref.shape, (got.shape, ref.shape)
    gnan, rnan = np.isnan(got), np.isnan(ref)
    assert np.array_equal(gnan, rnan), "%s: NaN pattern differs" % what
    same = (got == ref) | rnan
    with np.errstate(invalid="ignore"):
        err = np.where(same, 0.0, np.abs(got.astype(np.float64) - ref.astype(np.float64)))
    at = np.abs(ref.astype(np.float64))
    if magnitude is not None:
        at = np.maximum(at, np.asarray(magnitude, np.float64) / 4096.0)
    ulp = err / f16_ulp_size(at)
    bad = (ulp > F16_MAX_ULP) | ((err > F16_ATOL) & (ulp > 1))
    if bad.any():
        i = np.unravel_index(np.argmax(bad), bad.shape)
        raise AssertionError("%s: %d elements out of tolerance; first at %s got %r ref %r (%.2f ulp)" %
                             (what, int(bad.sum()), i, got[i], ref[i], float(ulp[i])))
    frac = float((~same).mean()) if same.size else 0.0
    assert frac <= max_mismatch_fraction, "%s: %.3f%% of elements differ from the oracle" % (
        what, 100 * frac)
    return (float(ulp.max()) if ulp.size else 0.0), frac


def assert_f32_close(got, ref, what, scale=None, rtol=F32_RTOL):
    """fp32 criterion: |got - ref| <= 1e-5 * scale, scale = |ref| unless the caller supplies the
    magnitude the result is relative to (e.g. the rotation radius for RoPE, where the result itself
    can cancel to zero)."""
    got = np.asarray(got, dtype=np.float64)
    ref = np.asarray(ref, dtype=np.float64)
    assert got.shape == ref.shape, (got.shape, ref.shape)
    scale = np.abs(ref) if scale is None else np.asarray(scale, dtype=np.float64)
    err = np.abs(got - ref)
    bad = err > rtol * scale + 1e-30
    if bad.any():
        i = np.unravel_index(np.argmax(err - rtol * scale), bad.shape)
        raise AssertionError("%s: %d elements out of tolerance; worst at %s got %r ref %r" %
                             (what, int(bad.sum()), i, got[i], ref[i]))
    return float((err / np.maximum(scale, 1e-30)).max()) if err.size else 0.0


# ------------------------------------------------------------------ seeded inputs (numpy PCG64)

def norm_inputs(tokens, hidden, dtype, seed=0, with_residual=True, with_bias=True):
    r = np.random.default_rng(seed)
    out = r.standard_normal((tokens, hidden)).astype(dtype)
    residual = r.standard_normal((tokens, hidden)).astype(dtype) if with_residual else None
    bias = (0.02 * r.standard_normal(hidden)).astype(dtype) if with_bias else None
    gamma = r.uniform(0.5, 1.5, hidden).astype(dtype)
    return residual, out, bias, gamma


def embedding_inputs(tokens, hidden, vocab, dtype, seed=0):
    r = np.random.default_rng(seed)
    table = (0.02 * r.standard_normal((vocab, hidden), dtype=np.float32)).astype(dtype)
    ids = r.integers(0, vocab, tokens, dtype=np.int32)
    return ids, table


def swiglu_inputs(tokens, inter, dtype, seed=0):
    r = np.random.default_rng(seed)
    return r.standard_normal((tokens, 2, inter), dtype=np.float32).astype(dtype)


def padding_offsets_np(lens, max_q_len):
    """Independent numpy statement of the padding offsets (cumulative padding before each sequence)."""
    lens = np.asarray(lens, dtype=np.int64)
    before = np.concatenate([[0], np.cumsum(max_q_len - lens)[:-1]]) if len(lens) else np.zeros(0)
    po = np.repeat(before, lens).astype(np.int32)
    cum = np.concatenate([[0], np.cumsum(lens)]).astype(np.int32)
    return po, cum


def qkv_inputs(batch, max_seq, head_num, kv_head_num, head_size, dtype, seed=0, min_len=None,
               with_bias=True):
    r = np.random.default_rng(seed)
    lo = max_seq // 2 if min_len is None else min_len
    lens = r.integers(lo, max_seq + 1, batch, dtype=np.int32)
    tokens = int(lens.sum())
    qkv = r.standard_normal((tokens, head_num + 2 * kv_head_num, head_size),
                            dtype=np.float32).astype(dtype)
    bias = ((0.02 * r.standard_normal((head_num + 2 * kv_head_num) * head_size)).astype(dtype)
            if with_bias else None)
    po, _ = padding_offsets_np(lens, max_seq)
    history = np.zeros(batch, np.int32)
    return lens, qkv, bias, po, history


def rope_pair_radius(qkv, bias):
    """[tokens, heads, head_size]: sqrt(x_d^2 + x_{d+half}^2) of the (biased) rotation pair each
    element belongs to -- the magnitude a rotated output is relative to."""
    x = np.asarray(qkv, np.float64)
    hs = x.shape[-1]
    if bias is not None:
        x = x + np.asarray(bias, np.float64).reshape(1, -1, hs)
    half = hs // 2
    rad = np.sqrt(x[..., :half] ** 2 + x[..., half:] ** 2)
    return np.concatenate([rad, rad], axis=-1)


def reference_mover_configurations():
    """The inputs of the reference's own programs for the two cache movers
    (tests/unittests/test_concat_kv.cu:16-75, test_repeat_kv.cu:15-56).  Those programs print their results
    for inspection and state no expected values; the expectations here follow from the kernels' definitions
    (concat_past_kv.cu:7-39, repeat_kv.cu:10-50) by hand."""
    # append: batch 1, 2 kv heads, 16 query positions of 8 elements, cache rows of 32 positions, source = 1,
    # 16 valid tokens behind a history of 1  =>  cache rows 1..16 of both heads become 1, nothing else changes
    k_src = np.ones((1, 2, 16, 8), np.float32)
    cache = np.full((1, 1, 2, 32, 8), -9.0, np.float32)
    expect_cache = cache.copy()
    expect_cache[0, 0, :, 1:17, :] = 1.0
    # broadcast: 2 layers, batch 1, 2 heads = 2 kv heads, cache rows of 4 positions of 2 elements holding their own
    # flat index, context 2, 2 key positions, layer 0  =>  head 0 reads elements 0..3, head 1 elements 8..11
    src_cache = np.arange(2 * 1 * 2 * 4 * 2, dtype=np.float32).reshape(2, 1, 2, 4, 2)
    expect_rep = np.array([[[[0, 1], [2, 3]], [[8, 9], [10, 11]]]], np.float32)
    return k_src, cache, expect_cache, src_cache, expect_rep
