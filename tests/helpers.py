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


def assert_f16_close(got, ref, what, max_mismatch_fraction=0.02):
    """fp16 criterion: every element within 2 ulp of the oracle and within 1e-2 absolute.

    Where one fp16 ulp is itself larger than 1e-2 (|value| >= 16) a single last-bit rounding
    difference cannot meet the absolute bound, so there the bound is one ulp.  The share of
    elements that differ at all is bounded as well, so a systematic error cannot hide in the
    tolerance."""
    got = np.asarray(got)
    ref = np.asarray(ref)
    assert got.dtype == np.float16 and ref.dtype == np.float16, (got.dtype, ref.dtype)
    assert got.shape == ref.shape, (got.shape, ref.shape)
    gnan, rnan = np.isnan(got), np.isnan(ref)
    assert np.array_equal(gnan, rnan), "%s: NaN pattern differs" % what
    ulp = np.where(rnan, 0, f16_ulp_distance(got, ref))
    with np.errstate(invalid="ignore"):
        err = np.abs(got.astype(np.float64) - ref.astype(np.float64))
    err = np.where(rnan | (got == ref), 0.0, err)
    bad = (ulp > F16_MAX_ULP) | ((err > F16_ATOL) & (ulp > 1))
    if bad.any():
        i = np.unravel_index(np.argmax(bad), bad.shape)
        raise AssertionError("%s: %d elements out of tolerance; first at %s got %r ref %r (ulp %d)" %
                             (what, int(bad.sum()), i, got[i], ref[i], int(ulp[i])))
    frac = float((ulp > 0).mean()) if ulp.size else 0.0
    assert frac <= max_mismatch_fraction, "%s: %.3f%% of elements differ from the oracle" % (
        what, 100 * frac)
    return int(ulp.max()) if ulp.size else 0, frac


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
