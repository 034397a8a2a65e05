"""Pins the oracle's own binary16 <-> binary32 conversion against numpy's, exhaustively."""
import numpy as np


def test_h2f_all_65536_patterns(oracle):
    h = np.arange(65536, dtype=np.uint16)
    got = oracle.h2f(h)
    ref = h.view(np.float16).astype(np.float32)
    nan = np.isnan(ref)
    assert np.array_equal(np.isnan(got), nan)
    assert np.array_equal(got.view(np.uint32)[~nan], ref.view(np.uint32)[~nan])


def _check_f2h(oracle, x):
    x = np.ascontiguousarray(x, np.float32)
    got = oracle.f2h(x)
    with np.errstate(over="ignore"):
        ref = x.astype(np.float16).view(np.uint16)
    nan = np.isnan(x)
    assert np.array_equal(got[~nan], ref[~nan])
    assert np.all(np.isnan(got[nan].view(np.float16)))


def test_f2h_random_bit_patterns(oracle):
    r = np.random.default_rng(1)
    _check_f2h(oracle, r.integers(0, 2**32, 2_000_000, dtype=np.uint64).astype(np.uint32).view(np.float32))


def test_f2h_every_rounding_boundary(oracle):
    # the midpoint between every pair of adjacent finite halves, and its fp32 neighbours either side
    h = np.arange(0, 0x7C00, dtype=np.uint16)
    lo = h.view(np.float16).astype(np.float64)
    hi = (h + 1).astype(np.uint16).view(np.float16).astype(np.float64)
    hi[-1] = 65536.0  # the value that would follow 65504
    mid = ((lo + hi) / 2).astype(np.float32)
    pts = np.concatenate([mid, np.nextafter(mid, np.float32(np.inf)), np.nextafter(mid, np.float32(-np.inf)),
                          lo.astype(np.float32), np.float32([0.0, 65504, 65519.99, 65520, 1e9, np.inf])])
    _check_f2h(oracle, np.concatenate([pts, -pts]))


def test_round_trip(oracle):
    h = np.arange(65536, dtype=np.uint16)
    ok = ~np.isnan(h.view(np.float16))
    assert np.array_equal(oracle.f2h(oracle.h2f(h))[ok], h[ok])
