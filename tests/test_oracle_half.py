"""Pins for the oracle's half-precision conversions (CPU only).

f16_to_f32 (gguf_reader.cpp:515-539) is checked exhaustively against IEEE
binary16 semantics (numpy.float16).  f32_to_f16 (llama.cpp:445-482) is checked
against an arithmetic closed form -- "round half away from zero to binary16,
subnormals kept, |x| >= 65520 and NaN -> +-Inf" -- that shares no code with
the bit-twiddling restatement.
"""
import os

import numpy as np
import pytest

import oracle


def closed_form_f32_to_f16(x32: np.ndarray) -> np.ndarray:
    """Round-half-away-from-zero fp32 -> binary16 bits, in float64 arithmetic."""
    with np.errstate(invalid="ignore"):
        x = x32.astype(np.float64)
    sign = (x32.view(np.uint32) >> 16).astype(np.uint16) & np.uint16(0x8000)
    a = np.abs(x)
    nan = np.isnan(a)
    a = np.where(nan, np.inf, a)
    with np.errstate(divide="ignore", invalid="ignore", over="ignore"):
        e = np.floor(np.log2(np.where(a > 0, a, 1.0)))
        # log2 can be off by one next to powers of two: fix with exact tests
        e = np.where(np.ldexp(1.0, e.astype(np.int64)) > a, e - 1, e)
        e = np.where(np.ldexp(1.0, (e + 1).astype(np.int64)) <= a, e + 1, e)
        e = np.maximum(e, -14.0)  # subnormal range shares the ulp 2^-24
        ulp = np.ldexp(1.0, (e - 10).astype(np.int64))
        q = np.floor(a / ulp + 0.5)  # exact: a/ulp has < 2^35 magnitude, 24 bits
        val = q * ulp
    val = np.where(np.isinf(a) | (val >= 65520.0), np.inf, val)
    bits = val.astype(np.float16).view(np.uint16)  # val is exactly representable
    return bits | sign


def test_f16_to_f32_exhaustive_vs_ieee():
    h = np.arange(65536, dtype=np.uint16)
    got = oracle.f16_to_f32_array(h)
    want = h.view(np.float16).astype(np.float32)
    isnan = np.isnan(want)
    assert np.array_equal(got.view(np.uint32)[~isnan], want.view(np.uint32)[~isnan])
    # every NaN input gives the one canonical quiet NaN constant
    assert np.all(got.view(np.uint32)[isnan] == np.float32(np.nan).view(np.uint32))
    assert isnan.sum() == 2 * 1023


def test_runner_f16_to_f32_matches_and_keeps_nan_payload():
    h = np.arange(65536, dtype=np.uint16)
    got = oracle.f16_to_f32_array(h, runner=True)
    want = h.view(np.float16).astype(np.float32)
    isnan = np.isnan(want)
    assert np.array_equal(got.view(np.uint32)[~isnan], want.view(np.uint32)[~isnan])
    # llama.cpp:533-534: sign | 0x7F800000 | man << 13
    hn = h[isnan].astype(np.uint32)
    expect = ((hn & 0x8000) << 16) | 0x7F800000 | ((hn & 0x3FF) << 13)
    assert np.array_equal(got.view(np.uint32)[isnan], expect)


def _interesting_f32() -> np.ndarray:
    rng = np.random.default_rng(7)
    parts = []
    # every exact fp16 value (round trip must be the identity)
    parts.append(np.arange(65536, dtype=np.uint16).view(np.float16).astype(np.float32))
    # every tie point in the normal range, and its neighbours
    exps = np.arange(103, 144, dtype=np.uint32)  # 2^-24 .. 2^16
    mant = (np.arange(1024, dtype=np.uint32) << 13) | 0x1000
    tie = ((exps[:, None] << 23) | mant[None, :]).reshape(-1)
    for d in (-1, 0, 1):
        parts.append((tie + np.uint32(d % (1 << 32))).astype(np.uint32).view(np.float32))
    # subnormal-range ties: shift 14..25 -> significand low bits = 1 << (shift-1)
    sub = []
    for e in range(100, 114):
        shift = 126 - e
        if shift < 1 or shift > 26:
            continue
        for hi in range(0, 1 << max(0, 24 - shift), max(1, (1 << max(0, 24 - shift)) // 64)):
            sig = (hi << shift) | (1 << (shift - 1)) if shift <= 24 else 0
            sig |= 0x800000
            for d in (-1, 0, 1):
                sub.append(((e << 23) | ((sig + d) & 0x7FFFFF)))
    parts.append(np.array(sub, dtype=np.uint32).view(np.float32))
    # boundaries: overflow threshold, smallest subnormal, zeros, inf, nan
    special = np.array([65504.0, 65519.99, 65520.0, 65536.0, 1e30, 2.0 ** -24,
                        2.0 ** -25, np.nextafter(np.float32(2.0 ** -25), np.float32(1)),
                        np.nextafter(np.float32(2.0 ** -25), np.float32(0)),
                        2.0 ** -14, 0.0, np.inf], dtype=np.float32)
    parts.append(special)
    # random bit patterns, biased to the fp16 exponent range
    r = rng.integers(0, 1 << 32, 1 << 20, dtype=np.uint64).astype(np.uint32)
    parts.append(r.view(np.float32))
    rr = (rng.integers(95, 146, 1 << 20, dtype=np.uint64).astype(np.uint32) << 23) | \
         rng.integers(0, 1 << 23, 1 << 20, dtype=np.uint64).astype(np.uint32)
    parts.append(rr.view(np.float32))
    x = np.concatenate(parts)
    return np.concatenate([x, -x])


def test_f32_to_f16_vs_closed_form():
    x = _interesting_f32()
    got = oracle.f32_to_f16_array(x)
    want = closed_form_f32_to_f16(x)
    bad = np.nonzero(got != want)[0]
    assert bad.size == 0, (x[bad[:5]], got[bad[:5]], want[bad[:5]])


def test_f32_to_f16_documented_deviations():
    # NaN clamps to +-Inf (llama.cpp:467-468); ties go away from zero.
    assert oracle.f32_to_f16(float("nan")) & 0x7FFF == 0x7C00
    one_plus_half_ulp = np.uint32(0x3F801000).view(np.float32)  # 1 + 2^-11
    assert oracle.f32_to_f16(float(one_plus_half_ulp)) == 0x3C01  # RNE would give 0x3C00
    assert oracle.f32_to_f16(2.0 ** -25) == 0x0001  # RNE would give 0
    assert oracle.f32_to_f16(-(2.0 ** -25)) == 0x8001
    assert oracle.f32_to_f16(65520.0) == 0x7C00
    assert oracle.f32_to_f16(65519.0) == 0x7BFF


def test_round_trip_identity():
    h = np.arange(65536, dtype=np.uint16)
    f = oracle.f16_to_f32_array(h)
    ok = ~np.isnan(f)
    assert np.array_equal(oracle.f32_to_f16_array(f)[ok], h[ok])


def test_harness_truncating_helper():
    # OpRefs.h:164-177 truncates: 0.15f -> one ulp below round-to-nearest
    assert oracle.harness_f32_to_f16(1.0) == 0x3C00
    assert oracle.harness_f32_to_f16(0.1) == 0x2E66
    rne = int(np.float16(np.float32(0.15)).view(np.uint16))
    assert oracle.harness_f32_to_f16(0.15) == rne - 1
    assert oracle.harness_f32_to_f16(1e-6) == 0  # flushes subnormals


@pytest.mark.slow
@pytest.mark.skipif(not os.environ.get("CUT_SLOW"), reason="exhaustive 2^32 sweep: set CUT_SLOW=1")
def test_f32_to_f16_exhaustive():
    for hi in range(0, 1 << 16, 1 << 4):
        u = (np.arange(1 << 20, dtype=np.uint64) + (hi << 16)).astype(np.uint32)
        x = u.view(np.float32)
        assert np.array_equal(oracle.f32_to_f16_array(x), closed_form_f32_to_f16(x)), hi
