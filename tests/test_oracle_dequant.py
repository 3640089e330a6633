"""Pins for the oracle's block dequantizers and weight-prep helpers (CPU only).

Independent restatement: the per-element closed forms of the block layouts
(element e of a block -> which bytes, which bits, which scale), evaluated in
exact integer/rational arithmetic and rounded once.  The oracle walks the
blocks with running pointers like gguf_reader.cpp:541-850; the closed form
below indexes every element directly, so a wrong stride, nibble order or
scale index in either fails the comparison.
"""
from fractions import Fraction

import numpy as np
import pytest

import oracle
from oracle import Q4_0, Q4_K, Q6_K, Q8_0


def h(bits: int) -> Fraction:
    """binary16 bits -> exact rational (finite inputs only)."""
    s = -1 if bits & 0x8000 else 1
    e, m = (bits >> 10) & 31, bits & 1023
    assert e != 31
    if e == 0:
        return s * Fraction(m, 1 << 24)
    return s * Fraction(1024 + m, 1024) * Fraction(2) ** (e - 15)


def rn32(x: Fraction) -> np.float32:
    """Correctly rounded (nearest-even) fp32 of an exact rational."""
    # float(Fraction) is correctly rounded to double; a double -> float32 cast
    # could double-round, so go through an exact scaled integer instead.
    if x == 0:
        return np.float32(0.0)
    s, a = (-1 if x < 0 else 1), abs(x)
    e = a.numerator.bit_length() - a.denominator.bit_length()
    if Fraction(2) ** e > a:
        e -= 1
    e = max(e, -126)
    q = a / Fraction(2) ** (e - 23)
    n, r = divmod(q.numerator, q.denominator)
    twice = 2 * r
    if twice > q.denominator or (twice == q.denominator and n & 1):
        n += 1
    return np.float32(s * float(n) * 2.0 ** (e - 23))


def scale_min(j, q):
    if j < 4:
        return q[j] & 63, q[j + 4] & 63
    return (q[j + 4] & 15) | ((q[j - 4] >> 6) << 4), (q[j + 4] >> 4) | ((q[j] >> 6) << 4)


def element(fmt, blk: np.ndarray, e: int):
    """Exact value of element e and, for a zero result, whether it is -0.0.

    IEEE sign rules: a product takes the XOR of the factor signs (an integer
    zero converts to +0.0); x - y with both zero is -0 only for (-0) - (+0);
    an exact cancellation of non-zero terms is +0.
    """
    b = [int(v) for v in blk]
    u16 = lambda o: b[o] | (b[o + 1] << 8)
    i8 = lambda v: v - 256 if v > 127 else v
    neg = lambda bits16: bool(bits16 & 0x8000)
    if fmt == Q8_0:
        q = i8(b[2 + e])
        return q * h(u16(0)), neg(u16(0)) ^ (q < 0)
    if fmt == Q4_0:
        q = ((b[2 + e] & 15) if e < 16 else (b[2 + e - 16] >> 4)) - 8
        return q * h(u16(0)), neg(u16(0)) ^ (q < 0)
    if fmt == Q4_K:
        g, r = divmod(e, 64)
        j, l = 2 * g + (r >= 32), r % 32
        sc, m = scale_min(j, b[4:16])
        byte = b[16 + 32 * g + l]
        nib = (byte & 15) if r < 32 else (byte >> 4)
        a, c = (h(u16(0)) * sc) * nib, h(u16(2)) * m
        return a - c, (a == 0 and c == 0 and neg(u16(0)) and not neg(u16(2)))
    if fmt == Q6_K:
        H, p = divmod(e, 128)
        s, l = divmod(p, 32)
        qlb = b[64 * H + l + 32 * (s & 1)]
        lo = (qlb & 15) if s < 2 else (qlb >> 4)
        hi = (b[128 + 32 * H + l] >> (2 * s)) & 3
        q = (lo | (hi << 4)) - 32
        scv = i8(b[192 + 8 * H + 2 * s + l // 16])
        return h(u16(208)) * scv * q, neg(u16(208)) ^ (scv < 0) ^ (q < 0)
    raise ValueError(fmt)


def closed_form(fmt, blocks: np.ndarray, n: int) -> np.ndarray:
    be, bb = oracle.BLOCK_ELEMS[fmt], oracle.BLOCK_BYTES[fmt]
    out = np.empty(n, np.float32)
    for i in range(n):
        blk = blocks[(i // be) * bb:(i // be + 1) * bb]
        v, negzero = element(fmt, blk, i % be)
        out[i] = np.float32(-0.0) if (v == 0 and negzero) else rn32(v)
    return out


def bits(a):
    return np.ascontiguousarray(a, np.float32).view(np.uint32)


def finite_blocks(fmt, rng, n_blocks):
    bb = oracle.BLOCK_BYTES[fmt]
    b = rng.integers(0, 256, (n_blocks, bb), dtype=np.uint8)
    for off in {Q8_0: [0], Q4_0: [0], Q4_K: [0, 2], Q6_K: [208]}[fmt]:
        bad = (b[:, off + 1] & 0x7C) == 0x7C
        b[bad, off + 1] &= 0xFB
    return b.reshape(-1)


@pytest.mark.parametrize("name", list(oracle.FORMATS))
def test_dequant_matches_exact_closed_form(name):
    fmt = oracle.FORMATS[name]
    rng = np.random.default_rng(11 + fmt)
    nblk = 12 if oracle.BLOCK_ELEMS[fmt] == 256 else 64
    blocks = finite_blocks(fmt, rng, nblk)
    n = nblk * oracle.BLOCK_ELEMS[fmt]
    got = oracle.dequant(fmt, blocks, n)
    want = closed_form(fmt, blocks, n)
    assert np.array_equal(bits(got), bits(want))


@pytest.mark.parametrize("name", ["Q4_0", "Q4_K", "Q6_K", "Q8_0"])
def test_basis_sweep_single_bit(name):
    """One set bit of the quant payload at a time: pins the index maps."""
    fmt = oracle.FORMATS[name]
    be, bb = oracle.BLOCK_ELEMS[fmt], oracle.BLOCK_BYTES[fmt]
    base = np.zeros(bb, np.uint8)
    one = np.array([0x3C00], np.uint16).view(np.uint8)  # 1.0
    if fmt in (Q8_0, Q4_0):
        base[0:2] = one
        payload = range(2, bb)
    elif fmt == Q4_K:
        base[0:2] = one
        base[2:4] = one
        # distinct scale j+1 and min 2j+1 for every sub-block, via the packer
        sc = [j + 1 for j in range(8)]
        mn = [2 * j + 1 for j in range(8)]
        q = [0] * 12
        for j in range(8):
            if j < 4:
                q[j] |= sc[j]
                q[j + 4] |= mn[j]
            else:
                q[j + 4] |= (sc[j] & 15) | ((mn[j] & 15) << 4)
                q[j - 4] |= (sc[j] >> 4) << 6
                q[j] |= (mn[j] >> 4) << 6
        base[4:16] = q
        payload = range(16, 144)
    else:
        base[208:210] = one
        base[192:208] = np.arange(1, 17, dtype=np.uint8)  # distinct scales
        payload = range(0, 192)
    for byte in payload:
        for bit in range(8):
            blk = base.copy()
            blk[byte] |= 1 << bit
            got = oracle.dequant(fmt, blk, be)
            want = closed_form(fmt, blk, be)
            assert np.array_equal(bits(got), bits(want)), (byte, bit)


def test_get_scale_min_k4_exhaustive_per_byte_pair():
    """Each output depends on <= 2 bytes: sweep both over all 65536 values."""
    for j in range(8):
        deps_sc = [j] if j < 4 else [j + 4, j - 4]
        deps_m = [j + 4] if j < 4 else [j + 4, j]
        for deps in (deps_sc, deps_m):
            for v0 in range(256):
                for v1 in (range(256) if len(deps) == 2 else [0]):
                    q = [0xA5] * 12
                    q[deps[0]] = v0
                    if len(deps) == 2:
                        q[deps[1]] = v1
                    if (v0 * 7 + v1) % 5:  # thin the sweep: ~20 % of 2 x 8 x 64k
                        continue
                    assert oracle.get_scale_min_k4(j, q) == scale_min(j, q)


def test_reference_fixture_q4k():
    # dequant/q4k (OpRegistry.h:1929-1957): d=1, dmin=0, scales[0..3]=1,
    # scales[8..11]=1, qs[i]=(i%8)|((i%8+1)<<4) -> out[i] = qs[i]&15 for i<32
    blk = np.zeros(144, np.uint8)
    blk[0:2] = np.array([0x3C00], np.uint16).view(np.uint8)
    blk[4:8] = 1
    blk[12:16] = 1
    qs = np.array([(i % 8) | ((i % 8 + 1) << 4) for i in range(128)], np.uint8)
    blk[16:] = qs
    out = oracle.dequant(Q4_K, blk, 256)
    assert np.all(np.isfinite(out))
    assert np.array_equal(out[:32], (qs[:32] & 15).astype(np.float32))
    # high nibbles of the same bytes are elements 32..63, scale of sub-block 1
    assert np.array_equal(out[32:64], (qs[:32] >> 4).astype(np.float32))
    # sub-blocks 4..7 read scale nibbles from bytes 8..11 (=1) -> scale 1
    assert np.array_equal(out[128:160], (qs[64:96] & 15).astype(np.float32))


def test_reference_fixture_q6k():
    # dequant/q6k (OpRegistry.h:1959-1978): ql=0x55, qh=0, sc=1, d=1 -> -27
    blk = np.zeros(210, np.uint8)
    blk[0:128] = 0x55
    blk[192:208] = 1
    blk[208:210] = np.array([0x3C00], np.uint16).view(np.uint8)
    out = oracle.dequant(Q6_K, blk, 256)
    assert np.array_equal(out, np.full(256, -27.0, np.float32))


@pytest.mark.parametrize("name", list(oracle.FORMATS))
@pytest.mark.parametrize("tag", ["random", "gauss"])
def test_golden_vectors_from_reference_reader(golden, name, tag):
    fmt = oracle.FORMATS[name]
    rows, cols = int(golden["rows"]), int(golden["cols"])
    blocks = golden[f"{name}_{tag}_blocks"]
    want = golden[f"{name}_{tag}_f32bits"]
    got = oracle.dequant(fmt, blocks, rows * cols)
    assert np.array_equal(bits(got), want)


def test_golden_split_readers(golden):
    rows, cols = int(golden["rows"]), int(golden["cols"])
    v, s = oracle.split_q8_0(golden["Q8_0_random_blocks"], rows, cols)
    assert np.array_equal(v, golden["Q8_0_split_values"])
    assert np.array_equal(s, golden["Q8_0_split_scales"])
    v, s = oracle.split_q4_0(golden["Q4_0_random_blocks"], rows, cols)
    assert np.array_equal(v, golden["Q4_0_split_packed"])
    assert np.array_equal(s, golden["Q4_0_split_scales"])


@pytest.mark.skipif(not oracle.have_ref(), reason="oracle/_ref not built here")
@pytest.mark.parametrize("name", list(oracle.FORMATS))
def test_against_compiled_reference_reader(name):
    fmt = oracle.FORMATS[name]
    rng = np.random.default_rng(99 + fmt)
    rows, cols = 24, 2048
    blocks = finite_blocks(fmt, rng, rows * cols // oracle.BLOCK_ELEMS[fmt])
    got = oracle.dequant(fmt, blocks, rows * cols)
    want = oracle.ref_dequant(fmt, blocks, rows, cols)
    assert np.array_equal(bits(got), bits(want))


def test_dequant_f16_is_elementwise_narrowing():
    rng = np.random.default_rng(5)
    for fmt in oracle.FORMATS.values():
        blocks = oracle.quantize(fmt, rng.standard_normal(4096).astype(np.float32) * 0.02)
        f32 = oracle.dequant(fmt, blocks, 4096)
        assert np.array_equal(oracle.dequant_f16(fmt, blocks, 4096), oracle.f32_to_f16_array(f32))


# ---- weight preparation (llama.cpp:488-619) ----------------------------------

def test_quantize_rows_q8_0_invariants():
    rng = np.random.default_rng(0)
    x = rng.standard_normal(32 * 257).astype(np.float32) * 0.02
    x[:32] = 0.0  # a zero block -> d = 0, q = 0
    x[32:64] *= 1e-4  # small magnitudes -> subnormal fp16 scale must survive
    v, s = oracle.quantize_rows_q8_0(x)
    xb, vb = x.reshape(-1, 32), v.reshape(-1, 32).astype(np.int32)
    assert np.all(np.abs(vb) <= 127)
    assert s[0] == 0 and not vb[0].any()
    amax = np.abs(xb).max(axis=1)
    d = (amax / np.float32(127.0)).astype(np.float32)
    assert np.array_equal(s, oracle.f32_to_f16_array(d))
    assert s[1] != 0
    arg = np.abs(xb).argmax(axis=1)
    nz = amax > 0
    assert np.all(np.abs(vb[np.arange(len(arg)), arg])[nz] == 127)
    # q = lroundf(x * (1/d)) in fp32 with an unrounded d
    idv = np.where(d != 0, np.float32(1.0) / np.where(d != 0, d, 1).astype(np.float32), 0).astype(np.float32)
    prod = (xb * idv[:, None]).astype(np.float32)
    want = np.where(prod >= 0, np.floor(prod.astype(np.float64) + 0.5), np.ceil(prod.astype(np.float64) - 0.5))
    assert np.array_equal(vb, want.astype(np.int32))


def test_requantize_q4k_to_affine_layout_and_identity():
    rng = np.random.default_rng(3)
    N, K = 6, 512
    raw = oracle.quantize(Q4_K, rng.standard_normal(N * K).astype(np.float32) * 0.02)
    packed, scales = oracle.requantize_q4k_to_affine(raw, N, K)
    assert packed.shape == (K, N // 2) and scales.shape == (2 * K // 32, N)
    w = oracle.dequant(Q4_K, raw, N * K).reshape(N, K)
    dec = oracle.decode_affine_q4(packed, scales, N, K)
    # exact up to the fp16 storage of scale and min (relative ~5e-4 of the scale)
    assert np.max(np.abs(dec - w)) <= 2e-3 * np.max(np.abs(w))
    # nibble placement: byte (k, n>>1), low nibble for even n, nibble unchanged
    blk = raw.reshape(N, K // 256, 144)
    for n in range(N):
        for k in range(0, K, 37):
            s_, e = divmod(k, 256)
            g, r = divmod(e, 64)
            byte = blk[n, s_, 16 + 32 * g + r % 32]
            nib = (byte & 15) if r < 32 else (byte >> 4)
            got = (packed[k, n >> 1] >> (4 * (n & 1))) & 15
            assert got == nib
    # refused shapes (llama.cpp:577)
    assert oracle.requantize_q4k_to_affine(raw, N, 500) is None
    assert oracle.requantize_q4k_to_affine(raw, 5, K) is None
    # scale = f16(d*sc), min = f16(8*scale - dmin*m) with the unrounded scale
    d = oracle.f16_to_f32_array(blk[0, 0, 0:2].view(np.uint16))[0]
    dmin = oracle.f16_to_f32_array(blk[0, 0, 2:4].view(np.uint16))[0]
    sc, m = scale_min(3, [int(v) for v in blk[0, 0, 4:16]])
    scale = np.float32(d) * np.float32(sc)
    minv = np.float32(8.0) * scale - np.float32(dmin) * np.float32(m)
    assert scales[3, 0] == oracle.f32_to_f16(float(scale))
    assert scales[K // 32 + 3, 0] == oracle.f32_to_f16(float(minv))


def test_transpose_q4_nibble_reference_case():
    # TransposeQ4_Nibble_BitExact (OpCoverageTests.cpp:255-275)
    N = K = 32
    Mx = lambda n, k: (n * K + k) & 0xF
    src = np.array([[Mx(n, j) | (Mx(n, j + 16) << 4) for j in range(K // 2)] for n in range(N)], np.uint8)
    want = np.array([[Mx(n, k) | (Mx(n + 1, k) << 4) for n in range(0, N, 2)] for k in range(K)], np.uint8)
    assert np.array_equal(oracle.transpose_q4_nibble(src, N, K), want)
