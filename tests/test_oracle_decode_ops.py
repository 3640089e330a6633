"""Pins the oracle's restatements of the operators between the matmuls of a
decode step (RMSNorm.cu, FusedRoPEKVWrite.cu, Attention.cu of the reference)
with closed forms and independent arithmetic, not with the oracle's own formula."""
import numpy as np

import oracle


def test_rmsnorm_closed_forms():
    w = np.linspace(0.5, 1.5, 64).astype(np.float32)
    # constant row c: out = c / sqrt(c^2 + eps) * w
    for c, eps in ((2.0, 1e-5), (-3.0, 0.25), (1e-3, 1e-6)):
        got = oracle.rmsnorm(np.full(64, c, np.float32), w, eps)
        want = c / np.sqrt(np.float64(c) ** 2 + eps) * w.astype(np.float64)
        np.testing.assert_allclose(got, want, rtol=3e-7)
    # eps = 0: invariant to scaling of x; output has unit mean square when weight = 1
    rng = np.random.default_rng(0)
    x = rng.standard_normal((3, 96)).astype(np.float32)
    a = oracle.rmsnorm(x, np.ones(96, np.float32), 0.0)
    b = oracle.rmsnorm(x * np.float32(8.0), np.ones(96, np.float32), 0.0)   # power of two: exact scaling
    np.testing.assert_array_equal(a, b)
    np.testing.assert_allclose((a.astype(np.float64) ** 2).mean(axis=1), 1.0, rtol=1e-6)
    # rows are independent
    np.testing.assert_array_equal(oracle.rmsnorm(x[1], np.ones(96, np.float32), 1e-5), oracle.rmsnorm(x, np.ones(96, np.float32), 1e-5)[1])


def _tables(max_pos, head_dim, theta=10000.0):
    half = head_dim // 2
    inv = 1.0 / theta ** (np.arange(half, dtype=np.float64) * 2 / head_dim)
    ang = np.arange(max_pos, dtype=np.float64)[:, None] * inv[None]
    return np.cos(ang).astype(np.float32), np.sin(ang).astype(np.float32), ang


def test_rope_is_a_complex_rotation_of_half_split_pairs():
    hd, nq, nkv, pos = 16, 3, 2, 5
    cos_t, sin_t, ang = _tables(8, hd)
    rng = np.random.default_rng(1)
    q = rng.standard_normal(nq * hd).astype(np.float32)
    k = rng.standard_normal(nkv * hd).astype(np.float32)
    v = rng.standard_normal(nkv * hd).astype(np.float32)
    kc = np.zeros((8, nkv * hd), np.uint16)
    vc = np.zeros((8, nkv * hd), np.uint16)
    q_rot = oracle.rope_kv_write(q, k, v, pos, cos_t, sin_t, hd, kc, vc)
    # element d pairs with d + hd/2: (x0 + i x1) * exp(i * angle)
    for src, got in ((q, q_rot), (k, oracle.f16_to_f32_array(kc[pos]))):
        z = src.reshape(-1, 2, hd // 2).astype(np.float64)
        zc = (z[:, 0] + 1j * z[:, 1]) * np.exp(1j * ang[pos])[None]
        want = np.stack([zc.real, zc.imag], axis=1).reshape(-1)
        tol = 1e-6 if got is q_rot else 1e-3   # the cache holds fp16
        np.testing.assert_allclose(got, want, rtol=tol, atol=tol)
    # v is stored unrotated, rounded to fp16 (nearest even); other cache rows untouched
    np.testing.assert_array_equal(vc[pos], v.astype(np.float16).view(np.uint16))
    assert not kc[:pos].any() and not kc[pos + 1:].any()
    # position 0 is the identity
    q0 = oracle.rope_kv_write(q, k, v, 0, cos_t, sin_t, hd, kc, vc)
    np.testing.assert_array_equal(q0, q)
    # rotation keeps the norm of every head
    np.testing.assert_allclose(np.linalg.norm(q_rot.reshape(nq, hd), axis=1), np.linalg.norm(q.reshape(nq, hd), axis=1), rtol=1e-6)


def test_kv_store_rounds_to_nearest_even():
    # exact ties between adjacent fp16 values and ordinary values, against numpy's conversion
    h = np.arange(0x0001, 0x7BFF, 37, dtype=np.uint16)
    lo, hi = oracle.f16_to_f32_array(h).astype(np.float64), oracle.f16_to_f32_array(h + 1).astype(np.float64)
    ties = ((lo + hi) / 2).astype(np.float32)
    vals = np.concatenate([ties, -ties, np.random.default_rng(2).standard_normal(4096).astype(np.float32)])
    kc = np.zeros((1, vals.size), np.uint16)
    vc = np.zeros((1, vals.size), np.uint16)
    cos_t, sin_t = np.ones((1, vals.size // 2), np.float32), np.zeros((1, vals.size // 2), np.float32)
    oracle.rope_kv_write(np.zeros(vals.size, np.float32), np.zeros(vals.size, np.float32), vals, 0, cos_t, sin_t, vals.size, kc, vc)
    np.testing.assert_array_equal(vc[0], vals.astype(np.float16).view(np.uint16))


def _softmax_attention(q, K, V, scale):   # float64 numpy, one head
    s = K.astype(np.float64) @ q.astype(np.float64) * scale
    p = np.exp(s - s.max())
    return (p / p.sum()) @ V.astype(np.float64)


def test_attention_special_cases_and_numpy_softmax():
    nh, nkv, hd, T = 4, 2, 8, 11
    rng = np.random.default_rng(3)
    q = rng.standard_normal(nh * hd).astype(np.float32)
    K = rng.standard_normal((T, nkv * hd)).astype(np.float16)
    V = rng.standard_normal((T, nkv * hd)).astype(np.float16)
    kc, vc = K.view(np.uint16), V.view(np.uint16)
    scale = 1 / np.sqrt(hd)
    got = oracle.attention_decode(q, kc, vc, T, nh, nkv, hd, scale).reshape(nh, hd)
    for h in range(nh):
        kvh = h // (nh // nkv)
        want = _softmax_attention(q[h * hd:(h + 1) * hd], K[:, kvh * hd:(kvh + 1) * hd].astype(np.float32),
                                  V[:, kvh * hd:(kvh + 1) * hd].astype(np.float32), scale)
        np.testing.assert_allclose(got[h], want, rtol=1e-6, atol=1e-7)
    # one cached position: the output is that V row
    one = oracle.attention_decode(q, kc, vc, 1, nh, nkv, hd, scale).reshape(nh, hd)
    np.testing.assert_array_equal(one[0], V[0, :hd].astype(np.float32))
    np.testing.assert_array_equal(one[3], V[0, hd:].astype(np.float32))
    # identical keys: uniform weights, the output is the mean of V
    Ku = np.repeat(K[:1], T, axis=0)
    uni = oracle.attention_decode(q, Ku.view(np.uint16), vc, T, nh, nkv, hd, scale).reshape(nh, hd)
    np.testing.assert_allclose(uni[0], V[:, :hd].astype(np.float64).mean(axis=0), rtol=1e-6, atol=1e-7)
    # a dominating score selects its V row; only the first seq_len rows are read
    Kd = np.zeros_like(K)
    Kd[7, :hd] = (q[:hd] * 50).astype(np.float16)
    dom = oracle.attention_decode(q, Kd.view(np.uint16), vc, T, nh, nkv, hd, 1.0).reshape(nh, hd)
    np.testing.assert_allclose(dom[0], V[7, :hd].astype(np.float32), rtol=1e-5, atol=1e-6)
    short = oracle.attention_decode(q, kc, vc, 5, nh, nkv, hd, scale)
    np.testing.assert_array_equal(short, oracle.attention_decode(q, kc[:5].copy(), vc[:5].copy(), 5, nh, nkv, hd, scale))


def test_silu_mul():
    g = np.array([0.0, 1.0, -1.0, 20.0, -20.0, 3.5], np.float32)
    u = np.array([2.0, 2.0, 2.0, 0.5, 0.5, -1.0], np.float32)
    got = oracle.silu_mul(np.concatenate([g, u]))
    want = g.astype(np.float64) / (1 + np.exp(-g.astype(np.float64))) * u
    np.testing.assert_allclose(got, want, rtol=2e-7, atol=1e-12)
    assert got[0] == 0.0 and abs(got[3] - 10.0) < 1e-6


# ---- embedding gather and repetition penalty ---------------------------------------------------------------

def test_embedding_col_int8_equals_dequant_of_the_gguf_row():
    """EmbeddingCol on the loader's separated Q8_0 tensors (values [N, K] and scales [N, K/32] transposed to the
    column-wise [K, N] / [K/32, N] form the GPU upload produces) gathers exactly the dequantized GGUF row: the
    pinned dequantizer fixes every index of the column-wise addressing (d * vocabStride + t, (d >> 5) * scaleStride + t)."""
    vocab, dim = 40, 96
    rng = np.random.default_rng(5)
    blocks = oracle.quantize(oracle.Q8_0, (rng.standard_normal(vocab * dim) * 0.05).astype(np.float32))
    vals, scales = oracle.split_q8_0(blocks, vocab, dim)           # [vocab, dim] int8, [vocab, dim/32] fp16 bits
    matrix = np.ascontiguousarray(vals.reshape(vocab, dim).T)       # [dim, vocab]
    sc = np.ascontiguousarray(scales.reshape(vocab, dim // 32).T)   # [dim/32, vocab]
    idx = np.array([0, 39, 7, 7, 21], np.uint32)
    got = oracle.embedding_col(idx, matrix, sc, dim, 1)
    want = oracle.dequant(oracle.Q8_0, blocks, vocab * dim).reshape(vocab, dim)[idx]
    assert np.array_equal(got.view(np.uint32), want.view(np.uint32))


def test_embedding_col_fp16_is_the_table_column():
    vocab, dim = 17, 24
    rng = np.random.default_rng(6)
    table = rng.standard_normal((dim, vocab)).astype(np.float16)
    got = oracle.embedding_col(np.array([3, 16, 0], np.uint32), table.view(np.uint16), None, dim, 0)
    assert np.array_equal(got, table.astype(np.float32).T[[3, 16, 0]])


def test_repetition_penalty_closed_forms():
    """factor 1 is the identity; a positive logit is divided, a negative one multiplied, zero stays zero (the sign
    test is `> 0`); the factor vector built from a token window marks each token once."""
    lg = np.array([2.0, -2.0, 0.0, 5.0, -0.5, 3.0], np.float32)
    assert np.array_equal(oracle.repetition_penalty(lg, np.ones(6, np.float32)), lg)
    f = np.array([1.0, 1.0, 4.0, 2.0, 2.0, 1.0], np.float32)
    assert np.array_equal(oracle.repetition_penalty(lg, f), np.array([2.0, -2.0, 0.0, 2.5, -1.0, 3.0], np.float32))
    fac = oracle.penalty_factors([3, 4, 3, 3, -1, 99], 2.0, 6)
    assert np.array_equal(fac, np.array([1, 1, 1, 2, 2, 1], np.float32))
    # penalising twice is not what a repeated token gets
    once = oracle.repetition_penalty(lg, fac)
    assert once[3] == 2.5 and once[4] == -1.0
