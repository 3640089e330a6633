"""Pins for the oracle's matmul loops (CPU only): the reference's known-answer
cases (OpRegistry.h:1995-2192, RuntimeTests.cpp:2861-2938), invariants, and a
float64 numpy anchor."""
import numpy as np
import pytest

import oracle
from helpers import generate_test_data, normwise_rel_err, quantized_weights, stl_uniform

f16 = lambda v: oracle.f16_to_f32(oracle.harness_f32_to_f16(v))


def pack(lo, hi):
    return (lo & 0xF) | ((hi & 0xF) << 4)


def test_stl_uniform_known_values():
    # first draws of std::mt19937(42) through uniform_real_distribution<float>,
    # printed by a libstdc++ program
    assert np.allclose(generate_test_data(4), [3.80794692, 7.98577547, 9.51207161, 1.9160043], rtol=0, atol=5e-7)
    assert np.allclose(stl_uniform(4, 42, -1.0, 1.0), [-0.250919759, 0.593086004, 0.90142858, -0.633130431], rtol=0, atol=5e-8)


def test_q8_simple():
    K, N = 32, 2
    B = np.zeros((K, N), np.int8)
    B[:, 0], B[:, 1] = 1, 2
    C = oracle.matmul_sep_q8(np.ones((1, K), np.float32), B, np.ones((1, N), np.float32))
    assert np.array_equal(C, [[32.0, 64.0]])


def test_q8_withscales():
    K, N = 64, 2
    C = oracle.matmul_sep_q8(np.ones((1, K), np.float32), np.full((K, N), 4, np.int8),
                             np.array([[0.5, 2.0], [1.0, 0.25]], np.float32))
    assert np.array_equal(C, [[192.0, 288.0]])


def test_q4_simple_and_withscales():
    K, N = 32, 2
    Bp = np.full((K, 1), pack(9, 10), np.uint8)
    C = oracle.matmul_sep_q4(np.ones((1, K), np.float32), Bp, np.ones((1, N), np.float32))
    assert np.array_equal(C, [[32.0, 64.0]])
    K = 64
    Bp = np.full((K, 1), pack(12, 12), np.uint8)
    C = oracle.matmul_sep_q4(np.ones((1, K), np.float32), Bp, np.array([[0.5, 2.0], [1.0, 0.25]], np.float32))
    assert np.array_equal(C, [[192.0, 288.0]])


def _pattern_case(M, K, N):
    A = generate_test_data(M * K).reshape(M, K)
    i = np.arange(K * N)
    B = ((i * 7 + 3) % 21 - 10).astype(np.int8).reshape(K, N)
    nib = ((i * 7 + 3) % 16).astype(np.uint8).reshape(K, N)
    S = (np.float32(0.1) + np.float32(0.05) * np.arange(K // 32 * N, dtype=np.float32)).reshape(K // 32, N)
    return A, B, nib, S


@pytest.mark.parametrize("M,K,N", [(2, 64, 4), (1, 512, 16)])
def test_q8_pattern_cases_vs_float64(M, K, N):
    # q8_vsregular / q8_allvariants inputs; the loop itself is the reference's
    A, B, _, S = _pattern_case(M, K, N)
    got = oracle.matmul_sep_q8(A, B, S)
    W = B.astype(np.float64) * np.repeat(S.astype(np.float64), 32, axis=0)
    want = A.astype(np.float64) @ W
    assert np.all(np.abs(got - want) <= np.abs(want) * 1e-5 + 1e-4)
    # the reference's own tolerance, with room to spare
    assert np.all(np.abs(got - want) <= np.abs(want) * 0.01 + 0.1)


@pytest.mark.parametrize("M,K,N", [(2, 64, 4), (1, 64, 4)])
def test_q4_pattern_cases_vs_float64(M, K, N):
    A, _, nib, S = _pattern_case(M, K, N)
    Bp = (nib[:, 0::2] | (nib[:, 1::2] << 4)).astype(np.uint8)
    got = oracle.matmul_sep_q4(A, Bp, S)
    W = (nib.astype(np.float64) - 8) * np.repeat(S.astype(np.float64), 32, axis=0)
    want = A.astype(np.float64) @ W
    assert np.all(np.abs(got - want) <= np.abs(want) * 1e-5 + 1e-4)


def test_q4_affine_adds_min_rows():
    A, _, nib, S = _pattern_case(2, 64, 4)
    Bp = (nib[:, 0::2] | (nib[:, 1::2] << 4)).astype(np.uint8)
    mins = (np.arange(2 * 4, dtype=np.float32) * np.float32(0.25) - 1).reshape(2, 4)
    got = oracle.matmul_sep_q4(A, Bp, np.concatenate([S, mins]), affine=True)
    W = (nib.astype(np.float64) - 8) * np.repeat(S.astype(np.float64), 32, axis=0) + np.repeat(mins.astype(np.float64), 32, axis=0)
    want = A.astype(np.float64) @ W
    assert np.all(np.abs(got - want) <= np.abs(want) * 1e-5 + 1e-4)


def test_mistral_geometry_double_reference():
    # RuntimeTests.cpp:2861-2938 at a quarter of N (same strides, same data rule)
    M, K, N = 4, 5120, 1024
    A = stl_uniform(M * K, 42, -1.0, 1.0).reshape(M, K)
    i = np.arange(K * N, dtype=np.int64)
    B = ((i * 7 + 3) % 21 - 10).astype(np.int8).reshape(K, N)
    S = ((1.0 + (np.arange(K // 32 * N) % 7)) * 0.03125).astype(np.float32).reshape(K // 32, N)
    ref64 = oracle.matmul_sep_q8(A, B, S, f64=True)
    want = (A.astype(np.float64) @ (B.astype(np.float64) * np.repeat(S.astype(np.float64), 32, axis=0))).astype(np.float32)
    assert np.max(np.abs(ref64 - want)) <= 1e-4
    got32 = oracle.matmul_sep_q8(A, B, S)
    assert np.all(np.abs(got32 - ref64) <= np.abs(ref64) * 2e-3 + 0.05)  # the reference's bound
    # batched == per-row (the property the reference test asserts)
    for m in range(M):
        assert np.array_equal(oracle.matmul_sep_q8(A[m:m + 1], B, S), got32[m:m + 1])


@pytest.mark.parametrize("name", list(oracle.FORMATS))
def test_gguf_matmul_is_a_times_dequant_transposed(name):
    fmt = oracle.FORMATS[name]
    N, K, M = 48, 1024, 3
    W = quantized_weights(fmt, N, K, seed=4)
    A = np.random.default_rng(1).standard_normal((M, K), dtype=np.float32)
    Wf = oracle.dequant(fmt, W, N * K).reshape(N, K)
    want = A.astype(np.float64) @ Wf.astype(np.float64).T
    got32 = oracle.matmul_gguf(fmt, W, A, N)
    got64 = oracle.matmul_gguf(fmt, W, A, N, f64=True)
    assert normwise_rel_err(got64, want) < 1e-14
    assert normwise_rel_err(got32, want) < 1e-5
    # invariants: linearity in A, independent batch rows, zero rows, row permutation
    assert np.allclose(oracle.matmul_gguf(fmt, W, 2 * A, N, f64=True), 2 * got64, rtol=1e-12)
    assert np.array_equal(oracle.matmul_gguf(fmt, W, A[1:2], N), got32[1:2])
    rb = oracle.n_bytes(fmt, K)
    perm = np.random.default_rng(2).permutation(N)
    Wp = W.reshape(N, rb)[perm].reshape(-1)
    assert np.array_equal(oracle.matmul_gguf(fmt, Wp, A, N), got32[:, perm])
    Wz = W.copy().reshape(N, rb)
    Wz[5] = 0
    assert np.all(oracle.matmul_gguf(fmt, Wz.reshape(-1), A, N)[:, 5] == 0)


def test_quantize_act_q8():
    rng = np.random.default_rng(8)
    a = rng.standard_normal(32 * 9).astype(np.float32)
    a[:32] = 0
    a[32] = 0.5  # exact ties after scaling: amax = 1 -> a*127 = 63.5
    a[33] = 1.0
    a[34:64] = 0
    q, s = oracle.quantize_act_q8(a)
    assert not q[:32].any() and s[0] == 0
    assert q[32] == 64 and q[33] == 127  # half away from zero
    ab = a.reshape(-1, 32)
    assert np.array_equal(s, (np.abs(ab).max(1) / np.float32(127)).astype(np.float32))
    assert np.all(np.abs(q.astype(np.int32)) <= 127)
    back = q.reshape(-1, 32) * s[:, None]
    assert np.max(np.abs(back - ab)) <= np.max(s) * 0.5 + 1e-7


# ---- int8-activation arithmetic (MatMulQ8GemvDot.cu:60-85) on Q8_0 blocks ----------------------------

def q8_blocks(q, d):
    """Q8_0 blocks from int8 values [N, K] and fp16-exact scales [N, K/32]."""
    N, K = q.shape
    blocks = np.zeros((N, K // 32, 34), np.uint8)
    blocks[:, :, :2] = np.asarray(d, np.float16).reshape(N, K // 32, 1).view(np.uint8)
    blocks[:, :, 2:] = q.reshape(N, K // 32, 32).view(np.uint8)
    return blocks.reshape(-1)


def test_q8_i8_known_answer():
    # all-ones activations quantize to 127 with a_scale = fl(1/127); weights 1 / 2 with d = 1: 32 and 64 per block
    K, N = 64, 2
    q = np.zeros((N, K), np.int8)
    q[0], q[1] = 1, 2
    C = oracle.matmul_q8_i8(q8_blocks(q, np.ones((N, 2))), np.ones((1, K), np.float32), N)
    np.testing.assert_allclose(C, [[64.0, 128.0]], rtol=3e-7)
    # scales {0.5, 2} / {1, 0.25} with weight 4 as in q8_withscales (OpRegistry.h:2012-2026): 4*32*(0.5+1), 4*32*(2+0.25)
    q[:] = 4
    C = oracle.matmul_q8_i8(q8_blocks(q, np.array([[0.5, 1.0], [2.0, 0.25]])), np.ones((1, K), np.float32), N)
    np.testing.assert_allclose(C, [[192.0, 288.0]], rtol=3e-7)


def test_q8_i8_reduces_to_the_exact_path_on_int8_activations():
    # integer activations whose every block holds +-127: a_scale = 1, 127/amax = 1, so the quantizer is the
    # identity and the result must equal the float64 matmul on the dequantized weights
    rng = np.random.default_rng(3)
    M, K, N = 3, 256, 40
    A = rng.integers(-127, 128, (M, K)).astype(np.float32)
    A.reshape(M, K // 32, 32)[:, :, 5] = 127.0
    A.reshape(M, K // 32, 32)[:, ::2, 9] = -127.0
    W = quantized_weights(oracle.Q8_0, N, K, seed=4)
    q, s = oracle.quantize_act_q8(A)
    assert np.array_equal(q.astype(np.float32).reshape(A.shape), A) and np.all(s == 1.0)
    ref = oracle.matmul_gguf(oracle.Q8_0, W, A, N, f64=True)
    np.testing.assert_allclose(oracle.matmul_q8_i8(W, A, N, f64=True), ref, rtol=1e-12, atol=1e-12)
    assert normwise_rel_err(oracle.matmul_q8_i8(W, A, N), ref) < 1e-6


def test_q8_i8_against_an_integer_numpy_restatement_and_the_fp32_path():
    rng = np.random.default_rng(5)
    M, K, N = 4, 512, 64
    A = rng.standard_normal((M, K), dtype=np.float32)
    A[1, 32:64] = 0.0                                   # an all-zero block: scale 0, q 0
    W = quantized_weights(oracle.Q8_0, N, K, seed=6)
    blocks = W.reshape(N, K // 32, 34)
    d = blocks[:, :, :2].copy().view(np.float16).astype(np.float64).reshape(N, K // 32)
    qw = blocks[:, :, 2:].copy().view(np.int8).astype(np.int64)
    Ab = A.reshape(M, K // 32, 32)
    amax = np.abs(Ab).max(axis=2)
    sa = (amax / np.float32(127.0)).astype(np.float32)
    inv = np.where(amax > 0, np.float32(127.0) / np.where(amax > 0, amax, 1), 0).astype(np.float32)
    t = Ab * inv[:, :, None]
    qa = np.clip(np.sign(t) * np.floor(np.abs(t) + np.float32(0.5)), -127, 127).astype(np.int64)
    dots = np.einsum("mbk,nbk->mnb", qa, qw)
    want = (dots * sa.astype(np.float64)[:, None, :] * d[None, :, :]).sum(axis=2)
    np.testing.assert_allclose(oracle.matmul_q8_i8(W, A, N, f64=True), want, rtol=1e-12, atol=1e-12)
    assert normwise_rel_err(oracle.matmul_q8_i8(W, A, N), want) < 1e-6
    # what the 8-bit activations cost against the fp32-activation path the other kernels are held to
    err = normwise_rel_err(want, oracle.matmul_gguf(oracle.Q8_0, W, A, N, f64=True))
    assert 1e-3 < err < 2e-2
