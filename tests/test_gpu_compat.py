"""GPU parity of the separated-layout (reference tensor layout) quantized
matmul through the C ABI against the oracle's restatement of the harness loops
(tests/harness/OpRegistry.h:2043-2051, 2107-2112 of the reference), including
the reference's own known-answer cases and the affine Q4 path fed by the
oracle's requantizeQ4KToAffine.  Tolerance 1e-3 normwise (fp32 throughout;
observed ~1e-6), known answers to the reference's own tolerances."""
import numpy as np
import pytest

import oracle
from helpers import normwise_rel_err

torch = pytest.importorskip("torch")
pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def ops():
    from cut_amd import lib, ops as _ops
    lib.check(lib.load().cuthip_init(0))
    return _ops


def dev(a):
    return torch.from_numpy(np.ascontiguousarray(a)).cuda()


def run(ops, A, B, S, N, **kw):
    out = ops.matmul_sep(dev(A), dev(B), dev(S.astype(np.float16)), N, **kw)
    torch.cuda.synchronize()
    return out.cpu().numpy()


def test_reference_known_answers(ops):
    # q8_simple (OpRegistry.h:1995-2010): A = 1, B[k,0] = 1, B[k,1] = 2, scales 1 -> [32, 64]
    A = np.ones((1, 32), np.float32)
    B = np.stack([np.ones(32, np.int8), np.full(32, 2, np.int8)], axis=1)
    np.testing.assert_allclose(run(ops, A, B, np.ones((1, 2), np.float32), 2), [[32, 64]], atol=1e-3)
    # q8_withscales (:2012-2026): K = 64, B = 4, scales [[0.5, 2], [1, 0.25]] -> [192, 288]
    A = np.ones((1, 64), np.float32)
    B = np.full((64, 2), 4, np.int8)
    np.testing.assert_allclose(run(ops, A, B, np.array([[0.5, 2], [1, 0.25]], np.float32), 2), [[192, 288]], atol=1.0)
    # q4: nibbles 9 / 10 (values 1 / 2) -> [32, 64]; nibble 12 with the same scales -> [192, 288]
    A = np.ones((1, 32), np.float32)
    Bp = np.full((32, 1), 9 | (10 << 4), np.uint8)
    np.testing.assert_allclose(run(ops, A, Bp, np.ones((1, 2), np.float32), 2, q4=True), [[32, 64]], atol=1e-3)
    A = np.ones((1, 64), np.float32)
    Bp = np.full((64, 1), 12 | (12 << 4), np.uint8)
    np.testing.assert_allclose(run(ops, A, Bp, np.array([[0.5, 2], [1, 0.25]], np.float32), 2, q4=True), [[192, 288]], atol=1.0)


@pytest.mark.parametrize("M", [1, 2, 3, 4, 5, 9])
@pytest.mark.parametrize("K,N", [(256, 1024), (4096, 1088), (96, 50)])
def test_q8_against_oracle(ops, M, K, N):
    rng = np.random.default_rng(M * K + N)
    A = rng.standard_normal((M, K)).astype(np.float32)
    B = rng.integers(-127, 128, (K, N)).astype(np.int8)
    S = rng.uniform(0.001, 0.02, (K // 32, N)).astype(np.float16).astype(np.float32)
    want = oracle.matmul_sep_q8(A, B, S, f64=True)
    assert normwise_rel_err(run(ops, A, B, S, N), want) < 2e-6


@pytest.mark.parametrize("affine", [False, True])
@pytest.mark.parametrize("M", [1, 4, 6])
@pytest.mark.parametrize("K,N", [(256, 2048), (4096, 1056), (64, 34)])
def test_q4_against_oracle(ops, affine, M, K, N):
    rng = np.random.default_rng(M * K + N + affine)
    A = rng.standard_normal((M, K)).astype(np.float32)
    Bp = rng.integers(0, 256, (K, N // 2)).astype(np.uint8)
    S = rng.uniform(0.001, 0.02, ((2 if affine else 1) * (K // 32), N)).astype(np.float16).astype(np.float32)
    if affine:
        S[K // 32:] = rng.uniform(-0.1, 0.1, (K // 32, N)).astype(np.float16).astype(np.float32)
    want = oracle.matmul_sep_q4(A, Bp, S, affine=affine).astype(np.float64)   # the harness loop sums in fp32
    assert normwise_rel_err(run(ops, A, Bp, S, N, q4=True, affine=affine), want) < 2e-5


def test_affine_layout_from_q4k_requantizer(ops):
    """Q4_K blocks -> requantizeQ4KToAffine (oracle restatement of llama.cpp:573-619) -> separated affine matmul
    agrees with the matmul over the decoded affine weights."""
    N, K = 64, 512
    rng = np.random.default_rng(3)
    raw = oracle.quantize(oracle.Q4_K, (rng.standard_normal(N * K) * 0.02).astype(np.float32))
    packedT, scalesT = oracle.requantize_q4k_to_affine(raw, N, K)
    Wf = oracle.decode_affine_q4(packedT, scalesT, N, K)          # [N, K]
    A = rng.standard_normal((2, K)).astype(np.float32)
    want = A.astype(np.float64) @ Wf.astype(np.float64).T
    S = oracle.f16_to_f32_array(np.asarray(scalesT).reshape(-1)).reshape(2 * K // 32, N)
    got = run(ops, A, np.asarray(packedT).reshape(K, N // 2), S, N, q4=True, affine=True)
    assert normwise_rel_err(got, want) < 5e-6


def test_fused_epilogues_and_errors(ops):
    from cut_amd import lib
    rng = np.random.default_rng(9)
    M, K, N = 3, 128, 96
    A = rng.standard_normal((M, K)).astype(np.float32)
    B = rng.integers(-127, 128, (K, N)).astype(np.int8)
    S = rng.uniform(0.001, 0.02, (K // 32, N)).astype(np.float16).astype(np.float32)
    base = run(ops, A, B, S, N)
    D = rng.standard_normal((M, N)).astype(np.float32)
    got = ops.matmul_sep(dev(A), dev(B), dev(S.astype(np.float16)), N, binary="add", d=dev(D))
    torch.cuda.synchronize()
    np.testing.assert_allclose(got.cpu().numpy(), base + D, rtol=1e-6, atol=1e-6)
    got = ops.matmul_sep(dev(A), dev(B), dev(S.astype(np.float16)), N, unary="relu")
    torch.cuda.synchronize()
    np.testing.assert_array_equal(got.cpu().numpy(), np.maximum(base, 0))
    with pytest.raises(lib.CutHipError):
        ops.matmul_sep(dev(A[:, :100].copy()), dev(B[:100]), dev(S.astype(np.float16)[:3]), N)   # K not a multiple of 32


# ---- prefill route: from 32 rows on (K a multiple of 128) the tensors are dequantized to fp16 [N][K] and multiplied by
# the dense GEMM; fp16 weights and activations, fp32 accumulation: the tolerance of the native prefill path -------------

@pytest.mark.parametrize("M,K,N", [(32, 128, 64), (70, 256, 200), (300, 1024, 520), (1030, 512, 264)])
def test_prefill_route_q8(ops, M, K, N):
    rng = np.random.default_rng(M + K + N)
    A = rng.standard_normal((M, K)).astype(np.float32)
    B = rng.integers(-127, 128, (K, N)).astype(np.int8)
    S = rng.uniform(0.001, 0.02, (K // 32, N)).astype(np.float16).astype(np.float32)
    want = oracle.matmul_sep_q8(A, B, S, f64=True)
    assert normwise_rel_err(run(ops, A, B, S, N), want) < 1e-3
    D = rng.standard_normal((M, N)).astype(np.float32)
    got = ops.matmul_sep(dev(A), dev(B), dev(S.astype(np.float16)), N, binary="add", d=dev(D))   # fused epilogue: own GEMM
    torch.cuda.synchronize()
    assert normwise_rel_err(got.cpu().numpy() - D, want) < 1e-3


def test_prefill_route_rounds_activations_to_fp16(ops):
    """The contract of the prefill route in cut_hip.h: fp32 activations are rounded to fp16 once.  Large magnitudes
    inside the fp16 range keep the 1e-3 normwise bound; beyond 65504 the result is not finite there, while the GEMV
    variant (reference index 1) computes in fp32 and stays within 1e-5."""
    M, K, N = 64, 512, 136
    rng = np.random.default_rng(77)
    A = (rng.standard_normal((M, K)) * 1.0e3).astype(np.float32)
    B = rng.integers(-127, 128, (K, N)).astype(np.int8)
    S = rng.uniform(0.001, 0.02, (K // 32, N)).astype(np.float16).astype(np.float32)
    want = oracle.matmul_sep_q8(A, B, S, f64=True)
    assert normwise_rel_err(run(ops, A, B, S, N), want) < 1e-3
    A[3, 17] = 1.0e5
    want = oracle.matmul_sep_q8(A, B, S, f64=True)
    assert not np.isfinite(run(ops, A, B, S, N)[3]).all()
    assert normwise_rel_err(run(ops, A, B, S, N, variant=1), want) < 1e-5


@pytest.mark.parametrize("affine", [False, True])
@pytest.mark.parametrize("M,K,N", [(32, 128, 66), (300, 1024, 520)])
def test_prefill_route_q4(ops, affine, M, K, N):
    rng = np.random.default_rng(M + K + N + affine)
    A = rng.standard_normal((M, K)).astype(np.float32)
    Bp = rng.integers(0, 256, (K, N // 2)).astype(np.uint8)
    S = rng.uniform(0.001, 0.02, ((2 if affine else 1) * (K // 32), N)).astype(np.float16).astype(np.float32)
    if affine:
        S[K // 32:] = rng.uniform(-0.1, 0.1, (K // 32, N)).astype(np.float16).astype(np.float32)
    want = oracle.matmul_sep_q4(A[:8], Bp, S, affine=affine).astype(np.float64)   # the CPU loop on the first rows
    got = run(ops, A, Bp, S, N, q4=True, affine=affine)
    assert normwise_rel_err(got[:8], want) < 1e-3
    # rows are independent: the GEMV route on a few rows gives what the prefill route gave for them
    few = run(ops, A[8:12], Bp, S, N, q4=True, affine=affine)
    assert normwise_rel_err(got[8:12], few) < 1e-3


def test_prefill_route_after_device_preparation(ops):
    """GGUF Q8_0 blocks -> cuthip_prepare_sep -> separated matmul at prefill size, against the native-block path."""
    from helpers import quantized_weights
    M, K, N = 256, 512, 384
    blocks = quantized_weights(oracle.Q8_0, N, K, seed=9)
    B, S = ops.prepare_sep(dev(blocks), "Q8_0", N, K)
    A = np.random.default_rng(10).standard_normal((M, K)).astype(np.float32)
    got = ops.matmul_sep(dev(A), B, S, N)
    torch.cuda.synchronize()
    want = oracle.matmul_gguf(oracle.Q8_0, blocks, A, N, f64=True)
    assert normwise_rel_err(got.cpu().numpy(), want) < 1e-3
