"""GPU parity of the Q8_0 x int8-activation matmul on the int8 matrix core
(C ABI: cuthip_matmul_q8_i8) against the oracle's restatement of the
reference's int8 dot-product arithmetic (MatMulQ8GemvDot.cu:60-85): per-32
activation quantization, integer block dot products, fp32 scaling.  The integer
part is exact on both sides, so GPU and oracle differ by fp32 summation order
only: 1e-5 normwise is asserted (observed ~1e-7).  The distance of this variant
from the fp32-activation path (~5e-3, the cost of 8-bit activations) is
asserted separately so that it stays documented."""
import numpy as np
import pytest

import oracle
from helpers import normwise_rel_err, quantized_weights

torch = pytest.importorskip("torch")
pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def ops():
    from cut_amd import lib, ops as _ops
    lib.check(lib.load().cuthip_init(0))
    return _ops


def dev(a):
    return torch.from_numpy(np.ascontiguousarray(a)).cuda()


def host(t):
    torch.cuda.synchronize()
    return t.float().cpu().numpy()


@pytest.mark.parametrize("M,K,N", [(1, 32, 2), (5, 96, 7), (33, 128, 130), (128, 256, 128), (200, 1056, 300), (257, 4096, 384)])
def test_against_oracle(ops, M, K, N):
    rng = np.random.default_rng(M * 3 + K + N)
    A = rng.standard_normal((M, K), dtype=np.float32)
    if K >= 64:
        A[0, 32:64] = 0.0
    W = quantized_weights(oracle.Q8_0, N, K, seed=N)
    ref = oracle.matmul_q8_i8(W, A, N, f64=True)
    got = host(ops.matmul_q8_i8(dev(A), dev(W), N, K))
    assert normwise_rel_err(got, ref) < 1e-5
    # the reference's fp32 accumulation, element by element
    np.testing.assert_allclose(got, oracle.matmul_q8_i8(W, A, N), rtol=2e-4, atol=2e-5 * np.abs(ref).max())


def test_fp16_activations_and_output(ops):
    M, K, N = 64, 512, 256
    A = np.random.default_rng(1).standard_normal((M, K), dtype=np.float32).astype(np.float16)
    W = quantized_weights(oracle.Q8_0, N, K, seed=2)
    ref = oracle.matmul_q8_i8(W, A.astype(np.float32), N, f64=True)
    got = host(ops.matmul_q8_i8(dev(A), dev(W), N, K))          # fp16 in, fp16 out
    assert normwise_rel_err(got, ref) < 5e-4                     # the fp16 store
    got32 = host(ops.matmul_q8_i8(dev(A), dev(W), N, K, out_dtype=torch.float32))
    assert normwise_rel_err(got32, ref) < 1e-5


def test_known_answers_and_exact_case(ops):
    # all-ones activations, weights 1 / 2, d = 1 (the shape of q8_simple, OpRegistry.h:1995-2010)
    K, N = 64, 2
    blocks = np.zeros((N, K // 32, 34), np.uint8)
    blocks[:, :, :2] = np.array([1.0], np.float16).view(np.uint8)
    blocks[0, :, 2:], blocks[1, :, 2:] = 1, 2
    got = host(ops.matmul_q8_i8(dev(np.ones((1, K), np.float32)), dev(blocks.reshape(-1)), N, K))
    np.testing.assert_allclose(got, [[64.0, 128.0]], rtol=1e-6)
    # integer activations with +-127 in every block: the quantizer is the identity, result = exact matmul
    rng = np.random.default_rng(3)
    M, K, N = 9, 256, 40
    A = rng.integers(-127, 128, (M, K)).astype(np.float32)
    A.reshape(M, K // 32, 32)[:, :, 5] = 127.0
    W = quantized_weights(oracle.Q8_0, N, K, seed=4)
    got = host(ops.matmul_q8_i8(dev(A), dev(W), N, K))
    assert normwise_rel_err(got, oracle.matmul_gguf(oracle.Q8_0, W, A, N, f64=True)) < 1e-6


def test_distance_from_the_fp32_path_and_epilogues(ops):
    M, K, N = 96, 1024, 192
    rng = np.random.default_rng(7)
    A = rng.standard_normal((M, K), dtype=np.float32)
    W = quantized_weights(oracle.Q8_0, N, K, seed=8)
    got = host(ops.matmul_q8_i8(dev(A), dev(W), N, K))
    err = normwise_rel_err(got, oracle.matmul_gguf(oracle.Q8_0, W, A, N, f64=True))
    assert 1e-3 < err < 2e-2
    ref = oracle.matmul_q8_i8(W, A, N, f64=True)
    D = rng.standard_normal((M, N), dtype=np.float32)
    np.testing.assert_allclose(host(ops.matmul_q8_i8(dev(A), dev(W), N, K, binary="add", d=dev(D))), ref + D, rtol=0, atol=1e-4)
    np.testing.assert_allclose(host(ops.matmul_q8_i8(dev(A), dev(W), N, K, unary="relu")), np.maximum(ref, 0), rtol=0, atol=1e-4)


@pytest.mark.parametrize("M", [512, 2048])
def test_full_shape_sampled(ops, M):
    # BASELINE configs[4] shapes (M = 512 and 2048): sampled rows and columns against the oracle, linearity in the scale of A
    K, N = 4096, 14336
    rng = np.random.default_rng(11)
    A = rng.standard_normal((M, K), dtype=np.float32).astype(np.float16)
    tile = quantized_weights(oracle.Q8_0, 512, K, seed=12)
    W = np.tile(tile, N // 512)
    Wd, Ad = dev(W), dev(A)
    got = host(ops.matmul_q8_i8(Ad, Wd, N, K, out_dtype=torch.float32))
    rows = [0, 1, 255, 256, 511, M - 129, M - 1]
    ref = oracle.matmul_q8_i8(tile, A[rows].astype(np.float32), 512, f64=True)
    for c0 in (0, 512 * 13, N - 512):
        assert normwise_rel_err(got[rows][:, c0:c0 + 512], ref) < 1e-5
    # scaling the activations by a power of two scales every block's a_scale exactly
    got2 = host(ops.matmul_q8_i8(dev(A * np.float16(4.0)), Wd, N, K, out_dtype=torch.float32))
    np.testing.assert_array_equal(got2, got * 4.0)


def test_argument_errors(ops):
    from cut_amd import lib
    W = dev(quantized_weights(oracle.Q8_0, 4, 64, seed=1))
    A = torch.zeros((2, 64), device="cuda")
    with pytest.raises(lib.CutHipError, match="workspace"):
        ops.matmul_q8_i8(A, W, 4, 64, workspace=torch.empty(16, dtype=torch.uint8, device="cuda"))
    with pytest.raises(lib.CutHipError, match="multiple of 32"):
        lib.check(lib.load().cuthip_matmul_q8_i8(W.data_ptr(), A.data_ptr(), lib.F32, A.data_ptr(), lib.F32, 2, 48, 4, 48, 4,
                                                 0, 0, None, A.data_ptr(), 1 << 20, None))
