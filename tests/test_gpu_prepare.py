"""GPU parity of the load-time weight preparation (C ABI: cuthip_prepare_sep,
cuthip_transpose_q4_nibble, cuthip_quantize_rows_q8_0) against the oracle's
restatements of the reference's host code: the separated readers
(gguf_reader.cpp:389-501) followed by a transpose, TransposeQ4Nibble.cu:17-61,
requantizeQ4KToAffine (llama.cpp:573-619) and quantizeRowsQ8_0 (llama.cpp:488-505).
Everything here is byte / integer / fp16-bit work: the bar is bit-exact.  Block
scales are finite (a non-finite d makes the reference's result depend on the
sign of the host's default NaN)."""
import numpy as np
import pytest

import oracle
from helpers import finite_random_blocks, gauss_weights, normwise_rel_err, quantized_weights

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
    return t.cpu().numpy()


SHAPES = [(2, 32), (6, 96), (128, 256), (130, 288), (258, 1024), (34, 4128), (1000, 160)]


@pytest.mark.parametrize("N,K", SHAPES)
def test_q8_0_blocks_to_separated(ops, N, K):
    blocks = finite_random_blocks(oracle.Q8_0, N * K // 32, seed=N + K)
    v, s = oracle.split_q8_0(blocks, N, K)          # [N, K], [N, K/32]
    B, S = ops.prepare_sep(dev(blocks), "Q8_0", N, K)
    B, S = host(B), host(S.view(torch.int16)).view(np.uint16)
    assert B.shape[1] % 4 == 0 and S.shape[1] % 4 == 0
    np.testing.assert_array_equal(B[:, :N], v.T)
    np.testing.assert_array_equal(S[:, :N], s.T)
    assert not B[:, N:].any() and not S[:, N:].any()   # padding columns stay untouched


@pytest.mark.parametrize("N,K", SHAPES)
def test_q4_0_blocks_to_separated(ops, N, K):
    blocks = finite_random_blocks(oracle.Q4_0, N * K // 32, seed=2 * N + K)
    p, s = oracle.split_q4_0(blocks, N, K)          # [N, K/2] GGML nibble order, [N, K/32]
    want = oracle.transpose_q4_nibble(p, N, K)      # [K, N/2]
    B, S = ops.prepare_sep(dev(blocks), "Q4_0", N, K)
    B, S = host(B), host(S.view(torch.int16)).view(np.uint16)
    np.testing.assert_array_equal(B[:, :N // 2], want)
    np.testing.assert_array_equal(S[:, :N], s.T)
    assert not B[:, N // 2:].any() and not S[:, N:].any()


@pytest.mark.parametrize("N,K", SHAPES)
def test_transpose_q4_nibble_operator(ops, N, K):
    rng = np.random.default_rng(N * 7 + K)
    stride_in = (K // 2 + 3) & ~3
    packed = rng.integers(0, 256, (N, stride_in), dtype=np.uint8)
    want = oracle.transpose_q4_nibble(np.ascontiguousarray(packed[:, :K // 2]), N, K)
    got = host(ops.transpose_q4_nibble(dev(packed), N, K))
    np.testing.assert_array_equal(got[:, :N // 2], want)
    assert not got[:, N // 2:].any()


def test_transpose_q4_nibble_basis(ops):
    # one non-zero nibble at every (n, k) position of a 4 x 64 matrix lands where the reference's indexing puts it
    N, K = 4, 64
    for n in range(N):
        for k in range(K):
            packed = np.zeros((N, K // 2), np.uint8)
            blk, e = divmod(k, 32)
            packed[n, blk * 16 + e % 16] = 0xB << (4 * (e // 16))
            got = host(ops.transpose_q4_nibble(dev(packed), N, K))
            want = np.zeros((K, N // 2), np.uint8)
            want[k, n // 2] = 0xB << (4 * (n & 1))
            np.testing.assert_array_equal(got[:, :N // 2], want)


@pytest.mark.parametrize("N,K", [(2, 256), (6, 512), (128, 256), (130, 768), (258, 1024), (1000, 256)])
def test_q4_k_to_affine(ops, N, K):
    blocks = finite_random_blocks(oracle.Q4_K, N * K // 256, seed=3 * N + K)
    want_p, want_s = oracle.requantize_q4k_to_affine(blocks, N, K)
    B, S = ops.prepare_sep(dev(blocks), "Q4_K", N, K)
    B, S = host(B), host(S.view(torch.int16)).view(np.uint16)
    np.testing.assert_array_equal(B[:, :N // 2], want_p)
    np.testing.assert_array_equal(S[:, :N], want_s)


def test_q4_k_to_affine_on_quantized_weights_feeds_the_matmul(ops):
    # real (encoder-made) blocks; the affine tensors then go through the separated-layout matmul
    N, K, M = 512, 1024, 3
    blocks = quantized_weights(oracle.Q4_K, N, K, seed=5)
    want_p, want_s = oracle.requantize_q4k_to_affine(blocks, N, K)
    B, S = ops.prepare_sep(dev(blocks), "Q4_K", N, K)
    np.testing.assert_array_equal(host(B)[:, :N // 2], want_p)
    np.testing.assert_array_equal(host(S.view(torch.int16)).view(np.uint16)[:, :N], want_s)
    A = np.random.default_rng(1).standard_normal((M, K), dtype=np.float32)
    got = host(ops.matmul_sep(dev(A), B, S, N, q4=True, affine=True))
    ref = A.astype(np.float64) @ oracle.decode_affine_q4(want_p, want_s, N, K).astype(np.float64).T
    assert normwise_rel_err(got, ref) < 1e-3
    # and the affine re-encoding stays within fp16 rounding of the native blocks (llama.cpp:704-738, verifyQ4KAffine)
    ref_native = A.astype(np.float64) @ oracle.dequant(oracle.Q4_K, blocks, N * K).reshape(N, K).astype(np.float64).T
    assert normwise_rel_err(got, ref_native) < 2e-3


def test_prepared_q8_feeds_the_matmul(ops):
    N, K, M = 384, 512, 2
    blocks = quantized_weights(oracle.Q8_0, N, K, seed=6)
    B, S = ops.prepare_sep(dev(blocks), "Q8_0", N, K)
    A = np.random.default_rng(2).standard_normal((M, K), dtype=np.float32)
    got = host(ops.matmul_sep(dev(A), B, S, N))
    ref = oracle.matmul_gguf(oracle.Q8_0, blocks, A, N, f64=True)
    assert normwise_rel_err(got, ref) < 1e-3


@pytest.mark.parametrize("n", [32, 96, 4096, 32 * 1001])
def test_quantize_rows_q8_0(ops, n):
    rng = np.random.default_rng(n)
    x = (rng.standard_normal(n, dtype=np.float32) * np.float32(0.02)).astype(np.float32)
    x[:32] = 0.0                                       # an all-zero block: d = 0, q = 0
    if n >= 96:
        x[32:64] = np.linspace(-127, 127, 32, dtype=np.float32) * np.float32(0.5)   # exact .5 ties in x * id
        x[64:96] = rng.standard_normal(32).astype(np.float32) * np.float32(1e4)
    v, s = oracle.quantize_rows_q8_0(x)
    got = host(ops.quantize_rows_q8_0(dev(x))).reshape(-1, 34)
    np.testing.assert_array_equal(got[:, :2].copy().view(np.uint16).reshape(-1), s)
    np.testing.assert_array_equal(got[:, 2:].copy().view(np.int8).reshape(-1), v)


def test_quantize_rows_q8_0_config1_weights(ops):
    # BASELINE configs[0]: 4096 x 4096 N(0, 0.02) weights through the reference quantizer, then the native GEMV
    N = K = 1024
    w = gauss_weights(N * K, seed=0)
    v, s = oracle.quantize_rows_q8_0(w)
    blocks = ops.quantize_rows_q8_0(dev(w))
    got = host(blocks).reshape(-1, 34)
    np.testing.assert_array_equal(got[:, :2].copy().view(np.uint16).reshape(-1), s)
    np.testing.assert_array_equal(got[:, 2:].copy().view(np.int8).reshape(-1), v)
    x = np.random.default_rng(1).standard_normal((1, K), dtype=np.float32)
    y = host(ops.matmul_gguf(dev(x), blocks, "Q8_0", N, K))
    ref = oracle.matmul_gguf(oracle.Q8_0, got.reshape(-1), x, N, f64=True)
    assert normwise_rel_err(y, ref) < 1e-3


def test_argument_errors(ops):
    from cut_amd import lib
    blocks = dev(finite_random_blocks(oracle.Q4_0, 3 * 2, seed=1))
    with pytest.raises(lib.CutHipError, match="even"):
        ops.prepare_sep(blocks, "Q4_0", 3, 64)
    with pytest.raises(lib.CutHipError, match="separated layout"):
        ops.prepare_sep(blocks, "Q6_K", 2, 256)
    with pytest.raises(lib.CutHipError, match="multiple of 32"):
        ops.quantize_rows_q8_0(torch.zeros(33, device="cuda"))
