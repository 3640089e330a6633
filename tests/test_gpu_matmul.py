"""GPU parity: quantized GEMV / skinny GEMM on native GGUF blocks through the
C ABI, against the CPU oracle ("A . dequant_cpu(W)^T").  Tolerance: 1e-3
normwise relative error, the bar BASELINE.json states; the asserted bound is
tighter where the arithmetic allows."""
import numpy as np
import pytest

import oracle
from helpers import gauss_acts, normwise_rel_err, quantized_weights, finite_random_blocks

torch = pytest.importorskip("torch")
pytestmark = pytest.mark.gpu

TOL = 1e-3          # stated tolerance
TOL_F16_ACT = 2e-5  # fp16 activations are consumed exactly; only fp32 summation order differs
TOL_F32_ACT = 4e-4  # fp32 activations are rounded to fp16 (2^-11 relative per element)


@pytest.fixture(scope="module")
def ops():
    from cut_amd import lib, ops as _ops
    lib.check(lib.load().cuthip_init(0))
    return _ops


def gpu_matmul(ops, fmt, W, A, N, K, out_dtype=None, **kw):
    w = torch.from_numpy(W).cuda()
    a = torch.from_numpy(A).cuda()
    c = ops.matmul_gguf(a, w, fmt, N, K, out_dtype=out_dtype, **kw)
    torch.cuda.synchronize()
    return c.float().cpu().numpy()


@pytest.mark.parametrize("name", list(oracle.FORMATS))
@pytest.mark.parametrize("M", [1, 2, 3, 4, 5, 8])
def test_gemv_fp16_activations(ops, name, M):
    fmt = oracle.FORMATS[name]
    N, K = 200, 2048  # N not a multiple of 32: ragged last tile
    W = quantized_weights(fmt, N, K, seed=2)
    A = gauss_acts((M, K), seed=1, dtype=np.float16)
    got = gpu_matmul(ops, fmt, W, A, N, K, out_dtype=torch.float32)
    want = oracle.matmul_gguf(fmt, W, A.astype(np.float32), N, f64=True)
    err = normwise_rel_err(got, want)
    assert err < TOL_F16_ACT, err
    # and against the reference's fp32 sequential loop, at the stated tolerance
    assert normwise_rel_err(got, oracle.matmul_gguf(fmt, W, A.astype(np.float32), N)) < TOL


@pytest.mark.parametrize("name", list(oracle.FORMATS))
def test_gemv_fp32_activations_config1_shape(ops, name):
    """BASELINE config 1 geometry (4096 x 4096, x fp32 [4096], y fp32) for each
    format; Q8_0 weights come from the reference quantizer."""
    fmt = oracle.FORMATS[name]
    N = K = 4096
    W = quantized_weights(fmt, N, K, seed=0)
    x = gauss_acts((1, K), seed=1)
    got = gpu_matmul(ops, fmt, W, x, N, K)
    want = oracle.matmul_gguf(fmt, W, x, N)  # the CPU harness path, fp32 sequential
    err = normwise_rel_err(got, want)
    assert err < TOL_F32_ACT, err


@pytest.mark.parametrize("M", [1, 2, 4, 8])
@pytest.mark.parametrize("N,K", [(14336, 4096), (4096, 14336)])
def test_q4k_ffn_shapes_fp16_io(ops, N, K, M):
    """BASELINE config 3: FFN shapes, fp16 in, fp32 accumulate, fp16 out.
    The oracle runs on a row sample to stay within seconds."""
    fmt = oracle.Q4_K
    W = quantized_weights(fmt, N, K, seed=0)
    A = gauss_acts((M, K), seed=1, dtype=np.float16)
    got = gpu_matmul(ops, fmt, W, A, N, K)  # fp16 out
    rows = np.unique(np.concatenate([np.arange(0, 64), np.arange(N - 64, N), np.random.default_rng(0).integers(0, N, 512)]))
    rb = oracle.n_bytes(fmt, K)
    Ws = W.reshape(N, rb)[rows].reshape(-1)
    want = oracle.matmul_gguf(fmt, Ws, A.astype(np.float32), len(rows), f64=True)
    err = normwise_rel_err(got[:, rows], want)
    assert err < 6e-4, err  # fp16 output rounding: 2^-11 / sqrt(3) ~ 2.8e-4 rms
    # batch rows are independent: row 0 of the batched call agrees with the M=1 call
    # (the two launches use different kernels and K orders, so fp32 sums can
    # round to neighbouring fp16 values, and outputs that cancel to almost
    # zero differ by the fp32 rounding of their terms)
    if M > 1:
        one = gpu_matmul(ops, fmt, W, A[:1], N, K)
        rms = float(np.sqrt(np.mean(got[0].astype(np.float64) ** 2)))
        assert np.all(np.abs(one[0] - got[0]) <= np.abs(got[0]) * 2.0 ** -10 + 1e-4 * rms)


@pytest.mark.parametrize("M", [16, 32, 64, 128])
@pytest.mark.parametrize("N,K", [(14336, 4096), (4096, 14336)])
def test_q4k_ffn_shapes_at_9_to_128_rows(ops, N, K, M):
    """The FFN shapes at the row counts between the GEMV and prefill, through the workspace entry point with the
    library's own choice (streaming MFMA kernel up to 32 rows, tiled GEMM with K split over workgroups beyond): fp32
    output against the float64 oracle on a sample of weight rows, and batch rows are independent: rows 0 and M - 1
    of the call agree with the same rows computed alone by the GEMV."""
    fmt = oracle.Q4_K
    W = quantized_weights(fmt, N, K, seed=0)
    A = gauss_acts((M, K), seed=M, dtype=np.float16)
    a, w = torch.from_numpy(A).cuda(), torch.from_numpy(W).cuda()
    ws = ops.matmul_gguf_workspace(fmt, M, K, N, a.dtype, "cuda")
    ws.fill_(0xFF)
    got = ops.matmul_gguf(a, w, fmt, N, K, out_dtype=torch.float32, workspace=ws)
    torch.cuda.synchronize()
    got = got.cpu().numpy()
    rows = np.unique(np.concatenate([np.arange(0, 64), np.arange(N - 64, N), np.random.default_rng(0).integers(0, N, 384)]))
    Ws = W.reshape(N, oracle.n_bytes(fmt, K))[rows].reshape(-1)
    want = oracle.matmul_gguf(fmt, Ws, A.astype(np.float32), len(rows), f64=True)
    assert normwise_rel_err(got[:, rows], want) < (TOL_F16_ACT if M <= 32 else 5e-4)   # exact products / fp16-decoded weights
    for r in (0, M - 1):
        one = ops.matmul_gguf(a[r:r + 1], w, fmt, N, K, out_dtype=torch.float32)
        torch.cuda.synchronize()
        assert normwise_rel_err(got[r:r + 1], one.cpu().numpy()) < (TOL_F16_ACT if M <= 32 else 5e-4)


def test_linearity_and_row_permutation(ops):
    fmt = oracle.Q4_K
    N, K = 4096, 4096
    W = quantized_weights(fmt, N, K, seed=3)
    A = gauss_acts((2, K), seed=4, dtype=np.float16)
    base = gpu_matmul(ops, fmt, W, A, N, K, out_dtype=torch.float32)
    twice = gpu_matmul(ops, fmt, W, (A * np.float16(2)), N, K, out_dtype=torch.float32)
    assert np.array_equal(twice, 2 * base)  # power-of-two scaling is exact
    rb = oracle.n_bytes(fmt, K)
    perm = np.random.default_rng(1).permutation(N)
    Wp = np.ascontiguousarray(W.reshape(N, rb)[perm]).reshape(-1)
    assert np.array_equal(gpu_matmul(ops, fmt, Wp, A, N, K, out_dtype=torch.float32), base[:, perm])
    Wz = W.copy().reshape(N, rb)
    Wz[17] = 0
    assert np.all(gpu_matmul(ops, fmt, Wz.reshape(-1), A, N, K, out_dtype=torch.float32)[:, 17] == 0)


@pytest.mark.parametrize("name", list(oracle.FORMATS))
def test_random_block_bytes(ops, name):
    """Uniformly random bytes: all scale bit patterns incl. negative and
    subnormal d, extreme sub-scales; compared in float64."""
    fmt = oracle.FORMATS[name]
    N, K = 64, 1024
    W = finite_random_blocks(fmt, N * K // oracle.BLOCK_ELEMS[fmt], seed=31)
    # keep the magnitudes finite in fp32: clear the top exponent bit of every fp16 scale
    bb = oracle.BLOCK_BYTES[fmt]
    Wb = W.reshape(-1, bb)
    for off in {oracle.Q8_0: [0], oracle.Q4_0: [0], oracle.Q4_K: [0, 2], oracle.Q6_K: [208]}[fmt]:
        Wb[:, off + 1] &= 0xBF
    A = gauss_acts((3, K), seed=9, dtype=np.float16)
    got = gpu_matmul(ops, fmt, W, A, N, K, out_dtype=torch.float32)
    want = oracle.matmul_gguf(fmt, W, A.astype(np.float32), N, f64=True)
    assert normwise_rel_err(got, want) < 5e-5


@pytest.mark.parametrize("name,K", [("Q8_0", 96), ("Q4_0", 32), ("Q8_0", 4128), ("Q4_K", 256), ("Q6_K", 768)])
def test_small_and_ragged_k(ops, name, K):
    fmt = oracle.FORMATS[name]
    N, M = 33, 2
    W = quantized_weights(fmt, N, K, seed=6)
    A = gauss_acts((M, K), seed=7, dtype=np.float16)
    got = gpu_matmul(ops, fmt, W, A, N, K, out_dtype=torch.float32)
    want = oracle.matmul_gguf(fmt, W, A.astype(np.float32), N, f64=True)
    assert normwise_rel_err(got, want) < TOL_F16_ACT


@pytest.mark.parametrize("M", [9, 33, 70])
def test_skinny_gemm_passes(ops, M):
    fmt = oracle.Q4_K
    N, K = 96, 1024
    W = quantized_weights(fmt, N, K, seed=8)
    A = gauss_acts((M, K), seed=3, dtype=np.float16)
    got = gpu_matmul(ops, fmt, W, A, N, K, out_dtype=torch.float32, variant=1)  # 32-row passes of the streaming kernel
    want = oracle.matmul_gguf(fmt, W, A.astype(np.float32), N, f64=True)
    assert normwise_rel_err(got, want) < TOL_F16_ACT


def test_fused_epilogues(ops):
    """SiLU on the gate projection and the residual add on wo / w_down
    (llama.cpp:2459-2463, 1790-1795 of the reference)."""
    fmt = oracle.Q4_K
    N, K, M = 256, 1024, 2
    W = quantized_weights(fmt, N, K, seed=12)
    A = gauss_acts((M, K), seed=13, dtype=np.float16)
    plain = gpu_matmul(ops, fmt, W, A, N, K, out_dtype=torch.float32)
    silu = gpu_matmul(ops, fmt, W, A, N, K, out_dtype=torch.float32, unary="silu")
    assert np.allclose(silu, plain / (1 + np.exp(-plain.astype(np.float64))), rtol=2e-6, atol=1e-7)
    D = gauss_acts((M, N), seed=14)
    add = gpu_matmul(ops, fmt, W, A, N, K, out_dtype=torch.float32, binary="add", d=torch.from_numpy(D).cuda())
    assert np.array_equal(add, plain + D)


# cut_writeOutput's operator set (operators/impl/matmul/MatMulQ8Common.cuh:58-109) restated in float64 numpy
UNARY_F64 = {
    "neg": lambda x: -x, "abs": np.abs, "sqrt": np.sqrt, "square": lambda x: x * x, "reciprocal": lambda x: 1.0 / x,
    "exp": np.exp, "log": np.log, "tanh": np.tanh, "floor": np.floor, "ceil": np.ceil,
    "round": lambda x: np.sign(x) * np.floor(np.abs(x) + 0.5),   # half away from zero, as roundf
    "relu": lambda x: np.maximum(0.0, x), "sigmoid": lambda x: 1.0 / (1.0 + np.exp(-x)),
    "gelu": lambda x: x * 0.5 * (1.0 + np.tanh(np.sqrt(2.0 / 3.14159265) * (x + 0.044715 * x * x * x))),
    "silu": lambda x: x / (1.0 + np.exp(-x)), "softplus": lambda x: np.log(1.0 + np.exp(x)),
    "relu6": lambda x: np.clip(x, 0.0, 6.0), "mish": lambda x: x * np.tanh(np.log(1.0 + np.exp(x))),
    "hardswish": lambda x: x * np.clip(x / 6.0 + 0.5, 0.0, 1.0), "hardsigmoid": lambda x: np.clip(x / 6.0 + 0.5, 0.0, 1.0),
    "rsqrt": lambda x: 1.0 / np.sqrt(x),
}
BINARY_F64 = {
    "add": lambda a, b: a + b, "sub": lambda a, b: a - b, "mul": lambda a, b: a * b, "div": lambda a, b: a / b,
    "mod": lambda a, b: a - b * np.floor(a / b), "pow": lambda a, b: np.power(a, b), "floor_div": lambda a, b: np.floor(a / b),
    "min": np.minimum, "max": np.maximum,
}


@pytest.mark.parametrize("M", [1, 3, 64])   # the 8-row GEMV (direct epilogue), the same kernel's batch path, the tiled GEMM
@pytest.mark.parametrize("op", sorted(UNARY_F64))
def test_every_unary_fusion_op(ops, op, M):
    """All 21 unary operators of the reference's fused epilogue, applied to the matmul result, against the float64
    formula on the unfused GPU result (so the comparison isolates the operator; the matmul itself is checked
    elsewhere).  Inputs are scaled so that sqrt / log / rsqrt see both signs (NaN where the reference gives NaN)."""
    fmt = oracle.Q4_K
    N, K = 264, 512
    W = quantized_weights(fmt, N, K, seed=30)
    A = (gauss_acts((M, K), seed=31) * 4.0).astype(np.float16)
    plain = gpu_matmul(ops, fmt, W, A, N, K, out_dtype=torch.float32)
    got = gpu_matmul(ops, fmt, W, A, N, K, out_dtype=torch.float32, unary=op)
    with np.errstate(all="ignore"):
        want = UNARY_F64[op](plain.astype(np.float64))
    assert np.array_equal(np.isnan(got), np.isnan(want))
    ok = ~np.isnan(want)
    if op in ("floor", "ceil", "round", "neg", "abs", "relu", "relu6", "square"):
        assert np.array_equal(got[ok], want[ok].astype(np.float32))   # exact in fp32
    else:
        # the formulas are evaluated in fp32 on the device, as the reference does: log(1 + exp(x)) loses up to 2^-24
        # absolute in the sum, hence the absolute term
        np.testing.assert_allclose(got[ok], want[ok], rtol=1e-5, atol=1e-6)


@pytest.mark.parametrize("M", [1, 3, 64])
@pytest.mark.parametrize("op", sorted(BINARY_F64))
def test_every_binary_fusion_op(ops, op, M):
    """All 9 binary operators (matmul result op D) against float64."""
    fmt = oracle.Q4_K
    N, K = 264, 512
    W = quantized_weights(fmt, N, K, seed=32)
    A = (gauss_acts((M, K), seed=33) * 4.0).astype(np.float16)
    D = gauss_acts((M, N), seed=34) * np.float32(1.5)
    if op == "pow":
        D = np.round(D * 2.0).astype(np.float32)   # integer exponents: defined for negative bases too
    plain = gpu_matmul(ops, fmt, W, A, N, K, out_dtype=torch.float32)
    got = gpu_matmul(ops, fmt, W, A, N, K, out_dtype=torch.float32, binary=op, d=torch.from_numpy(D).cuda())
    with np.errstate(all="ignore"):
        want = BINARY_F64[op](plain.astype(np.float64), D.astype(np.float64))
    if op in ("add", "sub", "mul", "div", "min", "max"):
        assert np.array_equal(got, want.astype(np.float32))   # one correctly rounded fp32 operation
    elif op in ("mod", "floor_div"):
        # a / b is rounded to fp32 before floor: where the float64 quotient sits within an ulp of an integer the two may
        # legitimately differ by one step of b; everywhere else they agree
        q = plain.astype(np.float64) / D.astype(np.float64)
        safe = np.abs(q - np.round(q)) > 1e-5 * np.maximum(1.0, np.abs(q))
        np.testing.assert_allclose(got[safe], want[safe], rtol=2e-6, atol=2e-6)
        assert safe.mean() > 0.99
    else:
        fin = np.isfinite(want) & (np.abs(want) < 1e30)
        np.testing.assert_allclose(got[fin], want[fin], rtol=3e-6, atol=1e-30)


def test_unknown_fusion_operator_is_refused(ops):
    from cut_amd import lib
    L = lib.load()
    assert L.cuthip_epilogue_op_supported(lib.EPI_UNARY, 133) == 1 and L.cuthip_epilogue_op_supported(lib.EPI_UNARY, 105) == 0
    assert L.cuthip_epilogue_op_supported(lib.EPI_BINARY, 14) == 1 and L.cuthip_epilogue_op_supported(lib.EPI_BINARY, 7) == 0
    t = torch.zeros(1024, dtype=torch.float32, device="cuda")
    rc = L.cuthip_matmul_gguf(lib.Q4_K, t.data_ptr(), t.data_ptr(), lib.F32, t.data_ptr(), lib.F32, 1, 256, 4, 256, 4,
                              lib.EPI_UNARY, 105, None, -1, None)   # OP_UNARY_SIGN: not in cut_writeOutput
    assert rc == -1 and b"operator code 105" in L.cuthip_last_error()


def test_strided_a_and_c(ops):
    fmt = oracle.Q6_K
    N, K, M = 64, 512, 2
    W = quantized_weights(fmt, N, K, seed=20)
    A = gauss_acts((M, K), seed=21, dtype=np.float16)
    a_buf = torch.zeros((M, K + 24), dtype=torch.float16, device="cuda")
    a_buf[:, :K] = torch.from_numpy(A).cuda()
    c_buf = torch.full((M, N + 4), 7.0, dtype=torch.float32, device="cuda")
    ops.matmul_gguf(a_buf[:, :K], torch.from_numpy(W).cuda(), fmt, N, K, out=c_buf[:, :N])
    torch.cuda.synchronize()
    want = oracle.matmul_gguf(fmt, W, A.astype(np.float32), N, f64=True)
    assert normwise_rel_err(c_buf[:, :N].cpu().numpy(), want) < TOL_F16_ACT
    assert torch.all(c_buf[:, N:] == 7.0)


def test_reference_known_answers_on_native_blocks(ops):
    """The reference's q8_simple / q8_withscales cases (OpRegistry.h:1995-2026)
    re-expressed as GGUF Q8_0 rows: A = 1, weights 1 / 2 with scale 1 -> 32, 64;
    weights 4 with block scales {0.5, 1} and {2, 0.25} -> 192, 288."""
    def q8_rows(values, scales):  # values [N, K] int8, scales [N, K/32] float
        N, K = values.shape
        out = np.zeros((N, K // 32, 34), np.uint8)
        out[:, :, 0:2] = np.array(scales, np.float16).reshape(N, K // 32, 1).view(np.uint8)
        out[:, :, 2:] = values.reshape(N, K // 32, 32).view(np.uint8)
        return out.reshape(-1)
    W = q8_rows(np.stack([np.full(32, 1, np.int8), np.full(32, 2, np.int8)]), [[1.0], [1.0]])
    got = gpu_matmul(ops, oracle.Q8_0, W, np.ones((1, 32), np.float32), 2, 32)
    assert np.array_equal(got, [[32.0, 64.0]])
    W = q8_rows(np.full((2, 64), 4, np.int8), [[0.5, 1.0], [2.0, 0.25]])
    got = gpu_matmul(ops, oracle.Q8_0, W, np.ones((1, 64), np.float32), 2, 64)
    assert np.array_equal(got, [[192.0, 288.0]])


@pytest.mark.parametrize("name", list(oracle.FORMATS))
@pytest.mark.parametrize("M,N,K", [(1, 1, 256), (1, 7, 512), (2, 9, 256), (3, 1030, 1024), (5, 64, 4096), (8, 40, 2048),
                                  (1, 96, 14336), (2, 24, 14336), (1, 4100, 512)])
def test_rows8_kernel_shapes(ops, name, M, N, K):
    """The 8-row GEMV (variant 3) at its corner shapes: one row, fewer rows than a wave, a single K step, K split over
    2/4/8 waves, every batch size class (dot path, 4/8/16 accumulators), long K; it agrees with the oracle and with
    the fallback kernel (variant 0)."""
    fmt = oracle.FORMATS[name]
    W = quantized_weights(fmt, N, K, seed=N + K)
    A = gauss_acts((M, K), seed=M, dtype=np.float16)
    want = oracle.matmul_gguf(fmt, W, A.astype(np.float32), N, f64=True)
    got3 = gpu_matmul(ops, fmt, W, A, N, K, out_dtype=torch.float32, variant=3)
    got0 = gpu_matmul(ops, fmt, W, A, N, K, out_dtype=torch.float32, variant=0)
    assert normwise_rel_err(got3, want) < TOL_F16_ACT
    assert normwise_rel_err(got0, want) < TOL_F16_ACT


# (row groups, K ranges) of a workgroup with step counts the shape is chosen for: K ranges of unequal length, a range
# longer than one staging batch, and N that fills neither the last wave's 8 rows nor the last workgroup's row groups
FORCED_ROWS8 = [("4,1", 1024, [1, 2, 4, 8]), ("4,1", 4096 + 256, [1, 3, 8]), ("8,1", 2304, [1, 2, 5, 8]),
                ("2,2", 1024, [1, 2, 4, 8]), ("2,2", 2304, [1, 3, 8]), ("1,4", 2048, [1, 2, 4, 8]), ("1,4", 3328, [1, 7]),
                ("1,4", 4352, [1, 2, 4, 8]), ("2,4", 8448, [1, 2]), ("1,8", 4096, [1, 2, 4, 8]), ("1,8", 5376, [1, 4])]


@pytest.mark.parametrize("name", list(oracle.FORMATS))
@pytest.mark.parametrize("shape,K,batches", FORCED_ROWS8)
def test_rows8_every_workgroup_shape(ops, tuning, name, shape, K, batches):
    """Every workgroup shape of the 8-row GEMV, forced through cuthip_set_tuning instead of left to the
    choice by N and K (which reaches only one shape per problem), for every format and batch class, with a fused
    residual add: against the oracle."""
    tuning("rows8_shape", shape)
    fmt = oracle.FORMATS[name]
    N = 8 * 37 + 3
    W = quantized_weights(fmt, N, K, seed=K + 1)
    for M in batches:
        A = gauss_acts((M, K), seed=M + 40, dtype=np.float16)
        D = gauss_acts((M, N), seed=M + 80)
        want = oracle.matmul_gguf(fmt, W, A.astype(np.float32), N, f64=True)
        got = gpu_matmul(ops, fmt, W, A, N, K, out_dtype=torch.float32, variant=3)
        assert normwise_rel_err(got, want) < TOL_F16_ACT, (shape, K, M)
        got = gpu_matmul(ops, fmt, W, A, N, K, out_dtype=torch.float32, variant=3, binary="add", d=torch.from_numpy(D).cuda())
        assert normwise_rel_err(got - D, want) < 10 * TOL_F16_ACT, (shape, K, M)


@pytest.mark.parametrize("name", list(oracle.FORMATS))
@pytest.mark.parametrize("shape", ["1,1", "1,2", "1,4", "1,8", "2,1", "2,2", "2,4", "2,8"])
def test_fallback_gemv_every_workgroup_shape(ops, tuning, name, shape):
    """The fallback GEMV (variant 0; 32 weight rows per workgroup, or 16 with two K parts per wave) under every
    (parts, waves) shape, forced through cuthip_set_tuning: step counts that take the straight-line instances
    (2, 4 and 7 steps per wave) and the generic loop, batch 1 to 8 in one pass and 20 rows as a 32-row pass."""
    tuning("gemv_shape", shape)
    fmt = oracle.FORMATS[name]
    N = 3 * 32 + 5
    for K, batches in [(2048, [1, 2, 4, 8, 20]), (7168, [1, 3]), (2304, [1, 5, 20])]:
        W = quantized_weights(fmt, N, K, seed=K + 3)
        for M in batches:
            A = gauss_acts((M, K), seed=M + 60, dtype=np.float16)
            want = oracle.matmul_gguf(fmt, W, A.astype(np.float32), N, f64=True)
            got = gpu_matmul(ops, fmt, W, A, N, K, out_dtype=torch.float32, variant=0)
            assert normwise_rel_err(got, want) < TOL_F16_ACT, (shape, K, M)


@pytest.mark.parametrize("M", [1, 5, 8, 16, 17, 32])
@pytest.mark.parametrize("N,K", [(200, 2048), (70, 256), (1030, 4096), (64, 14336), (300, 8192 + 256)])
def test_streaming_mfma_matmul(ops, M, N, K):
    """Variant 6 (Q4_K, up to 32 rows): integer-scaled nibbles as fp16 subnormals through 16 x 16 x 32 MFMAs.  One and
    two activation tiles, ragged N, one step, K ranges split over workgroups (needs the workspace) with ranges of
    unequal length, fp16 and fp32 activations, a fused residual add: the products are exact, so the bound is that of
    the fp32 summation order."""
    fmt = oracle.Q4_K
    W = quantized_weights(fmt, N, K, seed=N + K)
    A = gauss_acts((M, K), seed=M + 3, dtype=np.float16)
    want = oracle.matmul_gguf(fmt, W, A.astype(np.float32), N, f64=True)
    a, w = torch.from_numpy(A).cuda(), torch.from_numpy(W).cuda()
    ws = ops.matmul_gguf_workspace(fmt, M, K, N, a.dtype, "cuda")
    ws.fill_(0xFF)
    got = ops.matmul_gguf(a, w, fmt, N, K, out_dtype=torch.float32, variant=6, workspace=ws)
    torch.cuda.synchronize()
    assert normwise_rel_err(got.cpu().numpy(), want) < TOL_F16_ACT
    D = gauss_acts((M, N), seed=M + 5, dtype=np.float16)
    got16 = ops.matmul_gguf(a, w, fmt, N, K, out_dtype=torch.float16, variant=6, workspace=ws, binary="add",
                            d=torch.from_numpy(D).cuda())
    torch.cuda.synchronize()
    assert normwise_rel_err(got16.float().cpu().numpy() - D.astype(np.float32), want) < 2e-3   # fp16 rounding of sum + D
    got32 = ops.matmul_gguf(a.float(), w, fmt, N, K, out_dtype=torch.float32, variant=6, workspace=ws)
    torch.cuda.synchronize()
    assert normwise_rel_err(got32.cpu().numpy(), want) < TOL_F16_ACT
    if K <= 4096 and M <= 16:      # one K range: no workspace needed
        alone = ops.matmul_gguf(a, w, fmt, N, K, out_dtype=torch.float32, variant=6)
        torch.cuda.synchronize()
        assert normwise_rel_err(alone.cpu().numpy(), want) < TOL_F16_ACT


def test_streaming_mfma_matmul_refusals(ops):
    from cut_amd import lib
    K, N = 512, 64
    a = torch.zeros((33, K), dtype=torch.float16, device="cuda")
    for fmt, rows in ((oracle.Q4_K, 33), (oracle.Q6_K, 8)):
        w = torch.from_numpy(quantized_weights(fmt, N, K, seed=1)).cuda()
        with pytest.raises(lib.CutHipError, match="variant 6"):
            ops.matmul_gguf(a[:rows], w, fmt, N, K, variant=6)
    w = torch.from_numpy(quantized_weights(oracle.Q4_K, 64, 14336, seed=2)).cuda()
    with pytest.raises(lib.CutHipError, match="scratch"):       # K = 14336 is split over workgroups: workspace needed
        ops.matmul_gguf(torch.zeros((8, 14336), dtype=torch.float16, device="cuda"), w, oracle.Q4_K, 64, 14336, variant=6)


def test_rows8_refuses_what_does_not_fit_and_auto_falls_back(ops):
    from cut_amd import lib
    fmt = oracle.Q4_K
    N, K, M = 64, 14336, 8      # 8 rows of 14336 fp16 activations exceed the LDS budget of the 8-row kernel
    W = quantized_weights(fmt, N, K, seed=1)
    A = gauss_acts((M, K), seed=2, dtype=np.float16)
    with pytest.raises(lib.CutHipError, match="variant 3"):
        gpu_matmul(ops, fmt, W, A, N, K, variant=3)
    want = oracle.matmul_gguf(fmt, W, A.astype(np.float32), N, f64=True)
    assert normwise_rel_err(gpu_matmul(ops, fmt, W, A, N, K, out_dtype=torch.float32), want) < TOL_F16_ACT


@pytest.mark.parametrize("fa,fb", [("Q4_K", "Q6_K"), ("Q6_K", "Q4_K"), ("Q4_K", "Q4_K"), ("Q6_K", "Q6_K"), ("Q8_0", "Q4_K"),
                                   ("Q4_0", "Q8_0")])
@pytest.mark.parametrize("Na,Nb,K", [(5120, 1024, 4096), (70, 9, 1024), (1, 1, 256), (20000, 8, 2048)])
def test_pair_launch_equals_two_matmuls(ops, fa, fb, Na, Nb, K):
    """Two weight tensors on one activation vector: one launch for the K-quant pairs at decode shapes, two launches
    otherwise; either way each output must match the oracle and the single matmul (same kernel body; only the
    split of K may differ)."""
    A = gauss_acts((1, K), seed=60, dtype=np.float16)
    a = torch.from_numpy(A).cuda()
    outs, singles = [], []
    ws = [torch.from_numpy(quantized_weights(oracle.FORMATS[f], n, K, seed=61 + i)).cuda() for i, (f, n) in
          enumerate(((fa, Na), (fb, Nb)))]
    ca = torch.full((Na,), 7.0, dtype=torch.float32, device="cuda")
    cb = torch.full((Nb,), 7.0, dtype=torch.float32, device="cuda")
    ops.matmul_gguf_pair(a.view(-1), ws[0], oracle.FORMATS[fa], Na, ca, ws[1], oracle.FORMATS[fb], Nb, cb, K)
    torch.cuda.synchronize()
    for f, n, w, c in ((fa, Na, ws[0], ca), (fb, Nb, ws[1], cb)):
        fmt = oracle.FORMATS[f]
        want = oracle.matmul_gguf(fmt, w.cpu().numpy(), A.astype(np.float32), n, f64=True)
        assert normwise_rel_err(c.cpu().numpy()[None, :], want) < (TOL_F16_ACT if n > 4 else 1e-4)
        single = ops.matmul_gguf(a, w, fmt, n, K, out_dtype=torch.float32)
        torch.cuda.synchronize()
        # the pair may pick another split of K than the single launch (it sizes the grid for both tensors)
        assert normwise_rel_err(c.cpu().numpy()[None, :], single.cpu().numpy()) < 2e-6


@pytest.mark.parametrize("name", list(oracle.FORMATS))
@pytest.mark.parametrize("M,N,K", [(2, 4096, 14336), (4, 4096, 14336), (8, 4096, 14336), (3, 4096, 14336), (3, 100, 8192), (5, 9, 8192 + 32),
                                   (2, 100, 8192 + 256)])
def test_batched_gemv_with_k_split_across_workgroups(ops, name, M, N, K):
    """Batch 2-8 on long rows with a workspace: K ranges go to different workgroups, fp32 partial products are summed by
    a second kernel, which also applies the epilogue.  Against the oracle (sampled columns for the big shapes) and
    against the launch without a workspace."""
    fmt = oracle.FORMATS[name]
    if K % oracle.BLOCK_ELEMS[fmt]:
        pytest.skip("K is not a multiple of this format's block")
    W = quantized_weights(fmt, N, K, seed=110)
    A = gauss_acts((M, K), seed=111, dtype=np.float16)
    D = gauss_acts((M, N), seed=112)
    a, w, d = torch.from_numpy(A).cuda(), torch.from_numpy(W).cuda(), torch.from_numpy(D).cuda()
    ws = ops.matmul_gguf_workspace(fmt, M, K, N, a.dtype, "cuda")
    ws.fill_(0xFF)
    got = ops.matmul_gguf(a, w, fmt, N, K, out_dtype=torch.float32, binary="add", d=d, workspace=ws)
    ref = ops.matmul_gguf(a, w, fmt, N, K, out_dtype=torch.float32, binary="add", d=d)
    h16 = ops.matmul_gguf(a, w, fmt, N, K, out_dtype=torch.float16, workspace=ws)
    torch.cuda.synchronize()
    got, ref = got.cpu().numpy(), ref.cpu().numpy()
    assert normwise_rel_err(got - D, ref - D) < 2e-5
    cols = np.unique(np.concatenate([[0, N - 1], np.random.default_rng(7).integers(0, N, min(N, 96))]))
    Ws = np.ascontiguousarray(W.reshape(N, oracle.n_bytes(fmt, K))[cols]).reshape(-1)
    want = oracle.matmul_gguf(fmt, Ws, A.astype(np.float32), len(cols), f64=True)
    assert normwise_rel_err(got[:, cols] - D[:, cols], want) < TOL_F16_ACT
    assert normwise_rel_err(h16.float().cpu().numpy(), ref - D) < 4e-4   # fp16 output rounding


@pytest.mark.parametrize("name", list(oracle.FORMATS))
@pytest.mark.parametrize("M,N,K", [(8, 16, 90112), (7, 16384, 8192), (5, 12288, 8192), (3, 256, 28672)])
def test_batched_gemv_k_split_where_the_activations_exceed_lds(ops, name, M, N, K):
    """Batch rows x K beyond what one workgroup stages in LDS: with a workspace the K split takes as many parts as it
    needs for one part to fit (8 rows of K = 90112: 32 parts; 7 rows of K = 8192 on 16384 weight rows: 2 parts, where
    the chip would be full without any), whatever the number of weight rows.  Against the oracle on sampled columns and
    against the launch without a workspace (the 32-row fallback kernel).  The weights repeat a block of 256 rows."""
    fmt = oracle.FORMATS[name]
    rows = min(N, 256)
    tile = quantized_weights(fmt, rows, K, seed=140)
    W = np.tile(tile, N // rows)
    A = gauss_acts((M, K), seed=141, dtype=np.float16)
    a, w = torch.from_numpy(A).cuda(), torch.from_numpy(W).cuda()
    ws = ops.matmul_gguf_workspace(fmt, M, K, N, a.dtype, "cuda")
    assert ws is not None and ws.numel() > 0
    ws.fill_(0xFF)
    got = ops.matmul_gguf(a, w, fmt, N, K, out_dtype=torch.float32, workspace=ws)
    ref = ops.matmul_gguf(a, w, fmt, N, K, out_dtype=torch.float32)
    torch.cuda.synchronize()
    got, ref = got.cpu().numpy(), ref.cpu().numpy()
    assert normwise_rel_err(got, ref) < 2e-5
    cols = np.unique(np.concatenate([[0, N - 1], np.random.default_rng(8).integers(0, N, min(N, 64))]))
    Ws = np.ascontiguousarray(W.reshape(N, oracle.n_bytes(fmt, K))[cols]).reshape(-1)
    want = oracle.matmul_gguf(fmt, Ws, A.astype(np.float32), len(cols), f64=True)
    assert normwise_rel_err(got[:, cols], want) < TOL_F16_ACT


@pytest.mark.parametrize("name", list(oracle.FORMATS))
@pytest.mark.parametrize("M", [9, 19, 40])
def test_mid_size_batches_run_as_eight_row_passes(ops, name, M):
    """9-40 rows with the automatic choice: passes of 8 rows through the decode kernel, with strided A / C / D and a
    binary epilogue, so that a wrong row offset in any of the three operands shows."""
    fmt = oracle.FORMATS[name]
    N, K = 100, 1024
    W = quantized_weights(fmt, N, K, seed=130)
    A = gauss_acts((M, K), seed=131, dtype=np.float16)
    D = gauss_acts((M, N), seed=132)
    a_buf = torch.zeros((M, K + 8), dtype=torch.float16, device="cuda")
    a_buf[:, :K] = torch.from_numpy(A).cuda()
    d_buf = torch.zeros((M, N + 4), dtype=torch.float32, device="cuda")
    d_buf[:, :N] = torch.from_numpy(D).cuda()
    c_buf = torch.full((M, N + 4), 7.0, dtype=torch.float32, device="cuda")
    ops.matmul_gguf(a_buf[:, :K], torch.from_numpy(W).cuda(), fmt, N, K, out=c_buf[:, :N], binary="add", d=d_buf[:, :N])
    torch.cuda.synchronize()
    want = oracle.matmul_gguf(fmt, W, A.astype(np.float32), N, f64=True)
    assert normwise_rel_err(c_buf[:, :N].cpu().numpy() - D, want) < TOL_F16_ACT
    assert torch.all(c_buf[:, N:] == 7.0)


@pytest.mark.parametrize("M", [16, 32])
def test_streaming_kernel_rounds_fp32_activations_to_fp16(ops, M):
    """Variant 6 stages fp32 activations as fp16, nearest even: against the float64 oracle on the fp32 values the result
    carries that rounding (2^-11 relative per element, a few 1e-4 normwise); against the oracle on the rounded values it
    is as tight as with fp16 inputs, and bit-identical to the kernel fed the rounded values as fp16.  The automatic
    choice (at this small N the tiled kernel, which also decodes the weights to fp16) is held to the first bound only."""
    fmt = oracle.Q4_K
    N, K = 520, 2048
    W = quantized_weights(fmt, N, K, seed=170)
    A = gauss_acts((M, K), seed=171)
    a, w = torch.from_numpy(A).cuda(), torch.from_numpy(W).cuda()
    ws = ops.matmul_gguf_workspace(fmt, M, K, N, a.dtype, "cuda")
    rounded = A.astype(np.float16)
    want32 = oracle.matmul_gguf(fmt, W, A, N, f64=True)
    want16 = oracle.matmul_gguf(fmt, W, rounded.astype(np.float32), N, f64=True)
    assert normwise_rel_err(want16, want32) > 5 * TOL_F16_ACT      # the two bounds tell the roundings apart
    got = ops.matmul_gguf(a, w, fmt, N, K, out_dtype=torch.float32, workspace=ws, variant=6)
    torch.cuda.synchronize()
    got = got.cpu().numpy()
    assert normwise_rel_err(got, want32) < TOL_F32_ACT
    assert normwise_rel_err(got, want16) < TOL_F16_ACT
    same = ops.matmul_gguf(torch.from_numpy(rounded).cuda(), w, fmt, N, K, out_dtype=torch.float32, workspace=ws, variant=6)
    torch.cuda.synchronize()
    assert np.array_equal(got, same.cpu().numpy())
    auto = ops.matmul_gguf(a, w, fmt, N, K, out_dtype=torch.float32, workspace=ws)
    torch.cuda.synchronize()
    assert normwise_rel_err(auto.cpu().numpy(), want32) < TOL_F32_ACT


@pytest.mark.parametrize("op", ["mod", "pow", "floor_div"])
def test_long_binary_operator_refuses_aliased_operand_before_writing(ops, op):
    """The operators that run as a launch of their own after the matmul need D intact: D == C is refused by every
    entry point before the unfused matmul is launched, so the caller's buffer still holds D."""
    from cut_amd import lib
    fmt = oracle.Q4_K
    N, K, M = 64, 512, 3
    w = torch.from_numpy(quantized_weights(fmt, N, K, seed=180)).cuda()
    a = torch.from_numpy(gauss_acts((M, K), seed=181, dtype=np.float16)).cuda()
    d0 = gauss_acts((M, N), seed=182)
    c = torch.from_numpy(d0.copy()).cuda()
    ws = ops.matmul_gguf_workspace(fmt, M, K, N, a.dtype, "cuda")
    L = lib.load()
    rc = L.cuthip_matmul_gguf(fmt, w.data_ptr(), a.data_ptr(), lib.F16, c.data_ptr(), lib.F32, M, K, N, K, N, lib.EPI_BINARY,
                              lib.BINARY[op], c.data_ptr(), -1, None)
    assert rc != 0 and b"alias" in L.cuthip_last_error()
    rc = L.cuthip_matmul_gguf_ws(fmt, w.data_ptr(), a.data_ptr(), lib.F16, c.data_ptr(), lib.F32, M, K, N, K, N, lib.EPI_BINARY,
                                 lib.BINARY[op], c.data_ptr(), -1, ws.data_ptr(), ws.numel(), None)
    assert rc != 0 and b"alias" in L.cuthip_last_error()
    torch.cuda.synchronize()
    assert np.array_equal(c.cpu().numpy(), d0)
