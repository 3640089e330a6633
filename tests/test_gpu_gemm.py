"""GPU parity: the LDS-tiled MFMA GEMM (prefill path, M > 32) through the C
ABI against the CPU oracle.  Weights are rounded to fp16 after the fp32 decode
(2^-11 relative), activations are fp16: the asserted normwise bound is 5e-4,
inside the 1e-3 the baseline states."""
import numpy as np
import pytest

import oracle
from helpers import gauss_acts, normwise_rel_err, quantized_weights

torch = pytest.importorskip("torch")
pytestmark = pytest.mark.gpu

TOL = 1e-3
TOL_GEMM = 5e-4


@pytest.fixture(scope="module")
def ops():
    from cut_amd import lib, ops as _ops
    lib.check(lib.load().cuthip_init(0))
    return _ops


def gpu_matmul(ops, fmt, W, A, N, K, out_dtype=None, **kw):
    c = ops.matmul_gguf(torch.from_numpy(A).cuda(), torch.from_numpy(W).cuda(), fmt, N, K, out_dtype=out_dtype, **kw)
    torch.cuda.synchronize()
    return c.float().cpu().numpy()


@pytest.mark.parametrize("name", list(oracle.FORMATS))
@pytest.mark.parametrize("M,N,K", [(33, 200, 1024), (128, 128, 256), (300, 384, 2048)])
def test_gemm_vs_oracle(ops, name, M, N, K):
    fmt = oracle.FORMATS[name]
    W = quantized_weights(fmt, N, K, seed=11)
    A = gauss_acts((M, K), seed=12, dtype=np.float16)
    got = gpu_matmul(ops, fmt, W, A, N, K, out_dtype=torch.float32)
    want = oracle.matmul_gguf(fmt, W, A.astype(np.float32), N, f64=True)
    err = normwise_rel_err(got, want)
    assert err < TOL_GEMM, err
    assert normwise_rel_err(got, oracle.matmul_gguf(fmt, W, A.astype(np.float32), N)) < TOL


@pytest.mark.parametrize("name,K", [("Q8_0", 96), ("Q4_0", 160), ("Q4_K", 768)])
def test_gemm_ragged_k_and_fp32_activations(ops, name, K):
    fmt = oracle.FORMATS[name]
    M, N = 70, 130
    W = quantized_weights(fmt, N, K, seed=5)
    A = gauss_acts((M, K), seed=6)
    got = gpu_matmul(ops, fmt, W, A, N, K)
    want = oracle.matmul_gguf(fmt, W, A, N, f64=True)
    assert normwise_rel_err(got, want) < 8e-4  # activations and weights both rounded to fp16


def test_gemm_variants_agree(ops):
    """The same problem through the GEMM (variant 2) and the skinny passes
    (variant 1): the reference checks batched against per-row the same way
    (RuntimeTests.cpp:2861-2938)."""
    fmt = oracle.Q4_K
    M, N, K = 40, 256, 1024
    W = quantized_weights(fmt, N, K, seed=21)
    A = gauss_acts((M, K), seed=22, dtype=np.float16)
    g = gpu_matmul(ops, fmt, W, A, N, K, out_dtype=torch.float32, variant=2)
    s = gpu_matmul(ops, fmt, W, A, N, K, out_dtype=torch.float32, variant=1)
    want = oracle.matmul_gguf(fmt, W, A.astype(np.float32), N, f64=True)
    assert normwise_rel_err(g, want) < TOL_GEMM and normwise_rel_err(s, want) < 2e-5
    assert np.all(np.abs(g - s) <= np.abs(s) * 2e-3 + 2e-3)


def test_gemm_epilogues_and_fp16_out(ops):
    fmt = oracle.Q4_K
    M, N, K = 96, 256, 512
    W = quantized_weights(fmt, N, K, seed=31)
    A = gauss_acts((M, K), seed=32, dtype=np.float16)
    plain = gpu_matmul(ops, fmt, W, A, N, K, out_dtype=torch.float32)
    silu = gpu_matmul(ops, fmt, W, A, N, K, out_dtype=torch.float32, unary="silu")
    assert np.allclose(silu, plain / (1 + np.exp(-plain.astype(np.float64))), rtol=2e-6, atol=1e-7)
    D = gauss_acts((M, N), seed=33)
    add = gpu_matmul(ops, fmt, W, A, N, K, out_dtype=torch.float32, binary="add", d=torch.from_numpy(D).cuda())
    assert np.array_equal(add, plain + D)
    h = gpu_matmul(ops, fmt, W, A, N, K)  # fp16 out
    assert np.array_equal(h, plain.astype(np.float16).astype(np.float32))


@pytest.mark.parametrize("M", [512, 2048])
def test_prefill_shape_sampled(ops, M):
    """BASELINE config 5 geometry (K = 4096, N = 14336) on a sample of output
    rows and columns; the oracle cost is kept to seconds by slicing W and A."""
    fmt = oracle.Q4_K
    N, K = 14336, 4096
    W = quantized_weights(fmt, N, K, seed=0)
    A = gauss_acts((M, K), seed=1, dtype=np.float16)
    got = gpu_matmul(ops, fmt, W, A, N, K)  # fp16 out
    rng = np.random.default_rng(3)
    rows = np.unique(np.concatenate([[0, M - 1], rng.integers(0, M, 14)]))
    cols = np.unique(np.concatenate([np.arange(0, 32), np.arange(N - 32, N), rng.integers(0, N, 192)]))
    rb = oracle.n_bytes(fmt, K)
    Ws = np.ascontiguousarray(W.reshape(N, rb)[cols]).reshape(-1)
    want = oracle.matmul_gguf(fmt, Ws, A[rows].astype(np.float32), len(cols), f64=True)
    err = normwise_rel_err(got[np.ix_(rows, cols)], want)
    assert err < 8e-4, err  # fp16 weights (3e-4) and fp16 output rounding (3e-4)


# ---- variant 4: dequantize once to an fp16 workspace, then a dense fp16 MFMA GEMM --------------------------------

def gpu_matmul_ws(ops, fmt, W, A, N, K, out_dtype=None, variant=4, **kw):
    a = torch.from_numpy(A).cuda()
    ws = ops.matmul_gguf_workspace(fmt, a.shape[0], K, N, a.dtype, "cuda")
    ws.fill_(0xFF)  # the workspace is scratch: stale contents (NaN patterns) must not leak into C
    c = ops.matmul_gguf(a, torch.from_numpy(W).cuda(), fmt, N, K, out_dtype=out_dtype, variant=variant, workspace=ws, **kw)
    torch.cuda.synchronize()
    return c.float().cpu().numpy()


@pytest.mark.parametrize("name", list(oracle.FORMATS))
@pytest.mark.parametrize("M,N,K", [(1, 1, 256), (70, 130, 256), (300, 520, 1024), (512, 768, 512), (129, 2056, 256)])
def test_dense_gemm_vs_oracle(ops, name, M, N, K):
    """Ragged tiles on both sides (M, N not multiples of 128 / 256), one to eight slices of K, N-tile counts that are
    and are not multiples of 8 (both workgroup orders), 128- and 256-row tiles."""
    fmt = oracle.FORMATS[name]
    W = quantized_weights(fmt, N, K, seed=41)
    A = gauss_acts((M, K), seed=42, dtype=np.float16)
    got = gpu_matmul_ws(ops, fmt, W, A, N, K, out_dtype=torch.float32)
    want = oracle.matmul_gguf(fmt, W, A.astype(np.float32), N, f64=True)
    err = normwise_rel_err(got, want)
    assert err < (TOL_GEMM if M * N >= 1024 else TOL), err  # a single output has no averaging over elements
    assert normwise_rel_err(got, oracle.matmul_gguf(fmt, W, A.astype(np.float32), N)) < TOL


def test_dense_gemm_256_row_tiles_and_single_launch_gemm_agree(ops):
    """Enough tiles for the 256-row kernel (>= 256 tiles of 256 x 256), checked on sampled rows / columns against the
    oracle and everywhere against the single-launch GEMM (fp16 weights and activations, fp32 accumulation in both)."""
    fmt = oracle.Q4_K
    M, N, K = 2100, 8200, 256
    W = quantized_weights(fmt, N, K, seed=43)
    A = gauss_acts((M, K), seed=44, dtype=np.float16)
    got = gpu_matmul_ws(ops, fmt, W, A, N, K, out_dtype=torch.float32)
    ref = gpu_matmul(ops, fmt, W, A, N, K, out_dtype=torch.float32, variant=2)
    # the dequant kernel rounds the reference's exact fp32 expression, the single-launch GEMM a contracted one: a few
    # weights differ by one fp16 ulp
    assert normwise_rel_err(got, ref) < 2e-4
    assert np.all(np.abs(got - ref) <= 2e-3 * np.abs(ref) + 1e-3)
    rng = np.random.default_rng(5)
    rows = np.unique(np.concatenate([[0, 255, 256, M - 1], rng.integers(0, M, 12)]))
    cols = np.unique(np.concatenate([[0, 255, 256, N - 1], rng.integers(0, N, 200)]))
    Ws = np.ascontiguousarray(W.reshape(N, oracle.n_bytes(fmt, K))[cols]).reshape(-1)
    want = oracle.matmul_gguf(fmt, Ws, A[rows].astype(np.float32), len(cols), f64=True)
    assert normwise_rel_err(got[np.ix_(rows, cols)], want) < TOL_GEMM


def test_dense_gemm_fp32_activations_strides_epilogues(ops):
    fmt = oracle.Q6_K
    M, N, K = 200, 300, 512
    W = quantized_weights(fmt, N, K, seed=45)
    A = gauss_acts((M, K), seed=46)
    want = oracle.matmul_gguf(fmt, W, A, N, f64=True)
    w = torch.from_numpy(W).cuda()
    a_buf = torch.zeros((M, K + 8), dtype=torch.float32, device="cuda")
    a_buf[:, :K] = torch.from_numpy(A).cuda()
    c_buf = torch.full((M, N + 4), 7.0, dtype=torch.float32, device="cuda")
    ws = ops.matmul_gguf_workspace(fmt, M, K, N, torch.float32, "cuda")
    ops.matmul_gguf(a_buf[:, :K], w, fmt, N, K, out=c_buf[:, :N], variant=4, workspace=ws)
    torch.cuda.synchronize()
    plain = c_buf[:, :N].cpu().numpy()
    assert normwise_rel_err(plain, want) < 8e-4  # activations and weights both rounded to fp16
    assert torch.all(c_buf[:, N:] == 7.0)
    D = gauss_acts((M, N), seed=47)
    add = ops.matmul_gguf(torch.from_numpy(A).cuda(), w, fmt, N, K, binary="add", d=torch.from_numpy(D).cuda(), variant=4,
                          workspace=ws)
    silu = ops.matmul_gguf(torch.from_numpy(A).cuda(), w, fmt, N, K, unary="silu", variant=4, workspace=ws)
    h = ops.matmul_gguf(torch.from_numpy(A).cuda(), w, fmt, N, K, out_dtype=torch.float16, variant=4, workspace=ws)
    torch.cuda.synchronize()
    assert np.array_equal(add.cpu().numpy(), plain + D)
    assert np.allclose(silu.cpu().numpy(), plain / (1 + np.exp(-plain.astype(np.float64))), rtol=2e-6, atol=1e-7)
    assert np.array_equal(h.float().cpu().numpy(), plain.astype(np.float16).astype(np.float32))


def test_dense_gemm_refusals_and_automatic_choice(ops):
    from cut_amd import lib
    fmt = oracle.Q8_0
    M, N, K = 64, 64, 192  # K not a multiple of 128
    W = quantized_weights(fmt, N, K, seed=48)
    A = gauss_acts((M, K), seed=49, dtype=np.float16)
    with pytest.raises(lib.CutHipError, match="multiple of 128"):
        gpu_matmul_ws(ops, fmt, W, A, N, K)
    # the automatic choice falls back to the single-launch kernels for the same call
    got = gpu_matmul_ws(ops, fmt, W, A, N, K, out_dtype=torch.float32, variant=-1)
    assert normwise_rel_err(got, oracle.matmul_gguf(fmt, W, A.astype(np.float32), N, f64=True)) < TOL_GEMM
    K = 256
    W = quantized_weights(fmt, N, K, seed=48)
    A = gauss_acts((M, K), seed=49, dtype=np.float16)
    a, w = torch.from_numpy(A).cuda(), torch.from_numpy(W).cuda()
    with pytest.raises(lib.CutHipError, match="workspace"):
        ops.matmul_gguf(a, w, fmt, N, K, variant=4, workspace=torch.empty(1024, dtype=torch.uint8, device="cuda"))
    with pytest.raises(lib.CutHipError, match="cuthip_matmul_gguf_ws"):
        ops.matmul_gguf(a, w, fmt, N, K, variant=4)
    # automatic: M >= 1024 with a workspace takes the two-pass path
    M = 1100
    A = gauss_acts((M, K), seed=50, dtype=np.float16)
    auto = gpu_matmul_ws(ops, fmt, W, A, N, K, out_dtype=torch.float32, variant=-1)
    assert normwise_rel_err(auto, oracle.matmul_gguf(fmt, W, A.astype(np.float32), N, f64=True)) < TOL_GEMM


@pytest.mark.parametrize("M,N,K", [(2048, 14336, 4096), (512, 14336, 4096), (2048, 4096, 14336), (512, 4096, 14336)])
def test_dense_gemm_prefill_shapes_sampled(ops, M, N, K):
    """BASELINE config 5 geometry through the two-pass path, on a sample of output rows and columns."""
    fmt = oracle.Q4_K
    W = quantized_weights(fmt, N, K, seed=0)
    A = gauss_acts((M, K), seed=1, dtype=np.float16)
    got = gpu_matmul_ws(ops, fmt, W, A, N, K)  # fp16 out
    rng = np.random.default_rng(3)
    rows = np.unique(np.concatenate([[0, M - 1], rng.integers(0, M, 14)]))
    cols = np.unique(np.concatenate([np.arange(0, 32), np.arange(N - 32, N), rng.integers(0, N, 192)]))
    Ws = np.ascontiguousarray(W.reshape(N, oracle.n_bytes(fmt, K))[cols]).reshape(-1)
    want = oracle.matmul_gguf(fmt, Ws, A[rows].astype(np.float32), len(cols), f64=True)
    err = normwise_rel_err(got[np.ix_(rows, cols)], want)
    assert err < 8e-4, err


def test_dense_gemm_128x448_tiles(ops):
    """The tile shape chosen when it makes whole rounds over the CUs (N a multiple of 448, 256 tiles): sampled rows and
    columns against the oracle, every output against the single-launch GEMM."""
    fmt = oracle.Q4_K
    M, N, K = 4096 - 5, 3584, 512   # ragged last row tile
    W = quantized_weights(fmt, N, K, seed=51)
    A = gauss_acts((M, K), seed=52, dtype=np.float16)
    got = gpu_matmul_ws(ops, fmt, W, A, N, K, out_dtype=torch.float32)
    ref = gpu_matmul(ops, fmt, W, A, N, K, out_dtype=torch.float32, variant=2)
    assert normwise_rel_err(got, ref) < 2e-4
    assert np.all(np.abs(got - ref) <= 2e-3 * np.abs(ref) + 1e-3)
    rng = np.random.default_rng(6)
    rows = np.unique(np.concatenate([[0, 127, 128, M - 1], rng.integers(0, M, 12)]))
    cols = np.unique(np.concatenate([[0, 223, 224, 447, 448, N - 1], rng.integers(0, N, 200)]))
    Ws = np.ascontiguousarray(W.reshape(N, oracle.n_bytes(fmt, K))[cols]).reshape(-1)
    want = oracle.matmul_gguf(fmt, Ws, A[rows].astype(np.float32), len(cols), f64=True)
    assert normwise_rel_err(got[np.ix_(rows, cols)], want) < TOL_GEMM


@pytest.mark.parametrize("name,K", [("Q4_K", 4096), ("Q6_K", 2048), ("Q8_0", 4128), ("Q4_0", 2080), ("Q4_K", 14336)])
@pytest.mark.parametrize("M", [9, 70, 128, 200])
def test_tiled_gemm_splits_k_through_the_workspace(ops, tuning, name, K, M):
    """The single-launch GEMM (variant 2) with a workspace at hand: few tiles, so K is split over workgroups (fp32
    partial products, summed by the reduce kernel, which also applies the epilogue).  Ragged tiles, a K whose last
    range ends in a partial slice, fp16 and fp32 activations, the residual add, and a forced split of 3 ranges of
    unequal length: against the oracle and the unsplit launch."""
    fmt = oracle.FORMATS[name]
    N = 300
    W = quantized_weights(fmt, N, K, seed=K + M)
    A = gauss_acts((M, K), seed=M + 7, dtype=np.float16)
    want = oracle.matmul_gguf(fmt, W, A.astype(np.float32), N, f64=True)
    unsplit = gpu_matmul(ops, fmt, W, A, N, K, out_dtype=torch.float32, variant=2)
    got = gpu_matmul_ws(ops, fmt, W, A, N, K, out_dtype=torch.float32, variant=2)
    assert normwise_rel_err(got, want) < TOL_GEMM
    assert normwise_rel_err(got, unsplit) < 1e-6      # the same products, summed in another order
    auto = gpu_matmul_ws(ops, fmt, W, A, N, K, out_dtype=torch.float32, variant=-1)
    assert normwise_rel_err(auto, want) < TOL_GEMM
    D = gauss_acts((M, N), seed=M + 9, dtype=np.float16)
    got16 = gpu_matmul_ws(ops, fmt, W, A, N, K, out_dtype=torch.float16, variant=2, binary="add", d=torch.from_numpy(D).cuda())
    assert normwise_rel_err(got16 - D.astype(np.float32), want) < 2e-3   # fp16 rounding of sum + D
    got32 = gpu_matmul_ws(ops, fmt, W, A.astype(np.float32), N, K, out_dtype=torch.float32, variant=2)
    assert normwise_rel_err(got32, want) < TOL_GEMM
    tuning("gemm_ksplit", "3")
    got3 = gpu_matmul_ws(ops, fmt, W, A, N, K, out_dtype=torch.float32, variant=2)
    assert normwise_rel_err(got3, unsplit) < 1e-6


@pytest.mark.parametrize("mfma16", ["1", "0"])
@pytest.mark.parametrize("tile", ["256,224", "128,448", "256,256", "128,256", "128,256,2", "256,256,4"])
def test_dense_gemm_every_tile_shape_and_both_kernels(ops, tuning, tile, mfma16):
    """Every tile shape of the dense GEMM (with and without a K split) under both of its kernels (16 x 16 x 32 MFMAs,
    the default, and 32 x 32 x 16), forced through cuthip_set_tuning, on a problem with ragged tiles on
    both sides: every output against the single-launch GEMM, sampled rows and columns against the oracle, and the
    residual-add epilogue (the short output loop with an operand)."""
    tuning("dense_tile", tile)
    tuning("dense_mfma16", mfma16)
    fmt = oracle.Q4_K
    bn = int(tile.split(",")[1])
    M, N, K = 700, 3 * bn - 8, 1024
    W = quantized_weights(fmt, N, K, seed=151)
    A = gauss_acts((M, K), seed=152, dtype=np.float16)
    got = gpu_matmul_ws(ops, fmt, W, A, N, K, out_dtype=torch.float16)
    ref = gpu_matmul(ops, fmt, W, A, N, K, out_dtype=torch.float32, variant=2)
    assert normwise_rel_err(got, ref) < 5e-4      # fp16 output rounding
    rng = np.random.default_rng(7)
    rows = np.unique(np.concatenate([[0, 255, 256, M - 1], rng.integers(0, M, 12)]))
    cols = np.unique(np.concatenate([[0, bn - 1, bn, N - 1], rng.integers(0, N, 150)]))
    Ws = np.ascontiguousarray(W.reshape(N, oracle.n_bytes(fmt, K))[cols]).reshape(-1)
    want = oracle.matmul_gguf(fmt, Ws, A[rows].astype(np.float32), len(cols), f64=True)
    assert normwise_rel_err(got[np.ix_(rows, cols)], want) < TOL_GEMM
    D = gauss_acts((M, N), seed=153, dtype=np.float16)
    with_d = gpu_matmul_ws(ops, fmt, W, A, N, K, out_dtype=torch.float16, binary="add", d=torch.from_numpy(D).cuda())
    assert normwise_rel_err(with_d - D.astype(np.float32), ref) < 1e-3


def test_workspace_paths_under_hip_graph_replay(ops):
    """The two-pass GEMM (dequant + GEMM, with and without split K) and the K-split batched GEMV captured into one HIP
    graph and replayed with eager work in between: every replay equals the eager result (no allocation, no host
    dependence inside the calls)."""
    fmt = oracle.Q4_K
    cases = [(1100, 520, 512), (300, 256, 2048), (4, 200, 8192)]   # dense, dense with split K, K-split GEMV
    bufs = []
    for M, N, K in cases:
        w = torch.from_numpy(quantized_weights(fmt, N, K, seed=120 + M)).cuda()
        a = torch.from_numpy(gauss_acts((M, K), seed=121, dtype=np.float16)).cuda()
        ws = ops.matmul_gguf_workspace(fmt, M, K, N, a.dtype, "cuda")
        out = torch.empty((M, N), dtype=torch.float32, device="cuda")
        bufs.append((M, N, K, w, a, ws, out))

    def run():
        for M, N, K, w, a, ws, out in bufs:
            ops.matmul_gguf(a, w, fmt, N, K, out=out, workspace=ws)
    run()
    torch.cuda.synchronize()
    eager = [b[6].clone() for b in bufs]
    g = torch.cuda.CUDAGraph()
    with torch.cuda.graph(g):
        run()
    for rep in range(3):
        for b in bufs:
            b[6].zero_()
            b[5].fill_(rep)   # the workspace is scratch: its contents between calls do not matter
        torch.cuda.synchronize()
        g.replay()
        torch.cuda.synchronize()
        for b, e in zip(bufs, eager):
            assert torch.equal(b[6], e)
    for (M, N, K, w, a, ws, out), e in zip(bufs, eager):
        want = oracle.matmul_gguf(fmt, w.cpu().numpy(), a.float().cpu().numpy(), N, f64=True)
        assert normwise_rel_err(e.cpu().numpy(), want) < TOL_GEMM


# ---- variant 5: dequantize once, then the vendor library's dense fp16 GEMM ----------------------------------------

@pytest.mark.parametrize("name", list(oracle.FORMATS))
@pytest.mark.parametrize("M,N,K", [(70, 136, 256), (300, 520, 1024), (512, 768, 512), (1030, 2056, 256)])
def test_blaslt_gemm_vs_oracle(ops, name, M, N, K):
    fmt = oracle.FORMATS[name]
    W = quantized_weights(fmt, N, K, seed=51)
    A = gauss_acts((M, K), seed=52, dtype=np.float16)
    want = oracle.matmul_gguf(fmt, W, A.astype(np.float32), N, f64=True)
    got = gpu_matmul_ws(ops, fmt, W, A, N, K, out_dtype=torch.float32, variant=5)
    assert normwise_rel_err(got, want) < TOL_GEMM
    got16 = gpu_matmul_ws(ops, fmt, W, A, N, K, out_dtype=torch.float16, variant=5)
    assert normwise_rel_err(got16, want) < TOL
    # the same dequantized weights through the hand-written GEMM: fp32 accumulation on both sides
    own = gpu_matmul_ws(ops, fmt, W, A, N, K, out_dtype=torch.float32, variant=4)
    assert normwise_rel_err(got, own) < 1e-5


def test_blaslt_gemm_fp32_activations_and_automatic_choice(ops):
    fmt = oracle.Q4_K
    M, N, K = 1100, 520, 512
    W = quantized_weights(fmt, N, K, seed=53)
    A = gauss_acts((M, K), seed=54)
    want = oracle.matmul_gguf(fmt, W, A, N, f64=True)
    assert normwise_rel_err(gpu_matmul_ws(ops, fmt, W, A, N, K, variant=5), want) < 8e-4
    # the automatic choice never takes the vendor library (that is opt-in): it is the hand-written two-pass GEMM, bit for bit
    auto = gpu_matmul_ws(ops, fmt, W, A, N, K, variant=-1)
    assert normwise_rel_err(auto, want) < 8e-4
    assert np.array_equal(auto, gpu_matmul_ws(ops, fmt, W, A, N, K, variant=4))
    D = gauss_acts((M, N), seed=55)
    add = gpu_matmul_ws(ops, fmt, W, A, N, K, variant=-1, binary="add", d=torch.from_numpy(D).cuda())
    assert normwise_rel_err(add, want + D) < 8e-4
    from cut_amd import lib
    with pytest.raises(lib.CutHipError, match="no fused epilogue"):
        gpu_matmul_ws(ops, fmt, W, A, N, K, variant=5, unary="silu")


def test_blaslt_gemm_under_graph_replay(ops):
    fmt = oracle.Q4_K
    M, N, K = 1024, 1024, 512
    W = torch.from_numpy(quantized_weights(fmt, N, K, seed=56)).cuda()
    a = torch.from_numpy(gauss_acts((M, K), seed=57, dtype=np.float16)).cuda()
    ws = ops.matmul_gguf_workspace(fmt, M, K, N, a.dtype, "cuda")
    c = torch.empty((M, N), dtype=torch.float16, device="cuda")
    ops.matmul_gguf(a, W, fmt, N, K, out=c, variant=5, workspace=ws)
    torch.cuda.synchronize()
    eager = c.clone()
    g = torch.cuda.CUDAGraph()
    with torch.cuda.graph(g):
        ops.matmul_gguf(a, W, fmt, N, K, out=c, variant=5, workspace=ws)
    for _ in range(3):
        c.zero_()
        ws.fill_(0xFF)
        torch.cuda.synchronize()
        g.replay()
        torch.cuda.synchronize()
        assert torch.equal(c, eager)


def test_tuning_rules_select_the_variant(ops, tmp_path):
    """ops.enable_tuning: an exact-shape rule of the "hip" section decides the variant of a call with variant = -1."""
    import json
    fmt = oracle.Q4_K
    M, N, K = 48, 512, 512
    rules = {"operators": {"MatMulGgufQ4_K": {"backends": {"hip": {"default_variant": -1, "rules": [
        {"variant": 2, "conditions": {"shape": [M, K, N]}}]}}}}}
    path = tmp_path / "tuning_data.json"
    path.write_text(json.dumps(rules))
    W = quantized_weights(fmt, N, K, seed=61)
    A = gauss_acts((M, K), seed=62, dtype=np.float16)
    explicit = gpu_matmul_ws(ops, fmt, W, A, N, K, out_dtype=torch.float32, variant=2)
    assert ops.enable_tuning(str(path))
    try:
        tuned = gpu_matmul_ws(ops, fmt, W, A, N, K, out_dtype=torch.float32, variant=-1)
    finally:
        ops.disable_tuning()
    assert np.array_equal(tuned, explicit)
    assert normwise_rel_err(tuned, oracle.matmul_gguf(fmt, W, A.astype(np.float32), N, f64=True)) < TOL_GEMM
    assert not ops.enable_tuning(str(tmp_path / "missing.json"))
    assert ops.enable_tuning()          # the committed file loads
    ops.disable_tuning()


# ---- prefill on resident dequantized weights (cuthip_matmul_dense_f16) ---------------------------------------------

@pytest.mark.parametrize("name", list(oracle.FORMATS))
@pytest.mark.parametrize("M,N,K", [(3, 136, 256), (300, 520, 1024), (1030, 264, 512)])
def test_dense_f16_resident_weights(ops, name, M, N, K):
    fmt = oracle.FORMATS[name]
    W = quantized_weights(fmt, N, K, seed=71)
    w16 = ops.dequantize(torch.from_numpy(W).cuda(), fmt, N, K, torch.float16)
    # the resident copy is the reference's fp16 weight tensor bit for bit
    assert np.array_equal(w16.cpu().numpy().reshape(-1).view(np.uint16), oracle.dequant_f16(fmt, W, N * K))
    A = gauss_acts((M, K), seed=72, dtype=np.float16)
    want = oracle.matmul_gguf(fmt, W, A.astype(np.float32), N, f64=True)
    got = ops.matmul_dense_f16(torch.from_numpy(A).cuda(), w16, out_dtype=torch.float32)
    torch.cuda.synchronize()
    got = got.cpu().numpy()
    assert normwise_rel_err(got, want) < (TOL_GEMM if M * N >= 1024 else TOL)
    # same weights and accumulation as the two-pass path of cuthip_matmul_gguf_ws
    two_pass = gpu_matmul_ws(ops, fmt, W, A, N, K, out_dtype=torch.float32, variant=4)
    assert normwise_rel_err(got, two_pass) < 1e-5
    # fp32 activations and a fused epilogue (the hand-written GEMM)
    A32 = gauss_acts((M, K), seed=73)
    D = gauss_acts((M, N), seed=74)
    add = ops.matmul_dense_f16(torch.from_numpy(A32).cuda(), w16, binary="add", d=torch.from_numpy(D).cuda())
    torch.cuda.synchronize()
    want32 = oracle.matmul_gguf(fmt, W, A32, N, f64=True)
    assert normwise_rel_err(add.cpu().numpy() - D, want32) < 1e-3


def test_dense_f16_argument_errors(ops):
    from cut_amd import lib
    w16 = torch.zeros((64, 200), dtype=torch.float16, device="cuda")
    a = torch.zeros((4, 200), dtype=torch.float16, device="cuda")
    with pytest.raises(lib.CutHipError, match="multiple of 128"):
        ops.matmul_dense_f16(a, w16)
    w16 = torch.zeros((64, 256), dtype=torch.float16, device="cuda")
    a = torch.zeros((4, 256), dtype=torch.float16, device="cuda")
    with pytest.raises(lib.CutHipError, match="workspace"):
        ops.matmul_dense_f16(a, w16, workspace=torch.empty(256, dtype=torch.uint8, device="cuda"))
