"""The attention in two halves: wide context splits (at most 8 records per head) and their merge inside the staging
of the matmul that consumes the attention output, against the oracle (Attention.cu:35-106 restated in
oracle.attention_decode) and against the merge launch."""
import math

import numpy as np
import pytest

import oracle
from helpers import gauss_acts, normwise_rel_err, quantized_weights

torch = pytest.importorskip("torch")
pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def ops():
    from cut_amd import lib, ops as _ops
    lib.check(lib.load().cuthip_init(0))
    return _ops


def dev(a):
    return torch.from_numpy(np.ascontiguousarray(a)).to("cuda")


def merge_records(rec: np.ndarray) -> np.ndarray:
    """[heads, splits, 2 + hd] -> [heads, hd] in float64: weights exp(max_s - max), divisor = the weighted sums."""
    m, l, o = rec[:, :, 0].astype(np.float64), rec[:, :, 1].astype(np.float64), rec[:, :, 2:].astype(np.float64)
    M = m.max(axis=1, keepdims=True)
    with np.errstate(invalid="ignore"):
        w = np.where(np.isneginf(m), 0.0, np.exp(m - np.where(np.isneginf(M), 0.0, M)))
    L = (l * w).sum(axis=1)
    num = (o * w[:, :, None]).sum(axis=1)
    return np.where(L[:, None] > 0, num / np.where(L[:, None] > 0, L[:, None], 1.0), 0.0)


@pytest.mark.parametrize("q_dtype", [np.float32, np.float16])
@pytest.mark.parametrize("n_heads,n_kv,seq,max_ctx", [
    (32, 8, 2048, 2048), (32, 8, 1, 2048), (32, 8, 5, 2048), (32, 8, 257, 2048), (32, 8, 1999, 2048),
    (16, 4, 4100, 8192),    # four passes per wave
    (6, 1, 130, 256),       # six query heads on one KV head, four splits
    (4, 4, 64, 64),         # one split, three waves without a chunk
    (8, 2, 100, 100),       # a capacity that is no multiple of the chunk
    (8, 2, 3000, 2500),     # a length beyond the capacity attends the capacity
    (8, 2, 513, 512 + 64)])
def test_wide_split_attention_against_oracle(ops, q_dtype, n_heads, n_kv, seq, max_ctx):
    hd = 128
    rng = np.random.default_rng(seq + max_ctx)
    q = rng.standard_normal(n_heads * hd).astype(q_dtype)
    K = (rng.standard_normal((max_ctx, n_kv * hd)) * 0.5).astype(np.float16)
    V = rng.standard_normal((max_ctx, n_kv * hd)).astype(np.float16)
    # rows past the sequence must not matter
    K[seq:] = np.float16(60000.0)
    V[seq:] = np.float16(np.nan)
    scale = 1 / math.sqrt(hd)
    want = oracle.attention_decode(q.astype(np.float32), K.view(np.uint16), V.view(np.uint16), min(seq, max_ctx), n_heads, n_kv,
                                   hd, scale)
    rec = ops.attn_partial_records(n_heads, hd, max_ctx, "cuda")
    assert rec.shape[1] == min(8, (max_ctx + 63) // 64)
    rec.fill_(float("nan"))   # every record is written
    params = dev(np.array([seq - 1, seq], np.int32))
    ops.attn_decode_partial(dev(q), dev(K), dev(V), params, n_heads, n_kv, hd, scale, rec)
    torch.cuda.synchronize()
    r = rec.cpu().numpy()
    assert not np.isnan(r).any()
    assert normwise_rel_err(merge_records(r), want) < 2e-6
    for out_dtype, tol in ((torch.float32, 2e-6), (torch.float16, 4e-4)):
        out = torch.empty(n_heads * hd, dtype=out_dtype, device="cuda")
        ops.attn_merge(rec, out)
        torch.cuda.synchronize()
        assert normwise_rel_err(out.float().cpu().numpy(), want) < tol
    # an empty sequence: every record is empty (max = -inf, sum = 0) and the merge gives zeros
    ops.attn_decode_partial(dev(q), dev(K), dev(V), dev(np.array([0, 0], np.int32)), n_heads, n_kv, hd, scale, rec)
    out = torch.full((n_heads * hd,), 7.0, dtype=torch.float32, device="cuda")
    ops.attn_merge(rec, out)
    torch.cuda.synchronize()
    r = rec.cpu().numpy()
    assert np.all(np.isneginf(r[:, :, 0])) and np.all(r[:, :, 1:] == 0)
    assert torch.all(out == 0)


def test_wide_split_attention_refusals(ops):
    from cut_amd.lib import CutHipError
    q = torch.zeros(8 * 64, dtype=torch.float32, device="cuda")
    kv = torch.zeros((64, 2 * 64), dtype=torch.float16, device="cuda")
    params = dev(np.array([0, 1], np.int32))
    rec = torch.empty((8, 1, 2 + 64), dtype=torch.float32, device="cuda")
    with pytest.raises(CutHipError, match="head_dim"):
        ops.attn_decode_partial(q, kv, kv, params, 8, 2, 64, 0.125, rec)
    q = torch.zeros(4 * 128, dtype=torch.float32, device="cuda")
    kv = torch.zeros((2048, 2 * 128), dtype=torch.float16, device="cuda")
    small = torch.empty((4, 7, 130), dtype=torch.float32, device="cuda")
    with pytest.raises(CutHipError, match="records"):
        ops.attn_decode_partial(q, kv, kv, params, 4, 2, 128, 0.1, small)
    W = dev(quantized_weights(oracle.Q4_K, 8, 9 * 128, seed=1))
    nine = torch.zeros((2, 9, 130), dtype=torch.float32, device="cuda")
    out = torch.empty(8, dtype=torch.float32, device="cuda")
    with pytest.raises(CutHipError, match="splits"):
        ops.matmul_gguf_attn_merge(nine, W, oracle.Q4_K, 8, out)
    ok = torch.zeros((2, 8, 130), dtype=torch.float32, device="cuda")
    with pytest.raises(CutHipError, match="sumsq_parts"):
        ops.matmul_gguf_attn_merge(ok, W, oracle.Q4_K, 8, out,
                                   carry=ops.norm_carry(sumsq_parts=torch.zeros(32, dtype=torch.float32, device="cuda"), eps=1e-5))


def synthetic_records(rng, n_heads, splits, hd, empty_heads=(), empty_splits=()):
    rec = np.zeros((n_heads, splits, 2 + hd), np.float32)
    rec[:, :, 0] = rng.uniform(-6.0, 6.0, (n_heads, splits))
    rec[:, :, 1] = rng.uniform(0.5, 60.0, (n_heads, splits))
    rec[:, :, 2:] = rng.standard_normal((n_heads, splits, hd)) * rec[:, :, 1:2]
    for h, s in empty_splits:
        rec[h, s, 0], rec[h, s, 1:] = -np.inf, 0.0
    for h in empty_heads:
        rec[h, :, 0], rec[h, :, 1:] = -np.inf, 0.0
    return rec


@pytest.mark.parametrize("name,n_heads,hd,splits,N", [
    ("Q4_K", 32, 128, 8, 4096),    # the output projection of the 8B shape
    ("Q4_K", 32, 128, 3, 4096),
    ("Q6_K", 4, 128, 1, 40),
    ("Q4_K", 64, 128, 8, 200),     # K = 8192: two passes of groups per thread
    ("Q8_0", 8, 64, 5, 72),        # another head dimension
    ("Q4_K", 16, 80, 8, 9),        # a head dimension that is no power of two
    ("Q4_0", 2, 16, 2, 24)])
def test_matmul_with_attention_merge_in_the_staging(ops, name, n_heads, hd, splits, N):
    fmt = oracle.FORMATS[name]
    K = n_heads * hd
    rng = np.random.default_rng(N + splits)
    rec = synthetic_records(rng, n_heads, splits, hd, empty_heads=(1,), empty_splits=((0, splits - 1),) if splits > 1 else ())
    Wq = quantized_weights(fmt, N, K, seed=90)
    W = dev(Wq)
    Wd = oracle.dequant(fmt, Wq, N * K).reshape(N, K).astype(np.float64)
    x = merge_records(rec).reshape(-1)
    assert np.all(x[hd:2 * hd] == 0)   # the empty head
    x16 = x.astype(np.float16).astype(np.float64)
    want = Wd @ x16
    recd = dev(rec)
    out = torch.empty(N, dtype=torch.float32, device="cuda")
    ops.matmul_gguf_attn_merge(recd, W, fmt, N, out)
    torch.cuda.synchronize()
    assert normwise_rel_err(out.cpu().numpy(), want) < 2e-4
    # against the unfused chain (merge launch to fp16, then the matmul): the two merges round differently in a few
    # elements (one fp16 ulp), nothing more
    a16 = torch.empty(K, dtype=torch.float16, device="cuda")
    ops.attn_merge(recd, a16)
    plain = ops.matmul_gguf(a16.view(1, -1), W, fmt, N, K, out_dtype=torch.float32)
    torch.cuda.synchronize()
    assert normwise_rel_err(out.cpu().numpy(), plain.cpu().numpy()[0]) < 1e-4
    # residual add in place + the producer side of a carried RMSNorm, fp16 and fp32 outputs
    res = gauss_acts((N,), seed=91)
    g = rng.uniform(0.5, 1.5, N).astype(np.float32)
    for c_dtype, tol in ((torch.float32, 2e-4), (torch.float16, 6e-4)):
        c = dev(res).to(c_dtype)
        nx = torch.zeros(N, dtype=torch.float16, device="cuda")
        parts = torch.full(((N + 7) // 8,), -1.0, dtype=torch.float32, device="cuda")
        ops.matmul_gguf_attn_merge(recd, W, fmt, N, c, binary="add", d=c,
                                   carry=ops.norm_carry(next_norm_weight=dev(g), next_x16=nx, next_sumsq_parts=parts))
        torch.cuda.synchronize()
        cn = c.float().cpu().numpy()
        ref = want + res.astype(c.cpu().numpy().dtype).astype(np.float64)
        assert normwise_rel_err(cn, ref) < tol
        if c_dtype == torch.float32:
            d16 = nx.cpu().numpy().view(np.uint16).astype(np.int32) - (cn * g).astype(np.float16).view(np.uint16).astype(np.int32)
            assert np.max(np.abs(d16)) <= 1
            sq = np.zeros(((N + 7) // 8) * 8, np.float64)
            sq[:N] = cn.astype(np.float64) ** 2
            np.testing.assert_allclose(parts.cpu().numpy(), sq.reshape(-1, 8).sum(1), rtol=2e-6, atol=1e-30)
    again = torch.empty(N, dtype=torch.float32, device="cuda")
    ops.matmul_gguf_attn_merge(recd, W, fmt, N, again)
    torch.cuda.synchronize()
    assert torch.equal(again, out)


@pytest.mark.parametrize("seq", [1, 300, 2048])
def test_attention_then_output_projection_full_size(ops, seq):
    """The 8B shape end to end: wide-split attention over a cache of 2048, then wo with the merge in its staging, against
    the oracle attention followed by the dequantized product."""
    n_heads, n_kv, hd, max_ctx, N = 32, 8, 128, 2048, 4096
    rng = np.random.default_rng(seq)
    q = rng.standard_normal(n_heads * hd).astype(np.float32)
    Kc = (rng.standard_normal((max_ctx, n_kv * hd)) * 0.5).astype(np.float16)
    Vc = rng.standard_normal((max_ctx, n_kv * hd)).astype(np.float16)
    scale = 1 / math.sqrt(hd)
    att = oracle.attention_decode(q, Kc.view(np.uint16), Vc.view(np.uint16), seq, n_heads, n_kv, hd, scale)
    fmt = oracle.Q4_K
    Wq = quantized_weights(fmt, N, n_heads * hd, seed=5)
    want = oracle.dequant(fmt, Wq, N * n_heads * hd).reshape(N, -1).astype(np.float64) @ att.astype(np.float16).astype(np.float64)
    rec = ops.attn_partial_records(n_heads, hd, max_ctx, "cuda")
    ops.attn_decode_partial(dev(q), dev(Kc), dev(Vc), dev(np.array([seq - 1, seq], np.int32)), n_heads, n_kv, hd, scale, rec)
    out = torch.empty(N, dtype=torch.float32, device="cuda")
    ops.matmul_gguf_attn_merge(rec, dev(Wq), fmt, N, out)
    torch.cuda.synchronize()
    assert normwise_rel_err(out.cpu().numpy(), want) < 3e-4
