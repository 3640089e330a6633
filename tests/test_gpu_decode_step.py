"""GPU parity of the operators between the matmuls of a decode step (RMSNorm,
RoPE + KV write, GQA decode attention, SiLU * up, arg-max) through the C ABI
against the CPU oracle, and of a whole small decode step (two layers + head)
against the same chain composed from oracle calls.  Floating point: each
assert states its tolerance; the KV cache write is bit-exact."""
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
    return torch.from_numpy(np.ascontiguousarray(a)).cuda()


@pytest.mark.parametrize("dtype", [np.float32, np.float16])
@pytest.mark.parametrize("rows,dim", [(1, 4096), (3, 1000), (2, 64)])
def test_rmsnorm(ops, dtype, rows, dim):
    rng = np.random.default_rng(rows * dim)
    x = rng.standard_normal((rows, dim)).astype(dtype)
    w = rng.uniform(0.5, 1.5, dim).astype(np.float32)
    got = ops.rmsnorm(dev(x), dev(w), 1e-5, out_dtype=torch.float32)
    torch.cuda.synchronize()
    want = oracle.rmsnorm(x.astype(np.float32), w, 1e-5)
    np.testing.assert_allclose(got.cpu().numpy(), want, rtol=2e-6, atol=1e-7)
    got16 = ops.rmsnorm(dev(x), dev(w), 1e-5, out_dtype=torch.float16)
    assert normwise_rel_err(got16.float().cpu().numpy(), want) < 4e-4   # one fp16 rounding of the output


def _tables(max_pos, head_dim, theta=500000.0):
    half = head_dim // 2
    inv = 1.0 / theta ** (np.arange(half, dtype=np.float64) * 2 / head_dim)
    ang = np.arange(max_pos, dtype=np.float64)[:, None] * inv[None]
    return np.cos(ang).astype(np.float32), np.sin(ang).astype(np.float32)


@pytest.mark.parametrize("n_heads,n_kv,hd,pos", [(32, 8, 128, 2047), (8, 2, 64, 3), (4, 4, 16, 0)])
def test_rope_kv_write(ops, n_heads, n_kv, hd, pos):
    max_ctx = pos + 2
    rng = np.random.default_rng(pos + hd)
    q = rng.standard_normal(n_heads * hd).astype(np.float32)
    k = rng.standard_normal(n_kv * hd).astype(np.float32)
    v = rng.standard_normal(n_kv * hd).astype(np.float32)
    cos_t, sin_t = _tables(max_ctx, hd)
    kc = np.zeros((max_ctx, n_kv * hd), np.uint16)
    vc = np.zeros((max_ctx, n_kv * hd), np.uint16)
    want_q = oracle.rope_kv_write(q, k, v, pos, cos_t, sin_t, hd, kc, vc)
    kcd = torch.zeros((max_ctx, n_kv * hd), dtype=torch.float16, device="cuda")
    vcd = torch.zeros_like(kcd)
    params = dev(np.array([pos, pos + 1], np.int32))
    q_out = torch.empty(n_heads * hd, dtype=torch.float32, device="cuda")
    ops.rope_kv_write(dev(q), dev(k), dev(v), params, dev(cos_t), dev(sin_t), kcd, vcd, hd, q_out)
    torch.cuda.synchronize()
    # same fp32 expression: the rotated q may differ by fma contraction only
    np.testing.assert_allclose(q_out.cpu().numpy(), want_q, rtol=1e-6, atol=1e-6)
    got_k = kcd.cpu().numpy().view(np.uint16)
    assert np.array_equal(vcd.cpu().numpy().view(np.uint16), vc)          # v: bit-exact fp16 store
    assert np.max(np.abs(got_k.astype(np.int32) - kc.astype(np.int32))) <= 1   # k: at most one fp16 ulp (fma contraction)
    assert not got_k[:pos].any() and not got_k[pos + 1:].any()


@pytest.mark.parametrize("dtype", [np.float32, np.float16])
@pytest.mark.parametrize("rows,dim,stride,offset", [(1, 1001, 1001, 0), (3, 1001, 1001, 0), (2, 1000, 1003, 0), (2, 4096, 4096, 1),
                                                    (3, 5, 5, 0), (2, 7, 9, 3), (1, 8, 8, 1), (2, 9000, 9001, 0)])
def test_rmsnorm_unaligned_rows(ops, dtype, rows, dim, stride, offset):
    """Rows that do not start on a 16-byte boundary (odd dim or stride, a view that starts one element in), rows
    shorter than one 8-element group and rows longer than the register window: every element must be read (the sum of
    squares and every output), checked against the oracle."""
    rng = np.random.default_rng(rows * dim + stride + offset)
    buf = rng.standard_normal(offset + rows * stride).astype(dtype)
    x = np.stack([buf[offset + r * stride: offset + r * stride + dim] for r in range(rows)])
    w = rng.uniform(0.5, 1.5, dim).astype(np.float32)
    want = oracle.rmsnorm(x.astype(np.float32), w, 1e-5)
    xd = dev(buf)[offset:].as_strided((rows, dim), (stride, 1))
    assert xd.data_ptr() % 16 != 0 or stride % 8 != 0 or dim < 8
    for out_dtype, tol in ((torch.float32, 2e-6), (torch.float16, 1e-3)):
        out = torch.full((rows, stride), -7.0, dtype=out_dtype, device="cuda")
        ops.rmsnorm(xd, dev(w), 1e-5, out=out[:, :dim] if stride != dim else out)
        torch.cuda.synchronize()
        got = out.float().cpu().numpy()
        np.testing.assert_allclose(got[:, :dim], want, rtol=tol, atol=tol * 1e-1)
        assert np.all(got[:, dim:] == -7.0)   # the padding between rows is not written


@pytest.mark.parametrize("n_heads,n_kv,hd,seq,max_ctx", [(32, 8, 128, 2048, 2048), (32, 8, 128, 1, 2048), (8, 2, 64, 77, 128),
                                                       (6, 1, 128, 130, 256), (4, 4, 16, 64, 64),
                                                       # most splits empty; 128 splits (beyond the merge's register window);
                                                       # 64 full splits; 8 query heads per KV head (two passes over the waves)
                                                       (32, 8, 128, 5, 2048), (16, 4, 128, 4100, 8192), (8, 2, 64, 4096, 4096),
                                                       (8, 1, 32, 200, 512)])
def test_attention_decode(ops, n_heads, n_kv, hd, seq, max_ctx):
    rng = np.random.default_rng(seq)
    q = rng.standard_normal(n_heads * hd).astype(np.float32)
    K = (rng.standard_normal((max_ctx, n_kv * hd)) * 0.5).astype(np.float16)
    V = rng.standard_normal((max_ctx, n_kv * hd)).astype(np.float16)
    scale = 1 / math.sqrt(hd)
    want = oracle.attention_decode(q, K.view(np.uint16), V.view(np.uint16), seq, n_heads, n_kv, hd, scale)
    ws = ops.attn_decode_workspace(n_heads, hd, max_ctx, "cuda")
    params = dev(np.array([seq - 1, seq], np.int32))
    for out_dtype, tol in ((torch.float32, 2e-6), (torch.float16, 4e-4)):
        out = torch.empty(n_heads * hd, dtype=out_dtype, device="cuda")
        ops.attn_decode(dev(q), dev(K), dev(V), params, n_heads, n_kv, hd, scale, ws, out)
        torch.cuda.synchronize()
        assert normwise_rel_err(out.float().cpu().numpy(), want) < tol
    # rows past seq_len must not matter: poison them
    K2, V2 = K.copy(), V.copy()
    K2[seq:] = np.float16(60000.0)
    V2[seq:] = np.float16(np.nan)
    out = torch.empty(n_heads * hd, dtype=torch.float32, device="cuda")
    ops.attn_decode(dev(q), dev(K2), dev(V2), params, n_heads, n_kv, hd, scale, ws, out)
    torch.cuda.synchronize()
    assert normwise_rel_err(out.cpu().numpy(), want) < 2e-6
    # an empty sequence: every split is empty and the output is zero, not NaN
    ops.attn_decode(dev(q), dev(K2), dev(V2), dev(np.array([0, 0], np.int32)), n_heads, n_kv, hd, scale, ws, out)
    torch.cuda.synchronize()
    assert torch.all(out == 0)
    ops.attn_decode(dev(q), dev(K), dev(V), params, n_heads, n_kv, hd, scale, ws, out)
    torch.cuda.synchronize()
    assert normwise_rel_err(out.cpu().numpy(), want) < 2e-6


def test_silu_mul_and_argmax(ops):
    rng = np.random.default_rng(5)
    gu = (rng.standard_normal(2 * 14336) * 3).astype(np.float16)
    out = torch.empty(14336, dtype=torch.float32, device="cuda")
    ops.silu_mul(dev(gu), out)
    torch.cuda.synchronize()
    np.testing.assert_allclose(out.cpu().numpy(), oracle.silu_mul(gu.astype(np.float32)), rtol=2e-6, atol=1e-7)
    logits = rng.standard_normal(128256).astype(np.float32)
    logits[[77, 90001]] = 9.5    # a tie: the first index wins
    idx = torch.zeros(1, dtype=torch.int32, device="cuda")
    ops.argmax(dev(logits), idx)
    torch.cuda.synchronize()
    assert int(idx.item()) == 77
    ops.argmax(dev(logits.astype(np.float16)[:1000]), idx)
    torch.cuda.synchronize()
    assert int(idx.item()) == int(np.argmax(logits.astype(np.float16)[:1000]))
    # vector body and scalar tail, unaligned base, maximum in the tail / at the ends, fewer elements than one vector
    big = dev(logits)
    for dt in (np.float32, np.float16):
        for n, off, hot in ((128256, 0, 128255), (4099, 1, 4098), (4099, 3, 0), (70001, 2, 69999), (3, 1, 2), (1, 0, 0),
                            (8191, 0, 4096)):
            h = rng.standard_normal(n + off).astype(dt)
            h[off + hot] = 40.0
            ops.argmax(dev(h)[off:], idx)
            torch.cuda.synchronize()
            assert int(idx.item()) == hot, (dt, n, off)
    del big


@pytest.mark.parametrize("name", list(oracle.FORMATS))
@pytest.mark.parametrize("out_dtype", [torch.float32, torch.float16])
def test_embedding_rows_from_gguf_blocks(ops, name, out_dtype):
    """Gathered rows are bit-identical to the dequantized rows of the table (fp32: the CPU dequant; fp16: followed by the
    reference's narrowing); ids on the device, repeated ids, an id past the table (zero row), a padded output stride."""
    fmt = oracle.FORMATS[name]
    vocab, dim = 300, 1024
    table = quantized_weights(fmt, vocab, dim, seed=40)
    ids = np.array([0, 299, 17, 17, 123, 300, 4000000000], np.uint32)
    out = torch.full((len(ids), dim + 8), -3.0, dtype=out_dtype, device="cuda")
    ops.embedding_rows(dev(table), fmt, dev(ids.view(np.int32)), vocab, dim, out[:, :dim])
    torch.cuda.synchronize()
    got = out.cpu().numpy()
    assert np.all(got[:, dim:] == -3.0)
    if out_dtype == torch.float32:
        full = oracle.dequant(fmt, table, vocab * dim).reshape(vocab, dim)
        want = np.stack([full[i] if i < vocab else np.zeros(dim, np.float32) for i in ids])
        assert np.array_equal(got[:, :dim].view(np.uint32), want.view(np.uint32))
    else:
        full = oracle.dequant_f16(fmt, table, vocab * dim).reshape(vocab, dim)
        want = np.stack([full[i] if i < vocab else np.zeros(dim, np.uint16) for i in ids])
        assert np.array_equal(got[:, :dim].view(np.uint16), want)


def test_embedding_col_against_oracle(ops):
    """EmbeddingColOpNode on the tensors cuthip_prepare_sep writes (int8 [K, N] + fp16 scales [K/32, N]) and on an fp16
    table, bit-exact against the oracle's restatement; the same rows as the GGUF gather."""
    vocab, dim = 200, 256
    table = quantized_weights(oracle.Q8_0, vocab, dim, seed=41)
    B, S = ops.prepare_sep(dev(table), "Q8_0", vocab, dim)       # the loader's separated tensors, produced on the GPU
    ids = np.array([5, 199, 0, 5], np.uint32)
    got = ops.embedding_col(dev(ids.view(np.int32)), B.view(torch.int8), S, dim, vocab)
    torch.cuda.synchronize()
    want = oracle.embedding_col(ids, B.cpu().numpy().view(np.int8), S.cpu().numpy().view(np.uint16), dim, 1)
    assert np.array_equal(got.cpu().numpy().view(np.uint32), want.view(np.uint32))
    rows = oracle.dequant(oracle.Q8_0, table, vocab * dim).reshape(vocab, dim)[ids]
    assert np.array_equal(want.view(np.uint32), rows.view(np.uint32))
    t16 = np.random.default_rng(42).standard_normal((dim, vocab + 4)).astype(np.float16)
    got16 = ops.embedding_col(dev(np.array([1, 198, 250], np.int32)), dev(t16), None, dim, vocab)
    torch.cuda.synchronize()
    w16 = oracle.embedding_col(np.array([1, 198], np.uint32), np.ascontiguousarray(t16).view(np.uint16), None, dim, 0)
    assert np.array_equal(got16.cpu().numpy()[:2], w16) and not got16.cpu().numpy()[2].any()   # index past the vocabulary: zeros


def test_repetition_penalty_and_penalized_argmax(ops):
    """The dense operator against the oracle; the sparse list + arg-max against `dense penalty, then arg-max` with the
    factor vector the runner would have built (repeated tokens penalised once, later entries override, ids out of
    range ignored), for fp32 and fp16 logits; the logits are rewritten in place."""
    rng = np.random.default_rng(50)
    n = 128256
    lg = (rng.standard_normal(n) * 3).astype(np.float32)
    hot = int(np.argmax(lg))
    second = int(np.argsort(lg)[-2])
    fac = oracle.penalty_factors([hot, 12, 12, n + 5, -7, 99], 1.3, n)
    out = ops.repetition_penalty(dev(lg), dev(fac))
    torch.cuda.synchronize()
    assert np.array_equal(out.cpu().numpy(), oracle.repetition_penalty(lg, fac))
    idx = torch.zeros(1, dtype=torch.int32, device="cuda")
    for dt in (np.float32, np.float16):
        l_h = lg.astype(dt)
        cases = [([], []), ([hot, 12, 12, n + 5, -7, 99], [100.0] * 6), ([hot, second, hot], [50.0, 60.0, 1.0]),
                 ([hot] + [-1] * 63, [1e9] + [1.0] * 63)]
        for toks, facs in cases:
            dense = np.ones(n, np.float32)
            for t, f in zip(toks, facs):
                if 0 <= t < n:
                    dense[t] = f                       # later entries override, as successive writes to factors[t] do
            want_l = oracle.repetition_penalty(l_h.astype(np.float32), dense).astype(dt)
            d = dev(l_h.copy())
            pt = dev(np.array(toks, np.int32)) if toks else None
            pf = dev(np.array(facs, np.float32)) if toks else None
            ops.argmax_penalized(d, idx, pt, pf)
            torch.cuda.synchronize()
            assert int(idx.item()) == int(np.argmax(want_l)), (dt, toks)
            assert np.array_equal(d.cpu().numpy(), want_l)


@pytest.mark.parametrize("n_pen", [66, 100, 1000])
def test_penalized_argmax_with_lists_longer_than_a_wave(ops, n_pen):
    """Penalty lists of more than 64 entries (the runner's default window is 64 tokens plus the suppressed ones,
    llama.cpp:2566-2592): entries handled by the second and later waves of the finishing workgroup, a list length that
    is not a multiple of 64, the unpenalised winner and the runners-up listed late in the list, padding entries of -1,
    and a winner after the penalty that sits in a row scanned by a thread of another wave.  Against the oracle's dense
    penalty followed by arg-max, on the logits directly and through the matmul's per-wave winners."""
    rng = np.random.default_rng(70 + n_pen)
    n = 40000
    lg = (rng.standard_normal(n) * 2).astype(np.float32)
    order = np.argsort(lg)
    top = [int(t) for t in order[-5:][::-1]]                  # the five largest logits, largest first
    toks = [int(t) for t in rng.choice(n, n_pen, replace=False)]
    # the winners sit at the end of the list; the largest is listed twice and its last entry (the last of the list,
    # handled by the last thread that has an entry) is the one that counts
    toks = [t for t in toks if t not in top][:n_pen - 9] + [-1] * 3 + top + [top[0]]
    assert len(toks) == n_pen
    facs = [float(f) for f in rng.uniform(1.1, 3.0, n_pen)]
    for i, t in enumerate(toks):
        if t in top:
            facs[i] = 1e6
    facs[n_pen - 6] = 1.0                                     # the first entry of the largest: overridden
    dense = np.ones(n, np.float32)
    for t, f in zip(toks, facs):
        if 0 <= t < n:
            dense[t] = f
    idx = torch.full((1,), -1, dtype=torch.int32, device="cuda")
    for dt in (np.float32, np.float16):
        l_h = lg.astype(dt)
        want_l = oracle.repetition_penalty(l_h.astype(np.float32), dense).astype(dt)
        want = int(np.argmax(want_l))
        assert want not in top
        if dt is np.float32:
            assert (want % 1024) >= 64                        # found by a thread outside the first wave
        d = dev(l_h.copy())
        ops.argmax_penalized(d, idx, dev(np.array(toks, np.int32)), dev(np.array(facs, np.float32)))
        torch.cuda.synchronize()
        assert int(idx.item()) == want, (dt, n_pen)
        assert np.array_equal(d.cpu().numpy(), want_l)
    # through the head matmul: per-wave winners in the workspace, the listed groups re-derived from the logits
    fmt, N, K = oracle.Q8_0, 12296, 512
    W = dev(quantized_weights(fmt, N, K, seed=71))
    a = dev(gauss_acts((1, K), seed=72, dtype=np.float16)).view(-1)
    ref = ops.matmul_gguf(a, W, fmt, N, K, out_dtype=torch.float32)
    torch.cuda.synchronize()
    ref = ref.cpu().numpy()[0]
    order = np.argsort(ref)
    top = [int(t) for t in order[-5:][::-1]]
    toks = [int(t) for t in rng.choice(N, n_pen, replace=False) if int(t) not in top][:n_pen - 6] + [-1] + top
    toks = (toks + [-1] * n_pen)[:n_pen]
    facs = [1e6 if t in top else 1.5 for t in toks]
    dense = np.ones(N, np.float32)
    for t, f in zip(toks, facs):
        if 0 <= t < N:
            dense[t] = f
    want_l = oracle.repetition_penalty(ref, dense)
    for ws in (ops.lm_head_workspace(N, "cuda"), None):
        logits = torch.empty(N, dtype=torch.float32, device="cuda")
        ops.matmul_gguf_argmax(a, W, fmt, N, K, logits, idx, pen_tokens=dev(np.array(toks, np.int32)),
                               pen_factors=dev(np.array(facs, np.float32)), workspace=ws)
        torch.cuda.synchronize()
        assert np.array_equal(logits.cpu().numpy(), want_l)
        assert int(idx.item()) == int(np.argmax(want_l)), (n_pen, ws is None)


@pytest.mark.parametrize("max_ctx,seq", [(100, 120), (100, 128), (64, 1000), (130, 131)])
def test_attention_decode_clamps_the_length_to_the_cache_capacity(ops, max_ctx, seq):
    """A device-side sequence length beyond max_seq_len attends the max_seq_len cached positions once each (capacities
    that are not a multiple of the 64-position chunk included), through the workspace entry point and the
    allocation-free one."""
    n_heads, n_kv, hd = 8, 2, 64
    rng = np.random.default_rng(max_ctx + seq)
    q = rng.standard_normal(n_heads * hd).astype(np.float32)
    K = (rng.standard_normal((max_ctx, n_kv * hd)) * 0.5).astype(np.float16)
    V = rng.standard_normal((max_ctx, n_kv * hd)).astype(np.float16)
    scale = 1 / math.sqrt(hd)
    want = oracle.attention_decode(q, K.view(np.uint16), V.view(np.uint16), max_ctx, n_heads, n_kv, hd, scale)
    ws = ops.attn_decode_workspace(n_heads, hd, max_ctx, "cuda")
    params = dev(np.array([seq - 1, seq], np.int32))
    out = torch.empty(n_heads * hd, dtype=torch.float32, device="cuda")
    ops.attn_decode(dev(q), dev(K), dev(V), params, n_heads, n_kv, hd, scale, ws, out)
    torch.cuda.synchronize()
    assert normwise_rel_err(out.cpu().numpy(), want) < 2e-6
    out2 = torch.empty_like(out)
    ops.attn_decode_static(dev(q), dev(K), dev(V), params, n_heads, n_kv, hd, scale, out2)
    torch.cuda.synchronize()
    assert torch.equal(out, out2)


def test_memset_is_refused_on_a_capturing_stream(ops):
    """cuthip_memset records nothing into a graph: on a capturing stream it returns an error and the capture goes on."""
    from cut_amd import lib
    import ctypes as C
    L = lib.load()
    buf = torch.full((256,), 7, dtype=torch.uint8, device="cuda")
    st = C.c_void_p()
    lib.check(L.cuthip_stream_create(C.byref(st)))
    try:
        lib.check(L.cuthip_memset(buf.data_ptr(), 1, 256, st))          # eager: allowed
        lib.check(L.cuthip_stream_sync(st))
        assert bool((buf == 1).all())
        lib.check(L.cuthip_graph_begin_capture(st))
        rc = L.cuthip_memset(buf.data_ptr(), 2, 256, st)
        msg = L.cuthip_last_error()
        g = C.c_void_p()
        lib.check(L.cuthip_graph_end_capture(st, C.byref(g)))
        assert rc != 0 and b"capturing" in msg
        lib.check(L.cuthip_graph_launch(g, st))
        lib.check(L.cuthip_stream_sync(st))
        assert bool((buf == 1).all())
        lib.check(L.cuthip_graph_destroy(g))
    finally:
        L.cuthip_stream_destroy(st)


@pytest.mark.parametrize("name,N,K", [("Q6_K", 128256, 4096), ("Q4_K", 14336, 4096), ("Q8_0", 12296, 512), ("Q6_K", 1000, 512)])
def test_head_matmul_with_argmax_in_the_epilogue(ops, name, N, K):
    """cuthip_matmul_gguf_argmax against the plain matmul followed by `penalty, then arg-max`: same logits bit for bit,
    same token, with and without a penalty list that hits the unpenalised winner; N = 1000 takes the path without the
    epilogue (K split inside the workgroup), the others the per-wave winners."""
    fmt = oracle.FORMATS[name]
    tile = quantized_weights(fmt, min(N, 1002), K, seed=60)
    rb = oracle.n_bytes(fmt, K)
    reps = -(-N // 1002)
    W = dev(np.concatenate([np.roll(tile.reshape(-1, rb), 13 * t, axis=0) for t in range(reps)])[:N].reshape(-1))
    a = dev(gauss_acts((1, K), seed=61, dtype=np.float16)).view(-1)
    plain = ops.matmul_gguf(a, W, fmt, N, K, out_dtype=torch.float32)
    torch.cuda.synchronize()
    ref = plain.cpu().numpy()[0]
    # the logits themselves against the float64 oracle, on a sample of vocabulary rows
    rows = np.unique(np.concatenate([[0, N - 1], np.random.default_rng(62).integers(0, N, 512)]))
    Wh = W.cpu().numpy().reshape(N, rb)[rows].reshape(-1)
    want_rows = oracle.matmul_gguf(fmt, Wh, a.cpu().numpy().astype(np.float32)[None], len(rows), f64=True)[0]
    assert normwise_rel_err(ref[rows], want_rows) < 2e-5
    order = np.argsort(ref)
    top, runner_up = int(order[-1]), int(order[-2])
    ws = ops.lm_head_workspace(N, "cuda")
    idx = torch.full((1,), -1, dtype=torch.int32, device="cuda")
    for toks, facs in (([], []), ([top, 3, top], [1000.0, 2.0, 1000.0]), ([top, runner_up, 7], [1e9, 1e9, 1.5])):
        logits = torch.empty(N, dtype=torch.float32, device="cuda")
        dense = np.ones(N, np.float32)
        for t, f in zip(toks, facs):
            dense[t] = f
        want_l = oracle.repetition_penalty(ref, dense)
        pt = dev(np.array(toks, np.int32)) if toks else None
        pf = dev(np.array(facs, np.float32)) if toks else None
        ops.matmul_gguf_argmax(a, W, fmt, N, K, logits, idx, pen_tokens=pt, pen_factors=pf, workspace=ws)
        torch.cuda.synchronize()
        assert np.array_equal(logits.cpu().numpy(), want_l)
        assert int(idx.item()) == int(np.argmax(want_l)), toks
    # without a workspace: the logits are scanned instead, same answer
    ops.matmul_gguf_argmax(a, W, fmt, N, K, logits, idx)
    torch.cuda.synchronize()
    assert int(idx.item()) == int(np.argmax(ref))   # the tile repeats, so the maximum does too: the first row wins


def _oracle_step(cfg, layers_h, out_norm, head, x, pos, kc, vc, cos_t, sin_t):
    """The same chain from oracle calls; activations rounded to fp16 where the GPU chain stores fp16."""
    f16 = lambda a: a.astype(np.float16).astype(np.float32)
    for i, L in enumerate(layers_h):
        xn = f16(oracle.rmsnorm(x, L["attn_norm"], cfg.eps))
        qk = oracle.matmul_gguf(oracle.Q4_K, L["qk"], xn[None], cfg.q_dim + cfg.kv_dim, f64=True)[0].astype(np.float32)
        v = oracle.matmul_gguf(oracle.Q6_K, L["v"], xn[None], cfg.kv_dim, f64=True)[0].astype(np.float32)
        q_rot = oracle.rope_kv_write(qk[:cfg.q_dim], qk[cfg.q_dim:], v, pos, cos_t, sin_t, cfg.head_dim, kc[i], vc[i])
        attn = f16(oracle.attention_decode(q_rot, kc[i], vc[i], pos + 1, cfg.n_heads, cfg.n_kv_heads, cfg.head_dim,
                                           1 / math.sqrt(cfg.head_dim)))
        x = x + oracle.matmul_gguf(oracle.Q4_K, L["o"], attn[None], cfg.hidden, f64=True)[0].astype(np.float32)
        hn = f16(oracle.rmsnorm(x, L["ffn_norm"], cfg.eps))
        gu = f16(oracle.matmul_gguf(oracle.Q4_K, L["gate_up"], hn[None], 2 * cfg.ffn, f64=True)[0].astype(np.float32))
        act = f16(oracle.silu_mul(gu))
        x = x + oracle.matmul_gguf(oracle.Q4_K, L["down"], act[None], cfg.hidden, f64=True)[0].astype(np.float32)
    xn = f16(oracle.rmsnorm(x, out_norm, cfg.eps))
    return oracle.matmul_gguf(oracle.Q6_K, head, xn[None], cfg.vocab, f64=True)[0].astype(np.float32)


@pytest.mark.parametrize("name", list(oracle.FORMATS))
@pytest.mark.parametrize("N,K", [(200, 512), (64, 4096), (1000, 14336)])
def test_matmul_with_fused_prologues(ops, name, N, K):
    """RMSNorm and SiLU(gate) * up fused into the activation staging of the batch-1 matmul against the oracle chain
    (norm -> fp16 -> matmul).  The fused kernel rounds x * w to fp16 and applies rsqrt(mean + eps) in fp32 to the
    result, the chain rounds x * scale * w: both one fp16 rounding per activation, hence the 4e-4 bound."""
    fmt = oracle.FORMATS[name]
    rng = np.random.default_rng(N + K)
    W = oracle.quantize(fmt, (rng.standard_normal(N * K) * 0.02).astype(np.float32))
    x = (rng.standard_normal(K) * 3).astype(np.float32)
    w = rng.uniform(0.5, 1.5, K).astype(np.float32)
    xn = oracle.rmsnorm(x, w, 1e-5)
    want = oracle.matmul_gguf(fmt, W, xn[None], N, f64=True)[0]
    for xin in (x, x.astype(np.float16)):
        if xin.dtype == np.float16:
            want = oracle.matmul_gguf(fmt, W, oracle.rmsnorm(xin.astype(np.float32), w, 1e-5)[None], N, f64=True)[0]
        out = torch.empty(N, dtype=torch.float32, device="cuda")
        ops.matmul_gguf_pro(dev(xin), dev(W), fmt, N, K, out, "rmsnorm", dev(w), 1e-5)
        torch.cuda.synchronize()
        assert normwise_rel_err(out.cpu().numpy(), want) < 4e-4
    gu = (rng.standard_normal(2 * K) * 2).astype(np.float16)
    act = oracle.silu_mul(gu.astype(np.float32)).astype(np.float16).astype(np.float32)
    want = oracle.matmul_gguf(fmt, W, act[None], N, f64=True)[0]
    res = rng.standard_normal(N).astype(np.float32)
    out = dev(res.copy())
    ops.matmul_gguf_pro(dev(gu), dev(W), fmt, N, K, out, "swiglu", binary="add", d=out)   # in-place residual add
    torch.cuda.synchronize()
    assert normwise_rel_err(out.cpu().numpy() - res, want) < 4e-4


@pytest.mark.parametrize("fuse,hd", [(0, 64), (1, 64), (2, 64), (3, 64), (4, 64), (4, 128), (5, 128)])
def test_small_decode_step_against_oracle_chain(ops, fuse, hd):
    from cut_amd.decode import DecodeConfig, DecodeStep
    cfg = DecodeConfig(hidden=512, n_layers=2, n_heads=512 // hd, n_kv_heads=2, head_dim=hd, ffn=1024, vocab=2048, max_ctx=64)
    rng = np.random.default_rng(11)

    def qw(fmt, n, k):
        return oracle.quantize(fmt, (rng.standard_normal(n * k) * 0.05).astype(np.float32))
    layers_h = [{"qk": qw(oracle.Q4_K, cfg.q_dim + cfg.kv_dim, cfg.hidden), "v": qw(oracle.Q6_K, cfg.kv_dim, cfg.hidden),
                 "o": qw(oracle.Q4_K, cfg.hidden, cfg.q_dim), "gate_up": qw(oracle.Q4_K, 2 * cfg.ffn, cfg.hidden),
                 "down": qw(oracle.Q4_K, cfg.hidden, cfg.ffn),
                 "attn_norm": rng.uniform(0.5, 1.5, cfg.hidden).astype(np.float32),
                 "ffn_norm": rng.uniform(0.5, 1.5, cfg.hidden).astype(np.float32)} for _ in range(cfg.n_layers)]
    out_norm = rng.uniform(0.5, 1.5, cfg.hidden).astype(np.float32)
    head = qw(oracle.Q6_K, cfg.vocab, cfg.hidden)
    step = DecodeStep(cfg, [{k: dev(v) for k, v in L.items()} for L in layers_h], dev(out_norm), dev(head), fuse=fuse)
    # a context of 9 earlier tokens already in the caches (same bits on both sides), then token 9
    pos = 9
    kc = [np.zeros((cfg.max_ctx, cfg.kv_dim), np.uint16) for _ in range(cfg.n_layers)]
    vc = [np.zeros((cfg.max_ctx, cfg.kv_dim), np.uint16) for _ in range(cfg.n_layers)]
    for i in range(cfg.n_layers):
        kc[i][:pos] = (rng.standard_normal((pos, cfg.kv_dim)) * 0.5).astype(np.float16).view(np.uint16)
        vc[i][:pos] = rng.standard_normal((pos, cfg.kv_dim)).astype(np.float16).view(np.uint16)
        step.k_cache[i].copy_(dev(kc[i].view(np.float16)))
        step.v_cache[i].copy_(dev(vc[i].view(np.float16)))
    x = rng.standard_normal(cfg.hidden).astype(np.float32)
    cos_t, sin_t = step.cos_t.cpu().numpy(), step.sin_t.cpu().numpy()
    want = _oracle_step(cfg, layers_h, out_norm, head, x.copy(), pos, kc, vc, cos_t, sin_t)

    step.x.copy_(dev(x))
    step.set_position(pos)
    step.step()
    torch.cuda.synchronize()
    got = step.logits.cpu().numpy()
    assert normwise_rel_err(got, want) < 1e-3
    assert int(step.token.item()) == int(np.argmax(got))
    # the step captured in a HIP graph and replayed twice (with eager work in between) gives the eager result
    step.x.copy_(dev(x))
    g = torch.cuda.CUDAGraph()
    with torch.cuda.graph(g):
        step.step()
    for _ in range(2):
        step.x.copy_(dev(x))
        torch.cuda.synchronize()
        g.replay()
        torch.cuda.synchronize()
        assert np.array_equal(step.logits.cpu().numpy(), got)


@pytest.mark.parametrize("fuse", [4, 0])
def test_decode_steps_feed_themselves_through_embedding_and_penalty(ops, fuse):
    """Three consecutive tokens of a small model: every step gathers the embedding of the token the previous step
    sampled (on the device), and samples with a repetition-penalty window; the logits of every step are checked
    against the oracle chain fed with the same token, the sampled token against `penalty, then arg-max` of the step's
    own logits (so a near-tie cannot make the two chains drift apart), eagerly and under replay of one captured graph."""
    from cut_amd.decode import DecodeConfig, DecodeStep
    cfg = DecodeConfig(hidden=512, n_layers=2, n_heads=8, n_kv_heads=2, head_dim=64, ffn=1024, vocab=2048, max_ctx=64)
    rng = np.random.default_rng(21)

    def qw(fmt, n, k):
        return oracle.quantize(fmt, (rng.standard_normal(n * k) * 0.05).astype(np.float32))
    layers_h = [{"qk": qw(oracle.Q4_K, cfg.q_dim + cfg.kv_dim, cfg.hidden), "v": qw(oracle.Q6_K, cfg.kv_dim, cfg.hidden),
                 "o": qw(oracle.Q4_K, cfg.hidden, cfg.q_dim), "gate_up": qw(oracle.Q4_K, 2 * cfg.ffn, cfg.hidden),
                 "down": qw(oracle.Q4_K, cfg.hidden, cfg.ffn),
                 "attn_norm": rng.uniform(0.5, 1.5, cfg.hidden).astype(np.float32),
                 "ffn_norm": rng.uniform(0.5, 1.5, cfg.hidden).astype(np.float32)} for _ in range(cfg.n_layers)]
    out_norm = rng.uniform(0.5, 1.5, cfg.hidden).astype(np.float32)
    head = qw(oracle.Q6_K, cfg.vocab, cfg.hidden)
    embd = oracle.quantize(oracle.Q4_K, rng.standard_normal(cfg.vocab * cfg.hidden).astype(np.float32))
    embd_f = oracle.dequant(oracle.Q4_K, embd, cfg.vocab * cfg.hidden).reshape(cfg.vocab, cfg.hidden)

    def run(replay):
        step = DecodeStep(cfg, [{k: dev(v) for k, v in L.items()} for L in layers_h], dev(out_norm), dev(head), fuse=fuse,
                          embedding=dev(embd), penalty_window=8)
        kc = [np.zeros((cfg.max_ctx, cfg.kv_dim), np.uint16) for _ in range(cfg.n_layers)]
        vc = [np.zeros((cfg.max_ctx, cfg.kv_dim), np.uint16) for _ in range(cfg.n_layers)]
        cos_t, sin_t = step.cos_t.cpu().numpy(), step.sin_t.cpu().numpy()
        token, history, graph = 77, [77], None
        step.token.fill_(token)
        for pos in range(3):
            step.set_position(pos)
            step.set_penalties(history, 1.5, suppressed=[5])
            torch.cuda.synchronize()
            if replay:
                if graph is None:
                    step.step()                      # warm-up outside the capture (same inputs: the caches are rewritten)
                    step.token.fill_(token)
                    torch.cuda.synchronize()
                    graph = torch.cuda.CUDAGraph()
                    with torch.cuda.graph(graph):
                        step.step()
                    step.token.fill_(token)
                graph.replay()
            else:
                step.step()
            torch.cuda.synchronize()
            got = step.logits.cpu().numpy()
            want = _oracle_step(cfg, layers_h, out_norm, head, embd_f[token].copy(), pos, kc, vc, cos_t, sin_t)
            fac = oracle.penalty_factors(history, 1.5, cfg.vocab)
            fac[5] = 1e9
            assert normwise_rel_err(got, oracle.repetition_penalty(want, fac)) < 1e-3, pos   # the step leaves the penalised logits
            new = int(step.token.item())
            assert new == int(np.argmax(got)), pos
            assert new != 5
            token = new
            history.append(token)
            # the next step of the oracle chain attends over the rows the GPU stored (its own differ from them by an
            # fp16 ulp here and there, which a two-position softmax would amplify beyond the per-step bound)
            for i in range(cfg.n_layers):
                gk = step.k_cache[i].cpu().numpy().view(np.uint16)
                gv = step.v_cache[i].cpu().numpy().view(np.uint16)
                assert normwise_rel_err(gk[pos].view(np.float16).astype(np.float32), kc[i][pos].view(np.float16).astype(np.float32)) < 5e-3
                kc[i][:pos + 1], vc[i][:pos + 1] = gk[:pos + 1], gv[:pos + 1]
        return history
    assert run(False) == run(True)


def test_full_size_layer_and_head_against_oracle_chain(ops):
    """BASELINE config 4 at its real geometry, one layer deep: hidden 4096, 32 query / 8 KV heads of 128, FFN 14336,
    KV context 2048 (2047 cached positions + the current token), Q4_K projections, Q6_K w_v and the Q6_K
    128256 x 4096 output head (16,032 row groups, the largest launch of the step).  The logits are compared with the
    same chain composed from oracle calls on 512 sampled vocabulary rows (the head is sliced for the oracle; the GPU
    runs it whole), normwise <= 1e-3.  The head's rows are a 2004-row quantized tile, rolled by a different amount
    in each of its 64 repeats, so that sampled rows differ while the host encoder stays within seconds."""
    from cut_amd.decode import DecodeConfig, DecodeStep
    cfg = DecodeConfig(n_layers=1)
    assert (cfg.hidden, cfg.n_heads, cfg.n_kv_heads, cfg.head_dim, cfg.ffn, cfg.vocab, cfg.max_ctx) == \
        (4096, 32, 8, 128, 14336, 128256, 2048)
    rng = np.random.default_rng(2048)
    L = {"qk": quantized_weights(oracle.Q4_K, cfg.q_dim + cfg.kv_dim, cfg.hidden, seed=1),
         "v": quantized_weights(oracle.Q6_K, cfg.kv_dim, cfg.hidden, seed=2),
         "o": quantized_weights(oracle.Q4_K, cfg.hidden, cfg.q_dim, seed=3),
         "gate_up": quantized_weights(oracle.Q4_K, 2 * cfg.ffn, cfg.hidden, seed=4),
         "down": quantized_weights(oracle.Q4_K, cfg.hidden, cfg.ffn, seed=5),
         "attn_norm": rng.uniform(0.5, 1.5, cfg.hidden).astype(np.float32),
         "ffn_norm": rng.uniform(0.5, 1.5, cfg.hidden).astype(np.float32)}
    out_norm = rng.uniform(0.5, 1.5, cfg.hidden).astype(np.float32)
    tile_rows, reps = 2004, 64
    rb = oracle.n_bytes(oracle.Q6_K, cfg.hidden)
    tile = quantized_weights(oracle.Q6_K, tile_rows, cfg.hidden, seed=6).reshape(tile_rows, rb)
    head = np.concatenate([np.roll(tile, 37 * t, axis=0) for t in range(reps)]).reshape(-1)
    assert head.size == cfg.vocab * rb
    pos = cfg.max_ctx - 1
    kc = np.zeros((cfg.max_ctx, cfg.kv_dim), np.uint16)
    vc = np.zeros((cfg.max_ctx, cfg.kv_dim), np.uint16)
    kc[:pos] = (rng.standard_normal((pos, cfg.kv_dim)) * 0.5).astype(np.float16).view(np.uint16)
    vc[:pos] = rng.standard_normal((pos, cfg.kv_dim)).astype(np.float16).view(np.uint16)
    x = rng.standard_normal(cfg.hidden).astype(np.float32)
    sample = np.unique(np.concatenate([np.arange(0, 16), np.arange(cfg.vocab - 16, cfg.vocab),
                                       rng.choice(cfg.vocab, 480, replace=False)]))
    head_rows = head.reshape(cfg.vocab, rb)[sample].reshape(-1)

    for fuse in (4, 5, 0):
        step = DecodeStep(cfg, [{k: dev(v) for k, v in L.items()}], dev(out_norm), dev(head), fuse=fuse)
        step.k_cache[0].copy_(dev(kc.view(np.float16)))
        step.v_cache[0].copy_(dev(vc.view(np.float16)))
        step.x.copy_(dev(x))
        step.set_position(pos)
        step.step()
        torch.cuda.synchronize()
        got = step.logits.cpu().numpy()
        if fuse == 4:
            cos_t, sin_t = step.cos_t.cpu().numpy(), step.sin_t.cpu().numpy()
            sub = dataclasses_replace_vocab(cfg, len(sample))
            want = _oracle_step(sub, [L], out_norm, head_rows, x.copy(), pos, [kc.copy()], [vc.copy()], cos_t, sin_t)
        assert np.all(np.isfinite(got))
        assert normwise_rel_err(got[sample], want) < 1e-3, fuse
        assert int(step.token.item()) == int(np.argmax(got))
        # the cache row of the current token was appended, the cached context left as it was
        v_new = step.v_cache[0][pos].float().cpu().numpy()
        assert normwise_rel_err(v_new, _v_row(L, cfg, x)) < 1e-3
        assert np.array_equal(step.v_cache[0][:pos].cpu().numpy().view(np.uint16), vc[:pos])
        assert np.array_equal(step.k_cache[0][:pos].cpu().numpy().view(np.uint16), kc[:pos])
        del step
        torch.cuda.empty_cache()


def dataclasses_replace_vocab(cfg, vocab):
    import dataclasses
    return dataclasses.replace(cfg, vocab=vocab)


def _v_row(L, cfg, x):
    """The v projection of the current token by the oracle chain."""
    xn = oracle.rmsnorm(x, L["attn_norm"], cfg.eps).astype(np.float16).astype(np.float32)
    return oracle.matmul_gguf(oracle.Q6_K, L["v"], xn[None], cfg.kv_dim, f64=True)[0].astype(np.float32)


@pytest.mark.parametrize("name", ["Q4_K", "Q6_K", "Q8_0", "Q4_0"])
@pytest.mark.parametrize("M,ffn,K", [(1, 14336, 4096), (1, 44, 512), (2, 300, 1024), (8, 64, 2048), (1, 4, 256), (1, 1024, 256)])
def test_swiglu_row_pair_epilogue(ops, name, M, ffn, K):
    """Interleaved gate / up rows, SiLU(gate) * up in the matmul's epilogue, against the oracle's two matmuls and
    silu_mul; covers the direct (one K range) and folded (split K) epilogues and every batch size class."""
    from cut_amd.decode import interleave_gate_up
    fmt = oracle.FORMATS[name]
    W = quantized_weights(fmt, 2 * ffn, K, seed=70)           # [gate rows | up rows]
    A = gauss_acts((M, K), seed=71, dtype=np.float16)
    w_il = interleave_gate_up(dev(W), ffn)
    got = ops.matmul_gguf(dev(A), w_il, fmt, 2 * ffn, K, out_dtype=torch.float32, swiglu_pairs=True)
    torch.cuda.synchronize()
    assert tuple(got.shape) == (M, ffn)
    gu = oracle.matmul_gguf(fmt, W, A.astype(np.float32), 2 * ffn, f64=True).astype(np.float32)
    want = np.stack([oracle.silu_mul(gu[m]) for m in range(M)])
    assert normwise_rel_err(got.cpu().numpy(), want) < 5e-5
    # and the permutation itself: row 2i of the interleaved tensor is gate row i, row 2i+1 is up row i
    rb = oracle.n_bytes(fmt, K)
    il = w_il.cpu().numpy().reshape(2 * ffn, rb)
    Wr = W.reshape(2, ffn, rb)
    assert np.array_equal(il[0::2], Wr[0]) and np.array_equal(il[1::2], Wr[1])


def test_swiglu_row_pair_epilogue_refusals(ops):
    from cut_amd import lib
    fmt = oracle.Q4_K
    W = dev(quantized_weights(fmt, 64, 256, seed=72))
    with pytest.raises(lib.CutHipError, match="M <= 8"):
        ops.matmul_gguf(dev(gauss_acts((9, 256), seed=1, dtype=np.float16)), W, fmt, 64, 256, swiglu_pairs=True)
    with pytest.raises(lib.CutHipError, match="variant 3 only"):
        ops.matmul_gguf(dev(gauss_acts((2, 256), seed=1, dtype=np.float16)), W, fmt, 64, 256, swiglu_pairs=True, variant=2)
    with pytest.raises(lib.CutHipError, match="even N"):
        ops.matmul_gguf(dev(gauss_acts((1, 256), seed=1, dtype=np.float16)), W, fmt, 63, 256, swiglu_pairs=True)


@pytest.mark.parametrize("name", ["Q4_K", "Q6_K", "Q8_0"])
@pytest.mark.parametrize("N,K", [(4096, 14336), (4096, 4096), (14336, 4096), (40, 512), (9, 256)])
def test_carried_rmsnorm_producer_and_consumer(ops, name, N, K):
    """Producer: C = A . W^T + D as the plain matmul gives it, next_x16 = fp16(C * g), sum(C^2) of every group of 8
    outputs in its slot.  Consumer: the plain matmul times 1 / sqrt(sum(parts) / K + eps).  Shapes cover the direct and
    the folded (split K) epilogues and a ragged last group."""
    fmt = oracle.FORMATS[name]
    W = dev(quantized_weights(fmt, N, K, seed=80))
    A = gauss_acts((1, K), seed=81, dtype=np.float16)
    D = gauss_acts((1, N), seed=82)
    g = np.random.default_rng(83).uniform(0.5, 1.5, N).astype(np.float32)
    plain = ops.matmul_gguf(dev(A), W, fmt, N, K, out_dtype=torch.float32, binary="add", d=dev(D))
    c = torch.empty(N, dtype=torch.float32, device="cuda")
    x16 = torch.zeros(N, dtype=torch.float16, device="cuda")
    ng = (N + 7) // 8
    parts = torch.full((ng + 3,), -1.0, dtype=torch.float32, device="cuda")   # stale contents are overwritten, the tail is not touched
    ops.matmul_gguf_carry(dev(A).view(-1), W, fmt, N, K, c, binary="add", d=dev(D).view(-1),
                          carry=ops.norm_carry(next_norm_weight=dev(g), next_x16=x16, next_sumsq_parts=parts))
    torch.cuda.synchronize()
    cn = c.cpu().numpy()
    assert np.array_equal(cn, plain.cpu().numpy()[0])
    # the device rounds the exact product once (mixed-precision multiply), numpy rounds to fp32 first: at most one ulp apart
    d16 = x16.cpu().numpy().view(np.uint16).astype(np.int32) - (cn * g).astype(np.float16).view(np.uint16).astype(np.int32)
    assert np.max(np.abs(d16)) <= 1 and np.mean(d16 != 0) < 0.01
    sq = np.zeros(ng * 8, np.float64)
    sq[:N] = cn.astype(np.float64) ** 2
    pn = parts.cpu().numpy()
    np.testing.assert_allclose(pn[:ng], sq.reshape(ng, 8).sum(1), rtol=2e-6, atol=1e-30)
    assert np.all(pn[ng:] == -1.0)
    # consumer: K / 8 partial sums of some earlier producer
    A2 = gauss_acts((1, K), seed=84, dtype=np.float16)
    pk = np.random.default_rng(85).uniform(0.0, 2.0, (K + 7) // 8).astype(np.float32)
    base = ops.matmul_gguf(dev(A2), W, fmt, N, K, out_dtype=torch.float32).cpu().numpy()[0]
    out = torch.empty(N, dtype=torch.float32, device="cuda")
    ops.matmul_gguf_carry(dev(A2).view(-1), W, fmt, N, K, out, carry=ops.norm_carry(sumsq_parts=dev(pk), eps=1e-5))
    torch.cuda.synchronize()
    scale = 1.0 / np.sqrt(pk.astype(np.float64).sum() / K + 1e-5)
    # the scale multiplies the partial sums of the K ranges before they are folded: errors relative to those, not to the result
    np.testing.assert_allclose(out.cpu().numpy(), base * np.float32(scale), rtol=3e-6, atol=3e-6 * float(np.abs(base).max() * scale))
    again = torch.empty(N, dtype=torch.float32, device="cuda")
    ops.matmul_gguf_carry(dev(A2).view(-1), W, fmt, N, K, again, carry=ops.norm_carry(sumsq_parts=dev(pk), eps=1e-5))
    torch.cuda.synchronize()
    assert np.array_equal(again.cpu().numpy(), out.cpu().numpy())   # fixed summation order: reproducible


def test_carried_rmsnorm_equals_rmsnorm_then_matmul(ops):
    """producer -> consumer against RMSNorm kernel -> matmul on the same data (the fp16 rounding of the activations is
    taken before the scaling instead of after it: 2^-11 relative per element, well inside 1e-3 normwise)."""
    fmt = oracle.Q4_K
    hidden, N = 4096, 512
    rng = np.random.default_rng(90)
    x = rng.standard_normal(hidden).astype(np.float32)
    g = rng.uniform(0.5, 1.5, hidden).astype(np.float32)
    Wp = dev(quantized_weights(fmt, hidden, hidden, seed=91))   # producer weights (square)
    Wc = dev(quantized_weights(fmt, N, hidden, seed=92))
    a = gauss_acts((1, hidden), seed=93, dtype=np.float16)
    xs = torch.from_numpy(x).cuda()
    x16 = torch.empty(hidden, dtype=torch.float16, device="cuda")
    parts = torch.zeros(hidden // 8, dtype=torch.float32, device="cuda")
    ops.matmul_gguf_carry(dev(a).view(-1), Wp, fmt, hidden, hidden, xs, binary="add", d=xs,
                          carry=ops.norm_carry(next_norm_weight=dev(g), next_x16=x16, next_sumsq_parts=parts))
    got = torch.empty(N, dtype=torch.float32, device="cuda")
    ops.matmul_gguf_carry(x16, Wc, fmt, N, hidden, got, carry=ops.norm_carry(sumsq_parts=parts, eps=1e-5))
    xn = ops.rmsnorm(xs.view(1, -1), dev(g), 1e-5, out_dtype=torch.float16)
    want = ops.matmul_gguf(xn, Wc, fmt, N, hidden, out_dtype=torch.float32)
    torch.cuda.synchronize()
    assert normwise_rel_err(got.cpu().numpy()[None, :], want.cpu().numpy()) < 5e-4


@pytest.mark.parametrize("outlier", [1.0e3, 3.0e4])
def test_carried_rmsnorm_with_residual_outliers(ops, outlier):
    """The carried norm keeps x * norm_weight in fp16 between the producer and the consumer: a residual stream with a
    few very large entries (as real models have) must still give RMSNorm -> matmul of the float64 oracle, as long as
    |x * w| stays below the fp16 maximum (65504; the documented limit of the carry)."""
    fmt = oracle.Q4_K
    hidden, N = 4096, 256
    rng = np.random.default_rng(190)
    x = rng.standard_normal(hidden).astype(np.float32)
    x[[5, 1234, 4000]] = [outlier, -outlier, 0.7 * outlier]
    g = rng.uniform(0.5, 1.5, hidden).astype(np.float32)
    Wp = dev(quantized_weights(fmt, hidden, hidden, seed=191))
    Wc_h = quantized_weights(fmt, N, hidden, seed=192)
    a = np.zeros((1, hidden), dtype=np.float16)                 # the producer adds nothing: its output is the residual x
    xs = torch.from_numpy(x).cuda()
    x16 = torch.empty(hidden, dtype=torch.float16, device="cuda")
    parts = torch.zeros(hidden // 8, dtype=torch.float32, device="cuda")
    ops.matmul_gguf_carry(dev(a).view(-1), Wp, fmt, hidden, hidden, xs, binary="add", d=xs,
                          carry=ops.norm_carry(next_norm_weight=dev(g), next_x16=x16, next_sumsq_parts=parts))
    got = torch.empty(N, dtype=torch.float32, device="cuda")
    ops.matmul_gguf_carry(x16, dev(Wc_h), fmt, N, hidden, got, carry=ops.norm_carry(sumsq_parts=parts, eps=1e-5))
    torch.cuda.synchronize()
    assert np.array_equal(xs.cpu().numpy(), x)
    assert np.isfinite(x16.cpu().numpy().astype(np.float32)).all()
    x64 = x.astype(np.float64)
    xn = x64 / np.sqrt(np.mean(x64 * x64) + 1e-5) * g.astype(np.float64)
    want = oracle.dequant(fmt, Wc_h, N * hidden).astype(np.float64).reshape(N, hidden) @ xn
    assert normwise_rel_err(got.cpu().numpy()[None, :].astype(np.float64), want[None, :]) < 1e-3


@pytest.mark.parametrize("fa,fb", [("Q4_K", "Q6_K"), ("Q4_K", "Q4_K"), ("Q8_0", "Q8_0")])
@pytest.mark.parametrize("n_heads,n_kv,hd,K,pos", [(32, 8, 128, 4096, 2047), (4, 2, 64, 256, 0), (8, 2, 64, 1024, 17),
                                                   (2, 1, 16, 512, 3)])
def test_pair_launch_with_rope_and_cache_append(ops, fa, fb, n_heads, n_kv, hd, K, pos):
    """q | k | v projections with RoPE and the cache append in the epilogue (rows of q | k interleaved inside every
    head) against the plain pair launch followed by the RoPE kernel: rotated q, the new cache rows, and nothing else
    touched.  Shapes cover the direct and the folded epilogue and the two-launch fallback (Q8_0)."""
    q_dim, kv_dim, max_ctx = n_heads * hd, n_kv * hd, pos + 2
    fqa, fqb = oracle.FORMATS[fa], oracle.FORMATS[fb]
    Wqk = dev(quantized_weights(fqa, q_dim + kv_dim, K, seed=100))
    Wv = dev(quantized_weights(fqb, kv_dim, K, seed=101))
    x = dev(gauss_acts((1, K), seed=102, dtype=np.float16)).view(-1)
    cos_t, sin_t = _tables(max_ctx, hd)
    params = dev(np.array([pos, pos + 1], np.int32))
    # reference: plain pair launch, then the RoPE kernel
    qk = torch.empty(q_dim + kv_dim, dtype=torch.float32, device="cuda")
    v = torch.empty(kv_dim, dtype=torch.float32, device="cuda")
    ops.matmul_gguf_pair(x, Wqk, fqa, q_dim + kv_dim, qk, Wv, fqb, kv_dim, v, K)
    k1 = torch.full((max_ctx, kv_dim + 8), 3.0, dtype=torch.float16, device="cuda")
    v1 = torch.full_like(k1, 5.0)
    q1 = torch.empty(q_dim, dtype=torch.float32, device="cuda")
    ops.rope_kv_write(qk[:q_dim], qk[q_dim:], v, params, dev(cos_t), dev(sin_t), k1[:, :kv_dim], v1[:, :kv_dim], hd, q1)
    # fused
    Wqk_il = ops.interleave_rope_rows(Wqk, q_dim + kv_dim, hd)
    k2 = torch.full((max_ctx, kv_dim + 8), 3.0, dtype=torch.float16, device="cuda")
    v2 = torch.full_like(k2, 5.0)
    q2 = torch.empty(q_dim, dtype=torch.float32, device="cuda")
    ops.matmul_gguf_pair(x, Wqk_il, fqa, q_dim + kv_dim, None, Wv, fqb, kv_dim, None, K,
                         rope=ops.rope_append(params, dev(cos_t), dev(sin_t), q2, k2[:, :kv_dim], v2[:, :kv_dim], q_dim, hd))
    torch.cuda.synchronize()
    np.testing.assert_allclose(q2.cpu().numpy(), q1.cpu().numpy(), rtol=2e-6, atol=2e-6)
    kd = k2.cpu().numpy().view(np.uint16).astype(np.int32) - k1.cpu().numpy().view(np.uint16).astype(np.int32)
    assert np.max(np.abs(kd)) <= 1   # fma contraction may differ between the two code sites: at most one fp16 ulp
    assert np.array_equal(v2.cpu().numpy().view(np.uint16), v1.cpu().numpy().view(np.uint16))
    assert torch.all(k2[:, kv_dim:] == 3.0) and torch.all(v2[:, kv_dim:] == 5.0)
    assert torch.all(k2[:pos] == 3.0) and torch.all(k2[pos + 1:] == 3.0)
    # the row permutation itself
    rb = oracle.n_bytes(fqa, K)
    il = Wqk_il.cpu().numpy().reshape(-1, hd, rb)
    w = Wqk.cpu().numpy().reshape(-1, hd, rb)
    assert np.array_equal(il[:, 0::2], w[:, :hd // 2]) and np.array_equal(il[:, 1::2], w[:, hd // 2:])
