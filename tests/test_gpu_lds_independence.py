"""LDS keeps what the last workgroup left in it.  An operator that reads a location of LDS it has not written returns
results that depend on what ran before it (a first run on a fresh GPU against a replay, one process against another):
correct to the tolerance of the parity tests most of the time, and not reproducible.  Every operator that stages
through LDS is therefore run behind three fills of the whole LDS of the chip (all ones = NaN in every float type,
zeros, fp16 ones) and must return the same bits each time."""
import numpy as np
import pytest

import oracle
from helpers import gauss_acts, quantized_weights

torch = pytest.importorskip("torch")
pytestmark = pytest.mark.gpu

PATTERNS = (0xFFFFFFFF, 0x00000000, 0x3C003C00)


@pytest.fixture(scope="module")
def ops():
    from cut_amd import lib, ops as _ops
    lib.check(lib.load().cuthip_init(0))
    return _ops


def fill_lds(pattern):
    from cut_amd import lib
    lib.check(lib.load().cuthip_debug_fill_lds(pattern, torch.cuda.current_stream().cuda_stream))


def same_bits_behind_every_fill(run):
    """run() -> tuple of tensors; called once per pattern, each time right behind a fill."""
    outs = []
    for p in PATTERNS:
        fill_lds(p)
        got = run()
        torch.cuda.synchronize()
        outs.append([t.detach().clone().view(torch.uint8).cpu().numpy() for t in got])
    for later in outs[1:]:
        for a, b in zip(outs[0], later):
            assert np.array_equal(a, b)


@pytest.mark.parametrize("name", list(oracle.FORMATS))
@pytest.mark.parametrize("M", [1, 2, 3, 4, 8])
@pytest.mark.parametrize("N,K", [(72, 512), (520, 2048), (4096, 4096), (1000, 14336)])
def test_gemv_does_not_read_lds_it_did_not_write(ops, name, M, N, K):
    fmt = oracle.FORMATS[name]
    w = torch.from_numpy(quantized_weights(fmt, N, K, seed=N + M)).cuda()
    a = torch.from_numpy(gauss_acts((M, K), seed=5, dtype=np.float16)).cuda()
    ws = ops.matmul_gguf_workspace(fmt, M, K, N, a.dtype, "cuda")
    out = torch.empty((M, N), dtype=torch.float32, device="cuda")
    same_bits_behind_every_fill(lambda: (ops.matmul_gguf(a, w, fmt, N, K, out=out, workspace=ws),))
    if M <= 2:   # fp32 activations take the general staging path
        a32 = a.float()
        same_bits_behind_every_fill(lambda: (ops.matmul_gguf(a32, w, fmt, N, K, out=out, workspace=ws),))


@pytest.mark.parametrize("name", list(oracle.FORMATS))
@pytest.mark.parametrize("M", [9, 16, 32, 64, 200])
def test_wider_matmuls_do_not_read_lds_they_did_not_write(ops, name, M):
    fmt = oracle.FORMATS[name]
    N, K = 520, 2048
    w = torch.from_numpy(quantized_weights(fmt, N, K, seed=M)).cuda()
    a = torch.from_numpy(gauss_acts((M, K), seed=6, dtype=np.float16)).cuda()
    ws = ops.matmul_gguf_workspace(fmt, M, K, N, a.dtype, "cuda")
    out = torch.empty((M, N), dtype=torch.float32, device="cuda")
    same_bits_behind_every_fill(lambda: (ops.matmul_gguf(a, w, fmt, N, K, out=out, workspace=ws),))
    same_bits_behind_every_fill(lambda: (ops.matmul_gguf(a, w, fmt, N, K, out=out),))


@pytest.mark.parametrize("hd,fuses", [(64, (4, 0)), (128, (5,))])
def test_decode_step_does_not_read_lds_it_did_not_write(ops, hd, fuses):
    """Every kernel of the fused decode step, one fill in front of each launch (the step's own kernels would otherwise
    leave each other the same LDS every time)."""
    from cut_amd.decode import DecodeConfig, DecodeStep
    from cut_amd import ops as O
    cfg = DecodeConfig(hidden=512, n_layers=2, n_heads=512 // hd, n_kv_heads=2, head_dim=hd, ffn=1024, vocab=2048, max_ctx=64)
    rng = np.random.default_rng(11)

    def qw(fmt, n, k):
        return torch.from_numpy(oracle.quantize(fmt, (rng.standard_normal(n * k) * 0.05).astype(np.float32))).cuda()

    def vec(n):
        return torch.from_numpy(rng.uniform(0.5, 1.5, n).astype(np.float32)).cuda()
    layers = [{"qk": qw(oracle.Q4_K, cfg.q_dim + cfg.kv_dim, cfg.hidden), "v": qw(oracle.Q6_K, cfg.kv_dim, cfg.hidden),
               "o": qw(oracle.Q4_K, cfg.hidden, cfg.q_dim), "gate_up": qw(oracle.Q4_K, 2 * cfg.ffn, cfg.hidden),
               "down": qw(oracle.Q4_K, cfg.hidden, cfg.ffn), "attn_norm": vec(cfg.hidden), "ffn_norm": vec(cfg.hidden)}
              for _ in range(cfg.n_layers)]
    x = torch.from_numpy(rng.standard_normal(cfg.hidden).astype(np.float32)).cuda()
    kc = torch.from_numpy((rng.standard_normal((9, cfg.kv_dim)) * 0.5).astype(np.float16)).cuda()
    vc = torch.from_numpy(rng.standard_normal((9, cfg.kv_dim)).astype(np.float16)).cuda()
    for fuse in fuses:
        step = DecodeStep(cfg, layers, vec(cfg.hidden), qw(oracle.Q6_K, cfg.vocab, cfg.hidden), fuse=fuse)
        for i in range(cfg.n_layers):
            step.k_cache[i][:9].copy_(kc)
            step.v_cache[i][:9].copy_(vc)
        step.set_position(9)
        # a fill in front of every launch of the step: wrap the entry points the step calls
        names = [n for n in ("rmsnorm", "matmul_gguf", "matmul_gguf_pair", "matmul_gguf_carry", "matmul_gguf_argmax", "attn_decode",
                             "attn_decode_partial", "matmul_gguf_attn_merge", "rope_kv_write", "silu_mul", "argmax",
                             "argmax_penalized")]
        saved = {n: getattr(O, n) for n in names}
        pattern = [0]

        def wrap(fn):
            def inner(*a, **k):
                fill_lds(pattern[0])
                return fn(*a, **k)
            return inner
        outs = []
        try:
            for n in names:
                setattr(O, n, wrap(saved[n]))
            for p in PATTERNS:
                pattern[0] = p
                step.x.copy_(x)
                step.step()
                torch.cuda.synchronize()
                outs.append((step.logits.cpu().numpy().copy(), int(step.token.item())))
        finally:
            for n in names:
                setattr(O, n, saved[n])
        for lg, tok in outs[1:]:
            assert np.array_equal(lg.view(np.uint32), outs[0][0].view(np.uint32)) and tok == outs[0][1]


@pytest.mark.parametrize("name", ["Q8_0", "Q4_0", "Q4_K"])
@pytest.mark.parametrize("M", [1, 4, 40])
def test_separated_layout_and_preparation_do_not_read_lds_they_did_not_write(ops, name, M):
    fmt = oracle.FORMATS[name]
    N, K = 264, 1024
    w = torch.from_numpy(quantized_weights(fmt, N, K, seed=M + 1)).cuda()
    a = torch.from_numpy(gauss_acts((M, K), seed=7)).cuda()
    q4, affine = name != "Q8_0", name == "Q4_K"
    same_bits_behind_every_fill(lambda: ops.prepare_sep(w, fmt, N, K))
    b, s = ops.prepare_sep(w, fmt, N, K)
    out = torch.empty((M, N), dtype=torch.float32, device="cuda")
    same_bits_behind_every_fill(lambda: (ops.matmul_sep(a, b, s, N, q4=q4, affine=affine, out=out),))


@pytest.mark.parametrize("name", list(oracle.FORMATS))
def test_fused_prologues_do_not_read_lds_they_did_not_write(ops, name):
    fmt = oracle.FORMATS[name]
    N, K = 200, 1024
    w = torch.from_numpy(quantized_weights(fmt, N, K, seed=3)).cuda()
    x = torch.from_numpy(gauss_acts((K,), seed=8)).cuda()
    gu = torch.from_numpy(gauss_acts((2 * K,), seed=9, dtype=np.float16)).cuda()
    nw = torch.from_numpy(np.random.default_rng(2).uniform(0.5, 1.5, K).astype(np.float32)).cuda()
    out = torch.empty(N, dtype=torch.float32, device="cuda")
    same_bits_behind_every_fill(lambda: (ops.matmul_gguf_pro(x, w, fmt, N, K, out, "rmsnorm", nw, 1e-5),))
    same_bits_behind_every_fill(lambda: (ops.matmul_gguf_pro(gu, w, fmt, N, K, out, "swiglu"),))


def test_prefill_paths_do_not_read_lds_they_did_not_write(ops):
    fmt = oracle.Q4_K
    M, N, K = 300, 520, 1024
    w = torch.from_numpy(quantized_weights(fmt, N, K, seed=4)).cuda()
    a = torch.from_numpy(gauss_acts((M, K), seed=10, dtype=np.float16)).cuda()
    ws = ops.matmul_gguf_workspace(fmt, M, K, N, a.dtype, "cuda")
    out = torch.empty((M, N), dtype=torch.float16, device="cuda")
    for variant in (2, 4):
        same_bits_behind_every_fill(lambda: (ops.matmul_gguf(a, w, fmt, N, K, out=out, workspace=ws, variant=variant),))
    w16 = ops.dequantize(w, fmt, N, K, torch.float16)
    same_bits_behind_every_fill(lambda: (ops.matmul_dense_f16(a, w16, out=out),))
    w8 = torch.from_numpy(quantized_weights(oracle.Q8_0, N, K, seed=5)).cuda()
    same_bits_behind_every_fill(lambda: (ops.matmul_q8_i8(a, w8, N, K, out=out),))
    x = torch.from_numpy(gauss_acts((64, K), seed=11)).cuda()
    same_bits_behind_every_fill(lambda: (ops.quantize_rows_q8_0(x),))
