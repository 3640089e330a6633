#!/usr/bin/env python3
"""Benchmark of the GGUF quantized-matmul hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--no-extras] [--no-cpu]

Workload (BASELINE.json configs[2], the configuration the metric is quoted on):
Q4_K GEMV at the FFN shapes of an 8B dense transformer, batch 1, fp16
activations in and out, fp32 accumulation.  One step = the three GEMVs of one
FFN block (gate and up 14336 x 4096, down 4096 x 14336).  Weights are resident
in HBM before the timed region and every step reads a different copy of them
(COPIES sets, 595 MB in total), so they stream from HBM and not from the
256 MB Infinity Cache.  The K timed steps are one HIP graph, replayed once untimed
(the first replay also uploads the graph: 0.5-1 us per kernel node) and once timed.

Prints one JSON line: metric/value = algorithmic bytes per second over the
whole timed region, plus "roofline" (the GEMV kernel against the 8 TB/s HBM
peak) and "cpu_baseline" (the CPU restatement of the reference's path on the
same workload, single thread).  "extras" carries the other configurations.
"""
import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0
N_FF, N_EMBD = 14336, 4096
COPIES = 6


def log(*a):
    print(*a, file=sys.stderr, flush=True)


def make_q_weights(fmt_name, n, k, seed):
    import numpy as np
    from cut_amd import quantize as Q
    w = np.random.default_rng(seed).standard_normal(n * k, dtype=np.float32) * np.float32(0.02)
    return Q.quantize(fmt_name, w)


# untimed graph replays in front of a timed one (timed_graph, prime=True) last at least this long; 0 = one replay.
# (--prime-seconds: 50 ms of them bring the clocks of an idle GPU up and shorten the launches of a 20-step graph by 2 %
# by events, but the host thread that slept through them then takes 50 us longer over the timed launch, which costs the
# wall-clock figure of such a run 6 %; one replay, the default, only takes the upload of the graph out of the timing)
PRIME_SECONDS = 0.0


def timed_graph(torch, fn_step, steps, warmup, prime=False):
    """Runs `warmup` eager steps, captures `steps` steps into one HIP graph and times one replay of it.  prime: replay
    it once untimed before (part of the warm-up; longer with --prime-seconds).  The first replay of a graph also uploads it, 0.5-1 us per kernel
    node: 3-10 % of a graph of 9-15 us launches (the headline at 20 steps: 9.1 us per launch unprimed, 8.8 primed) and
    nothing of a graph of a few long ones.  The callers made of short launches (the FFN steps at every batch size, the
    decode step) prime; the others do not and stay comparable with their earlier figures: a second back-to-back replay
    of long bandwidth-bound launches runs 3-10 % slower than the first on this part (it recovers after a 50 ms pause,
    which in turn costs short launches 2-4 %: power management in both directions), so those are burst figures, and a
    primed run of thousands of short launches is a sustained one.  Returns (wall_seconds, event_ms, used_graph)."""
    for s in range(warmup):
        fn_step(s)
    torch.cuda.synchronize()
    used_graph = True
    try:
        g = torch.cuda.CUDAGraph()
        with torch.cuda.graph(g):
            for s in range(steps):
                fn_step(s)
        torch.cuda.synchronize()
        run = g.replay
        if prime:
            # the first untimed replay uploads the graph; further ones until PRIME_SECONDS of work have passed
            t_p = time.perf_counter()
            g.replay()
            torch.cuda.synchronize()
            one = max(time.perf_counter() - t_p, 1e-5)
            for _ in range(min(int(PRIME_SECONDS / one), 400)):
                g.replay()
    except Exception as e:  # noqa: BLE001
        log(f"[bench] graph capture failed ({e}); timing eager launches")
        used_graph = False

        def run():
            for s in range(steps):
                fn_step(s)
    ev0, ev1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    ev0.record()
    run()
    ev1.record()
    torch.cuda.synchronize()
    t1 = time.perf_counter()
    return t1 - t0, ev0.elapsed_time(ev1), used_graph


# HBM bytes per launch of the headline kernel from rocprofv3 --pmc FETCH_SIZE (x 2.000, the factor a plain
# 1 GiB copy gives on this part) + WRITE_SIZE (x 1.000), launch-weighted over gate, up, down
# (profiles/gemv_q4k_ffn_batch1.md holds the counters and the commands)
TRAFFIC_BYTES_PER_LAUNCH = 33689600


def bench_decode_step(torch, np, ops, dev, x_h, steps=5):
    """config 4: one full decode step of the 8B shape at KV context 2048 (embedding row of the previous step's token;
    32 layers: RMSNorm, fused q+k and v matmuls, RoPE + KV write, GQA attention over the fp16 cache, wo + residual,
    RMSNorm, fused gate+up, SiLU * up, w_down + residual; output norm, Q6_K head, arg-max), distinct weight memory
    per layer, random init, captured once into a HIP graph.  Bytes per token: weights + KV cache read."""
    from cut_amd.decode import DecodeConfig, DecodeStep
    cfg = DecodeConfig()
    lw = {"qk": (cfg.fmt_attn, cfg.q_dim + cfg.kv_dim, cfg.hidden), "v": (cfg.fmt_v, cfg.kv_dim, cfg.hidden),
          "o": (cfg.fmt_attn, cfg.hidden, cfg.q_dim), "gate_up": (cfg.fmt_ffn, 2 * cfg.ffn, cfg.hidden),
          "down": (cfg.fmt_ffn, cfg.hidden, cfg.ffn)}
    base = {k: torch.from_numpy(make_q_weights(f, min(n, 1024), kk, 7)).to(dev).repeat((n + 1023) // 1024)[:ops.n_bytes(f, n, kk)]
            for k, (f, n, kk) in lw.items()}
    ones = torch.ones(cfg.hidden, dtype=torch.float32, device=dev)
    layers = [dict({k: v.clone() for k, v in base.items()}, attn_norm=ones, ffn_norm=ones) for _ in range(cfg.n_layers)]
    head = torch.from_numpy(make_q_weights(cfg.fmt_head, 4008, cfg.hidden, 3)).to(dev).repeat(32)
    embd = torch.from_numpy(make_q_weights(cfg.fmt_embd, 4008, cfg.hidden, 4)).to(dev).repeat(32)
    dstep = DecodeStep(cfg, layers, ones, head, dev, fuse=int(os.environ.get("CUT_DECODE_FUSE", "4")), embedding=embd)
    for kc, vc in zip(dstep.k_cache, dstep.v_cache):
        kc.normal_(0.0, 0.5)
        vc.normal_(0.0, 1.0)
    dstep.set_position(cfg.max_ctx - 1)

    def decode_step(_s):
        dstep.step()           # embedding row of the token the previous step sampled, 32 layers, head, arg-max
    wall_c, ev_c, _ = timed_graph(torch, decode_step, steps, 1, prime=True)
    w_bytes_tok = cfg.n_layers * sum(v.numel() for v in base.values()) + head.numel()
    kv_bytes_tok = cfg.n_layers * 2 * cfg.max_ctx * cfg.kv_dim * 2
    # What the launch bound of the attention costs: 256 cached positions, once in the 2048-position cache (the attention
    # launches, and reads, for 2048) and once with a cache and a launch bound of 256 (same weights).
    dstep.set_position(255)
    _, ev_short, _ = timed_graph(torch, decode_step, steps, 1, prime=True)
    import dataclasses
    cfg256 = dataclasses.replace(cfg, max_ctx=256)
    dstep256 = DecodeStep(cfg256, layers, ones, head, dev, fuse=int(os.environ.get("CUT_DECODE_FUSE", "4")), embedding=embd)
    for kc, vc in zip(dstep256.k_cache, dstep256.v_cache):
        kc.normal_(0.0, 0.5)
        vc.normal_(0.0, 1.0)
    dstep256.set_position(255)
    _, ev_256, _ = timed_graph(torch, lambda _s: dstep256.step(), steps, 1, prime=True)
    return {"decode_step_8b_ctx256_in_cache2048_ms_per_token": round(ev_short / steps, 3),
            "decode_step_8b_ctx256_in_cache256_ms_per_token": round(ev_256 / steps, 3),
            "decode_step_8b_ctx2048_ms_per_token": round(ev_c / steps, 3),
            "decode_step_8b_ctx2048_tok_per_s": round(steps * 1e3 / ev_c, 1),
            "decode_step_8b_ctx2048_GBps": round((w_bytes_tok + kv_bytes_tok) * steps / (ev_c * 1e-3) / 1e9, 1),
            "decode_step_8b_bytes_per_token": int(w_bytes_tok + kv_bytes_tok)}


def bench_prepare(torch, ops, dev, reps=10):
    """Load-time preparation of one FFN matrix (14336 x 4096) on the device: GGUF blocks -> separated [K, N] tensors
    (cuthip_prepare_sep) and fp32 -> Q8_0 blocks (cuthip_quantize_rows_q8_0); GB/s over bytes read + bytes written."""
    from cut_amd import lib
    res = {}
    N, K = N_FF, N_EMBD
    for name in ("Q8_0", "Q4_0", "Q4_K"):
        w = torch.from_numpy(make_q_weights(name, 1024, K, 5)).to(dev).repeat(N // 1024)
        q4 = name != "Q8_0"
        B = torch.empty((K, N // 2 if q4 else N), dtype=torch.uint8, device=dev)
        S = torch.empty(((2 if name == "Q4_K" else 1) * K // 32, N), dtype=torch.float16, device=dev)
        f = lib.FORMATS[name]

        def prep(_s):
            lib.check(lib.load().cuthip_prepare_sep(f, w.data_ptr(), N, K, B.data_ptr(), B.shape[1], S.data_ptr(), N,
                                                    torch.cuda.current_stream().cuda_stream))
        _, ev, _ = timed_graph(torch, prep, reps, 2)
        res[f"prepare_sep_{name}_14336x4096_GBps"] = round((w.numel() + B.numel() + S.numel() * 2) * reps / (ev * 1e-3) / 1e9, 1)
        del w, B, S
    # the separated tensors at prefill size (fp32 in / out as the reference): dequantize to fp16 + dense GEMM
    w = torch.from_numpy(make_q_weights("Q8_0", 1024, K, 5)).to(dev).repeat(N // 1024)
    Bq, Sq = ops.prepare_sep(w, "Q8_0", N, K)
    a = torch.randn((2048, K), dtype=torch.float32, device=dev)
    c = torch.empty((2048, N), dtype=torch.float32, device=dev)

    def sep(_s):
        ops.matmul_sep(a, Bq, Sq, N, out=c)
    _, ev, _ = timed_graph(torch, sep, 5, 2)
    res["separated_q8_prefill_gemm_M2048_N14336_K4096_TFLOPs"] = round(2.0 * 2048 * N * K * 5 / (ev * 1e-3) / 1e12, 1)
    # the same tensors at decode size (one row of fp32 activations): bytes of values + scales over the launch time, the
    # weights rotated over four copies; then the affine Q4 tensors the reference makes of Q4_K
    a1 = torch.randn((1, K), dtype=torch.float32, device=dev)
    c1 = torch.empty((1, N), dtype=torch.float32, device=dev)
    copies8 = [(Bq.clone(), Sq.clone()) for _ in range(4)]

    def sep1(s_):
        b_, s2_ = copies8[s_ % 4]
        ops.matmul_sep(a1, b_, s2_, N, out=c1)
    _, ev, _ = timed_graph(torch, sep1, 40, 4)
    res["separated_q8_gemv_14336x4096_GBps"] = round((Bq.numel() + Sq.numel() * 2) * 40 / (ev * 1e-3) / 1e9, 1)
    del copies8
    w4 = torch.from_numpy(make_q_weights("Q4_K", 1024, K, 6)).to(dev).repeat(N // 1024)
    B4, S4 = ops.prepare_sep(w4, "Q4_K", N, K)
    copies4 = [(B4.clone(), S4.clone()) for _ in range(4)]

    def sep4(s_):
        b_, s2_ = copies4[s_ % 4]
        ops.matmul_sep(a1, b_, s2_, N, q4=True, affine=True, out=c1)
    _, ev, _ = timed_graph(torch, sep4, 40, 4)
    res["separated_q4_affine_gemv_14336x4096_GBps"] = round((B4.numel() + S4.numel() * 2) * 40 / (ev * 1e-3) / 1e9, 1)
    del w, Bq, Sq, a, c, w4, B4, S4, copies4, a1, c1
    x = torch.randn(N * K, dtype=torch.float32, device=dev) * 0.02

    def quant(_s):
        ops.quantize_rows_q8_0(x)
    _, ev, _ = timed_graph(torch, quant, reps, 2)
    res["quantize_rows_q8_0_14336x4096_GBps"] = round((x.numel() * 4 + x.numel() // 32 * 34) * reps / (ev * 1e-3) / 1e9, 1)
    del x
    torch.cuda.empty_cache()
    return res


def bench_q8_prefill(torch, ops, dev, shapes=((512, N_FF, N_EMBD), (2048, N_FF, N_EMBD)), reps=10):
    """Q8_0 prefill GEMM: cuthip_matmul_q8_i8 (int8 activations per 32, int8 MFMA; TOP/s = 2MNK / time including
    the activation quantizer) and the fp16-activation path of cuthip_matmul_gguf on the same blocks."""
    res = {}
    for (M, N, K) in shapes:
        wq = torch.from_numpy(make_q_weights("Q8_0", 1024, K, 4)).to(dev).repeat(N // 1024)
        a = torch.randn((M, K), dtype=torch.float16, device=dev)
        c = torch.empty((M, N), dtype=torch.float16, device=dev)
        ws8 = torch.empty(lib_q8_ws(ops, M, K), dtype=torch.uint8, device=dev)
        ws = ops.matmul_gguf_workspace("Q8_0", M, K, N, a.dtype, dev)

        def i8(_s):
            ops.matmul_q8_i8(a, wq, N, K, out=c, workspace=ws8)

        def f16(_s):
            ops.matmul_gguf(a, wq, "Q8_0", N, K, out=c, workspace=ws)
        _, ev, _ = timed_graph(torch, i8, reps, 2)
        tops = 2.0 * M * N * K * reps / (ev * 1e-3) / 1e12
        res[f"q8_0_i8_prefill_gemm_M{M}_N{N}_K{K}_TOPs"] = round(tops, 1)
        res[f"q8_0_i8_prefill_gemm_M{M}_N{N}_K{K}_pct_of_int8_mfma_peak"] = round(tops / 5000.0 * 100, 1)
        _, ev, _ = timed_graph(torch, f16, reps, 2)
        res[f"q8_0_f16_prefill_gemm_M{M}_N{N}_K{K}_TFLOPs"] = round(2.0 * M * N * K * reps / (ev * 1e-3) / 1e12, 1)
        del wq, a, c, ws8, ws
    torch.cuda.empty_cache()
    return res


def lib_q8_ws(ops, M, K):
    from cut_amd import lib
    return max(int(lib.load().cuthip_matmul_q8_i8_workspace_bytes(M, K)), 16)


def calibrate_read(torch, lib, dev, reps=40):
    """A launch that only loads: cuthip_argmax's sibling would do, but the plainest read kernel at hand is the
    library's own dequant-free pass, cuthip_read_probe (16-byte loads, one xor per load, one store per workgroup).
    Timed under HIP-graph replay like the headline: 33,030,144-byte buffers (one FFN weight matrix) rotated over
    18 copies (594 MB, beyond L2 + Infinity Cache), and one 1 GiB buffer."""
    res = {}
    sink = torch.zeros(1 << 16, dtype=torch.int32, device=dev)
    small = [torch.randint(0, 255, (33030144,), dtype=torch.uint8, device=dev) for _ in range(18)]

    def rd_small(s):
        b = small[s % len(small)]
        lib.check(lib.load().cuthip_read_probe(b.data_ptr(), b.numel(), sink.data_ptr(), torch.cuda.current_stream().cuda_stream))
    _, ev, _ = timed_graph(torch, rd_small, reps * 3, 6)
    us = ev * 1e3 / (reps * 3)
    res["read_33MB_rotated_us_per_launch"] = round(us, 2)
    res["read_33MB_rotated_GBps"] = round(33030144 / us / 1e3, 1)
    del small
    torch.cuda.empty_cache()
    big = torch.randint(0, 255, (1 << 30,), dtype=torch.uint8, device=dev)

    def rd_big(_s):
        lib.check(lib.load().cuthip_read_probe(big.data_ptr(), big.numel(), sink.data_ptr(), torch.cuda.current_stream().cuda_stream))
    _, ev, _ = timed_graph(torch, rd_big, 10, 2)
    us = ev * 1e3 / 10
    res["read_1GiB_us_per_launch"] = round(us, 1)
    res["read_1GiB_GBps"] = round((1 << 30) / us / 1e3, 1)
    return res


def bench_dequant(torch, ops, dev, reps=20):
    """config 2: dequant of 256 Mi elements to fp16 (a 4 Mi-element tile of quantized N(0, 0.02) weights repeated
    64 times); GB/s = (block bytes in + fp16 bytes out) / kernel time from events."""
    res = {}
    n_el = 256 * 1024 * 1024
    out = torch.empty((n_el // 4096, 4096), dtype=torch.float16, device=dev)
    for name in ("Q8_0", "Q4_0", "Q4_K", "Q6_K"):
        tile = make_q_weights(name, 1024, 4096, 2)
        raw = torch.from_numpy(tile).to(dev).repeat(64)
        in_bytes = raw.numel()

        def dq(_s, raw=raw, name=name):
            ops.dequantize(raw, name, n_el // 4096, 4096, torch.float16, out=out)
        wall_d, ev_d, _ = timed_graph(torch, dq, reps, 3)
        res[f"dequant_{name}_to_f16_256Mi_GBps"] = round((in_bytes + n_el * 2) * reps / (ev_d * 1e-3) / 1e9, 1)
        del raw
    del out
    torch.cuda.empty_cache()
    return res


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=2000)
    ap.add_argument("--warmup", type=int, default=100)
    ap.add_argument("--no-extras", action="store_true", help="skip the other configurations")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline")
    ap.add_argument("--calibrate-copy", action="store_true",
                    help="only run a plain 1 GiB device copy 5 times (reference traffic for rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE)")
    ap.add_argument("--calibrate-read", action="store_true",
                    help="only time a plain read kernel (torch's sum) over 33 MB buffers rotated through 594 MB and over "
                         "1 GiB: what a launch of the headline GEMV's size can reach on this part when it only loads")
    ap.add_argument("--gemm-variant", type=int, default=4, choices=(2, 4, 5),
                    help="with --gemm-only: 4 = dequantize once + hand-written dense GEMM (default), 5 = dequantize once + hipBLASLt, 2 = single-launch GEMM")
    ap.add_argument("--gemm-down", action="store_true", help="with --gemm-only: the down-projection shape (N = 4096, K = 14336)")
    ap.add_argument("--gemm-only", type=int, default=0, metavar="M",
                    help="only run the Q4_K prefill GEMM (M x 4096) . (14336 x 4096)^T twelve times (target of rocprofv3 runs)")
    ap.add_argument("--dequant-only", action="store_true",
                    help="only run the 256 Mi-element dequant of the four formats (target of rocprofv3 runs)")
    ap.add_argument("--prepare-only", action="store_true", help="only run the load-time preparation kernels")
    ap.add_argument("--q8-only", action="store_true",
                    help="only run the Q8_0 prefill GEMMs at M = 2048 (int8-activation variant and fp16 path)")
    ap.add_argument("--matmul-batch-only", type=int, default=0, metavar="B",
                    help="only run the FFN step at B rows (9..256) through the workspace entry point, for profiling")
    ap.add_argument("--gemv-batch-only", type=int, default=0, metavar="B",
                    help="only run the FFN GEMV step at batch B (2..8), for profiling")
    ap.add_argument("--prime-seconds", type=float, default=PRIME_SECONDS,
                    help="untimed replays of a graph of short launches in front of its timed replay last this long (0 = one replay)")
    ap.add_argument("--decode-only", action="store_true",
                    help="only run the 8B-shape decode step (target of rocprofv3 runs)")
    ap.add_argument("--head-only", action="store_true",
                    help="only run the batch-1 GEMV at the output-head shape (128256 x 4096) on Q6_K and on Q4_K, for profiling")
    args = ap.parse_args()
    globals()["PRIME_SECONDS"] = max(args.prime_seconds, 0.0)
    if args.gpus != 1:
        log("bench.py: this build measures one GPU only (--gpus 1); multi-GPU runs are not part of it")
        sys.exit(2)

    import numpy as np
    import torch
    from cut_amd import lib, ops

    lib.check(lib.load().cuthip_init(0))
    info = lib.device_info()
    dev = torch.device("cuda:0")
    if args.calibrate_copy:
        src = torch.ones(1 << 28, dtype=torch.float32, device=dev)
        dst = torch.empty_like(src)
        for _ in range(5):
            dst.copy_(src)
        torch.cuda.synchronize()
        print(json.dumps({"calibrate_copy_bytes_read": src.numel() * 4, "bytes_written": src.numel() * 4, "launches": 5}))
        return
    if args.calibrate_read:
        print(json.dumps(calibrate_read(torch, lib, dev)))
        return
    if args.dequant_only:
        print(json.dumps(bench_dequant(torch, ops, dev, reps=5)))
        return
    if args.prepare_only:
        print(json.dumps(bench_prepare(torch, ops, dev)))
        return
    if args.q8_only:
        print(json.dumps(bench_q8_prefill(torch, ops, dev, shapes=((2048, N_FF, N_EMBD),), reps=5)))
        return
    if args.head_only:
        res = {}
        xh = torch.randn((1, N_EMBD), dtype=torch.float16, device=dev)
        logits = torch.empty((1, 128256), dtype=torch.float16, device=dev)
        for fname in ("Q6_K", "Q4_K"):
            head = torch.from_numpy(make_q_weights(fname, 4008, N_EMBD, 3)).to(dev).repeat(32)   # 4008 rows, repeated
            heads = [head, head.clone()]

            def lm_head(s_):
                ops.matmul_gguf(xh, heads[s_ % 2], fname, 128256, N_EMBD, out=logits)
            _, ev_h, _ = timed_graph(torch, lm_head, 20, 3)
            res[f"{fname.lower()}_gemv_128256x4096_GBps"] = round((head.numel() + 2 * (N_EMBD + 128256)) * 20 / (ev_h * 1e-3) / 1e9, 1)
            res[f"{fname.lower()}_gemv_128256x4096_us"] = round(ev_h * 1e3 / 20, 1)
            del heads, head
            torch.cuda.empty_cache()
        print(json.dumps(res))
        return
    if args.decode_only:
        x_h = np.random.default_rng(1).standard_normal((8, N_EMBD), dtype=np.float32).astype(np.float16)
        print(json.dumps(bench_decode_step(torch, np, ops, dev, x_h)))
        return
    if args.gemm_only:
        M = args.gemm_only
        GN, GK = (N_EMBD, N_FF) if args.gemm_down else (N_FF, N_EMBD)
        wq = torch.from_numpy(make_q_weights("Q4_K", GN, GK, 0)).to(dev)
        a = torch.randn((M, GK), dtype=torch.float16, device=dev)
        c = torch.empty((M, GN), dtype=torch.float16, device=dev)
        # variant 4 = dequantize once + dense GEMM (two launches, both inside the timed region); 2 = single launch
        ws = ops.matmul_gguf_workspace("Q4_K", M, GK, GN, a.dtype, dev) if args.gemm_variant >= 4 else None
        for _ in range(2):
            ops.matmul_gguf(a, wq, "Q4_K", GN, GK, out=c, variant=args.gemm_variant, workspace=ws)
        torch.cuda.synchronize()
        ev0, ev1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        ev0.record()
        for _ in range(10):
            ops.matmul_gguf(a, wq, "Q4_K", GN, GK, out=c, variant=args.gemm_variant, workspace=ws)
        ev1.record()
        torch.cuda.synchronize()
        us = ev0.elapsed_time(ev1) * 1e3 / 10
        print(json.dumps({"gemm": f"Q4_K M={M} N={GN} K={GK}", "variant": args.gemm_variant,
                          "us_per_matmul": round(us, 1), "TFLOPs": round(2.0 * M * GN * GK / us / 1e6, 1)}))
        return
    log(f"[bench] {info['name']} {info['arch']} CUs={info['compute_units']}")

    # ---- resident inputs ---------------------------------------------------
    t_in = time.time()
    w_up_h = make_q_weights("Q4_K", N_FF, N_EMBD, 0)
    w_down_h = make_q_weights("Q4_K", N_EMBD, N_FF, 1)
    gate = [torch.from_numpy(w_up_h).to(dev).clone() for _ in range(COPIES)]
    up = [torch.from_numpy(w_up_h).to(dev).clone() for _ in range(COPIES)]
    down = [torch.from_numpy(w_down_h).to(dev).clone() for _ in range(COPIES)]
    rng = np.random.default_rng(1)
    x_h = rng.standard_normal((8, N_EMBD), dtype=np.float32).astype(np.float16)
    h_h = rng.standard_normal((8, N_FF), dtype=np.float32).astype(np.float16)
    x, h = torch.from_numpy(x_h).to(dev), torch.from_numpy(h_h).to(dev)
    y_gate = torch.empty((8, N_FF), dtype=torch.float16, device=dev)
    y_up = torch.empty((8, N_FF), dtype=torch.float16, device=dev)
    y_down = torch.empty((8, N_EMBD), dtype=torch.float16, device=dev)
    torch.cuda.synchronize()
    log(f"[bench] inputs ready in {time.time() - t_in:.1f}s")

    w_bytes = ops.n_bytes("Q4_K", N_FF, N_EMBD)  # 33,030,144 for either shape

    def ffn_step(b):
        # batch 2-8: with a workspace the long-row down projection splits K across workgroups
        ws_down = ops.matmul_gguf_workspace("Q4_K", b, N_FF, N_EMBD, torch.float16, dev) if b >= 2 else None

        def step(s):
            i = s % COPIES
            ops.matmul_gguf(x[:b], gate[i], "Q4_K", N_FF, N_EMBD, out=y_gate[:b])
            ops.matmul_gguf(x[:b], up[i], "Q4_K", N_FF, N_EMBD, out=y_up[:b])
            ops.matmul_gguf(h[:b], down[i], "Q4_K", N_EMBD, N_FF, out=y_down[:b], workspace=ws_down)
        return step

    def ffn_bytes(b):
        return 3 * w_bytes + b * 2 * (2 * (N_EMBD + N_FF) + (N_FF + N_EMBD))

    def ffn_step_ws(b):
        # 9 rows and more: the three matmuls through cuthip_matmul_gguf_ws, whose workspace lets the streaming MFMA
        # kernel and the tiled GEMM split K
        xb = torch.from_numpy(rng.standard_normal((b, N_EMBD), dtype=np.float32).astype(np.float16)).to(dev)
        hb = torch.from_numpy(rng.standard_normal((b, N_FF), dtype=np.float32).astype(np.float16)).to(dev)
        yb_ff = torch.empty((b, N_FF), dtype=torch.float16, device=dev)
        yb_em = torch.empty((b, N_EMBD), dtype=torch.float16, device=dev)
        ws_b = ops.matmul_gguf_workspace("Q4_K", b, N_FF, N_EMBD, torch.float16, dev)

        def step(s):
            i = s % COPIES
            ops.matmul_gguf(xb, gate[i], "Q4_K", N_FF, N_EMBD, out=yb_ff, workspace=ws_b)
            ops.matmul_gguf(xb, up[i], "Q4_K", N_FF, N_EMBD, out=yb_ff, workspace=ws_b)
            ops.matmul_gguf(hb, down[i], "Q4_K", N_EMBD, N_FF, out=yb_em, workspace=ws_b)
        return step

    if args.matmul_batch_only:
        b = args.matmul_batch_only
        wall_b, ev_b, _ = timed_graph(torch, ffn_step_ws(b), 60, 6, prime=True)
        print(json.dumps({f"q4k_ffn_matmul_batch{b}_GBps": round(ffn_bytes(b) * 60 / wall_b / 1e9, 1),
                          "us_per_matmul": round(ev_b * 1e3 / 180, 2)}))
        return
    if args.gemv_batch_only:
        b = args.gemv_batch_only
        wall_b, ev_b, _ = timed_graph(torch, ffn_step(b), 120, 12, prime=True)
        print(json.dumps({f"q4k_ffn_gemv_batch{b}_GBps": round(ffn_bytes(b) * 120 / wall_b / 1e9, 1),
                          "us_per_launch": round(ev_b * 1e3 / 360, 2)}))
        return
    # ---- headline: batch 1 --------------------------------------------------
    wall, ev_ms, used_graph = timed_graph(torch, ffn_step(1), args.steps, args.warmup, prime=True)
    step_bytes = ffn_bytes(1)
    value = step_bytes * args.steps / wall / 1e9
    launches = 3 * args.steps
    avg_launch_us = ev_ms * 1e3 / launches
    launch_bytes = step_bytes / 3.0
    achieved = launch_bytes / (avg_launch_us * 1e-6) / 1e9
    log(f"[bench] b=1: {value:.0f} GB/s wall, {achieved:.0f} GB/s by events ({avg_launch_us:.2f} us per launch)")

    result = {
        "metric": "Q4_K GEMV achieved HBM GB/s",
        "value": round(value, 1),
        "unit": "GB/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": round(wall / args.steps * 1e3, 5),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "f16",
        "data": "synthetic",
        "config": {"workload": "BASELINE configs[2]: Q4_K GEMV, FFN shapes 14336x4096 (gate, up) + 4096x14336 (down), "
                               "batch 1, fp16 in/out, fp32 accumulate; one step = the three GEMVs of one FFN block",
                   "weight_copies_rotated": COPIES, "hip_graph": used_graph, "pct_of_hbm_peak": round(value / HBM_PEAK_GBS * 100, 1)},
        "roofline": {"bound": "hbm", "achieved": round(achieved, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s",
                     "frac": round(achieved / HBM_PEAK_GBS, 4), "traffic": TRAFFIC_BYTES_PER_LAUNCH,
                     "kernel": "cuthip::gemv_rows8_kernel<Q4_K, MT=1>", "algorithmic_bytes_per_launch": int(launch_bytes),
                     "avg_launch_us": round(avg_launch_us, 3)},
    }

    # ---- other configurations ---------------------------------------------------
    extras = {}
    if not args.no_extras:
        for b in (2, 4, 8):
            wall_b, ev_b, _ = timed_graph(torch, ffn_step(b), 120, 12, prime=True)
            extras[f"q4k_ffn_gemv_batch{b}_GBps"] = round(ffn_bytes(b) * 120 / wall_b / 1e9, 1)
        # 16-128 rows (batched decode, short prefill chunks): the same three matmuls through cuthip_matmul_gguf_ws;
        # GB/s over the same bytes
        for b in (16, 32, 64, 128):
            wall_b, ev_b, _ = timed_graph(torch, ffn_step_ws(b), 60, 6, prime=True)
            extras[f"q4k_ffn_matmul_batch{b}_GBps"] = round(ffn_bytes(b) * 60 / wall_b / 1e9, 1)
            extras[f"q4k_ffn_matmul_batch{b}_us_per_matmul"] = round(wall_b * 1e6 / 180, 1)
        # gate and up as one launch (rows concatenated, the reference's fused w_gate_up: llama.cpp:1288-1330)
        gate_up = [torch.cat([gate[i], up[i]]) for i in range(COPIES)]
        y_gu = torch.empty((1, 2 * N_FF), dtype=torch.float16, device=dev)

        def gu_step(s):
            ops.matmul_gguf(x[:1], gate_up[s % COPIES], "Q4_K", 2 * N_FF, N_EMBD, out=y_gu)
        wall_gu, ev_gu, _ = timed_graph(torch, gu_step, 120, 12)
        gu_bytes = 2 * w_bytes + 2 * (N_EMBD + 2 * N_FF)
        extras["q4k_gate_up_fused_28672x4096_gemv_GBps"] = round(gu_bytes * 120 / (ev_gu * 1e-3) / 1e9, 1)
        del gate, up, down, gate_up
        torch.cuda.empty_cache()
        extras.update(bench_decode_step(torch, np, ops, dev, x_h))
        torch.cuda.empty_cache()
        extras.update(bench_dequant(torch, ops, dev))
        # LM head: Q6_K 128256 x 4096, batch 1 (431 MB per launch: streams from HBM by itself)
        head = torch.from_numpy(make_q_weights("Q6_K", 4008, 4096, 3)).to(dev).repeat(32)
        logits = torch.empty((1, 128256), dtype=torch.float16, device=dev)

        def lm_head(_s):
            ops.matmul_gguf(x[:1], head, "Q6_K", 128256, N_EMBD, out=logits)
        wall_h, ev_h, _ = timed_graph(torch, lm_head, 20, 3)
        extras["q6k_lm_head_128256x4096_gemv_GBps"] = round((head.numel() + 2 * (4096 + 128256)) * 20 / (ev_h * 1e-3) / 1e9, 1)
        del head, logits
        torch.cuda.empty_cache()
        # Q6_K at the FFN down-projection shape (half the down projections of a Q4_K_M file are Q6_K): 48 MB per launch,
        # six copies rotated
        q6_h = make_q_weights("Q6_K", N_EMBD, N_FF, 4)
        q6 = [torch.from_numpy(q6_h).to(dev).clone() for _ in range(COPIES)]
        y6 = torch.empty((1, N_EMBD), dtype=torch.float16, device=dev)

        def q6_down(s):
            ops.matmul_gguf(h[:1], q6[s % COPIES], "Q6_K", N_EMBD, N_FF, out=y6)
        wall_6, ev_6, _ = timed_graph(torch, q6_down, 60, 6)
        extras["q6k_gemv_4096x14336_GBps"] = round((q6[0].numel() + 2 * (N_FF + N_EMBD)) * 60 / (ev_6 * 1e-3) / 1e9, 1)
        del q6, y6
        torch.cuda.empty_cache()
        # the other three formats at the gate / up shape, batch 1 (the headline is the same launch on Q4_K): bytes of the
        # blocks + fp16 x and y over the launch time, six copies rotated
        yf = torch.empty((1, N_FF), dtype=torch.float16, device=dev)
        for fname in ("Q4_0", "Q6_K", "Q8_0"):
            wf_h = torch.from_numpy(make_q_weights(fname, 1024, N_EMBD, 7)).to(dev).repeat(N_FF // 1024)   # 1024 rows, repeated
            wf = [wf_h.clone() for _ in range(COPIES)]

            def gemv_f(s):
                ops.matmul_gguf(x[:1], wf[s % COPIES], fname, N_FF, N_EMBD, out=yf)
            _, ev_f, _ = timed_graph(torch, gemv_f, 60, 6)
            extras[f"{fname.lower()}_gemv_14336x4096_GBps"] = round((wf[0].numel() + 2 * (N_FF + N_EMBD)) * 60 / (ev_f * 1e-3) / 1e9, 1)
            del wf, wf_h
            torch.cuda.empty_cache()
        del yf
        # config 5: prefill GEMM, Q4_K weights, fp16 activations, fp16 MFMA with fp32 accumulate.  The headline keys
        # (q4k_prefill_gemm_*_TFLOPs, *_pct_of_f16_mfma_peak) are this library's own kernels through its own choice
        # by shape; the vendor library's GEMM behind the same dequantization (variant 5, opt-in) is reported under
        # vendor_hipblaslt_* keys, and the GEMM on weights kept dequantized (another workload: no dequantization
        # inside the call) under dense_f16_* keys.
        have_vendor = lib.load().cuthip_variant_available(lib.OP_MATMUL_GGUF, 5) == 1
        extras["prefill_automatic_choice"] = "hand-written kernels only (MatMulGgufDequantGemm / MatMulGgufGemmLds)"
        for (M, N, K) in ((512, N_FF, N_EMBD), (2048, N_FF, N_EMBD), (512, N_EMBD, N_FF), (2048, N_EMBD, N_FF)):
            w_h = w_up_h if N == N_FF else w_down_h
            wq = torch.from_numpy(w_h).to(dev)
            a = torch.randn((M, K), dtype=torch.float16, device=dev)
            c = torch.empty((M, N), dtype=torch.float16, device=dev)
            ws = ops.matmul_gguf_workspace("Q4_K", M, K, N, a.dtype, dev)

            def mk(variant, a=a, wq=wq, c=c, N=N, K=K, ws=ws):
                def run(_s):
                    ops.matmul_gguf(a, wq, "Q4_K", N, K, out=c, variant=variant, workspace=ws if variant != 2 else None)
                return run
            key = f"q4k_prefill_gemm_M{M}_N{N}_K{K}"
            tf = {}
            for label, variant in (("auto", -1), ("own_two_pass", 4), ("single_launch", 2)) + ((("vendor", 5),) if have_vendor else ()):
                _, ev_g, _ = timed_graph(torch, mk(variant), 10, 2)
                tf[label] = 2.0 * M * N * K * 10 / (ev_g * 1e-3) / 1e12
            extras[f"{key}_TFLOPs"] = round(tf["auto"], 1)
            extras[f"{key}_pct_of_f16_mfma_peak"] = round(tf["auto"] / 2500.0 * 100, 1)
            extras[f"{key}_own_two_pass_TFLOPs"] = round(tf["own_two_pass"], 1)
            extras[f"{key}_single_launch_TFLOPs"] = round(tf["single_launch"], 1)
            if have_vendor:
                extras[f"vendor_hipblaslt_dequant_gemm_M{M}_N{N}_K{K}_TFLOPs"] = round(tf["vendor"], 1)
            # another workload: the same product on weights that are kept dequantized (fp16 [N, K], 2 bytes per weight)
            w16 = ops.dequantize(wq, "Q4_K", N, K, torch.float16)
            ws16 = torch.empty(max(int(lib.load().cuthip_matmul_dense_f16_workspace_bytes(M, K, N, lib.F16)), 256),
                               dtype=torch.uint8, device=dev)

            def gemm16(_s, a=a, w16=w16, c=c, ws16=ws16):
                ops.matmul_dense_f16(a, w16, out=c, workspace=ws16)
            _, ev_g, _ = timed_graph(torch, gemm16, 10, 2)
            extras[f"dense_f16_gemm_M{M}_N{N}_K{K}_TFLOPs"] = round(2.0 * M * N * K * 10 / (ev_g * 1e-3) / 1e12, 1)
            del ws, w16, ws16
            del wq, a, c
        # config 5, second half: Q8_0 weights with activations quantized to int8 per 32 on the int8 matrix core
        # (both launches, quantizer + GEMM, inside the timed region), next to the fp16 path on the same blocks
        extras.update(bench_q8_prefill(torch, ops, dev))
        extras.update(bench_prepare(torch, ops, dev))
    result["extras"] = extras

    # ---- CPU baseline: the oracle's restatement of the reference path -------------
    # Two loops, both single-threaded as the reference's: (1) `value`: dequantize one row of GGUF blocks, contiguous
    # fp32 dot (the CPU dequant the matmul tolerance is defined against, followed by A . W^T); (2) the harness's
    # triple loop on the reference loader's separated [K, N] tensors, B read column-strided, term order (a * q) * s
    # (tests/harness/OpRegistry.h:2043-2051; Q4_K goes through the runner's affine Q4 form), reported beside it.
    if not args.no_cpu:
        import oracle
        a1 = x_h[:1].astype(np.float32)
        h1 = h_h[:1].astype(np.float32)
        t0 = time.perf_counter()
        reps = 0
        while True:
            oracle.matmul_gguf(oracle.Q4_K, w_up_h, a1, N_FF)
            oracle.matmul_gguf(oracle.Q4_K, w_up_h, a1, N_FF)
            oracle.matmul_gguf(oracle.Q4_K, w_down_h, h1, N_EMBD)
            reps += 1
            if time.perf_counter() - t0 > 10.0 or reps >= 100:
                break
        cpu_s = (time.perf_counter() - t0) / reps
        up_p, up_s = oracle.requantize_q4k_to_affine(w_up_h, N_FF, N_EMBD)
        dn_p, dn_s = oracle.requantize_q4k_to_affine(w_down_h, N_EMBD, N_FF)
        up_sf, dn_sf = oracle.f16_to_f32_array(up_s).reshape(up_s.shape), oracle.f16_to_f32_array(dn_s).reshape(dn_s.shape)
        t0 = time.perf_counter()
        reps_h = 0
        while True:
            oracle.matmul_sep_q4(a1, up_p, up_sf, affine=True)
            oracle.matmul_sep_q4(a1, up_p, up_sf, affine=True)
            oracle.matmul_sep_q4(h1, dn_p, dn_sf, affine=True)
            reps_h += 1
            if time.perf_counter() - t0 > 10.0 or reps_h >= 100:
                break
        harness_s = (time.perf_counter() - t0) / reps_h
        result["cpu_baseline"] = {
            "value": round(step_bytes / cpu_s / 1e9, 3), "unit": "GB/s", "cores": 1, "kind": "port",
            "harness_loop_value": round(step_bytes / harness_s / 1e9, 3),
            "sample": f"{reps} full FFN steps (gate, up, down GEMV at batch 1) through oracle/cut_oracle.c, loop "
                      f"orc_matmul_gguf_f32 (dequantize one row of GGUF blocks, fp32 sequential dot): {cpu_s * 1e3:.0f} ms "
                      f"per step = value; {reps_h} steps through orc_matmul_sep_q4_f32 (the harness's triple loop on the "
                      f"separated affine-Q4 [K, N] tensors, column-strided): {harness_s * 1e3:.0f} ms per step = "
                      f"harness_loop_value; host has {os.cpu_count()} logical cores, one used"}
    print(json.dumps(result), flush=True)


if __name__ == "__main__":
    main()
