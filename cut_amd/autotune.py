"""Autotune sweep for the "hip" section of tuning_data.json (the reference derives its sections with
scripts/bench/derive_rules.py from an autotune binary's output).

    python -m cut_amd.autotune [--output cut_amd/tuning_data.json] [--reps 20]

For every (format, M, K, N) of the sweep each variant of the MatMulGguf table that accepts the shape is timed through
the C ABI (HIP events, weights rotated over several copies so that small matrices are not served from cache) and the
fastest hand-written one (with --with-vendor: fastest of all) becomes an exact-shape rule
`{"variant": v, "conditions": {"shape": [M, K, N]}}` under operators.MatMulGguf<fmt>.backends.hip where it beats the
library's own choice by 6 % or more in every one of --sweeps (default 2) complete passes over the shapes, the same
variant winning each time: timings of one launch repeat within 2-4 % on this part, so a smaller or unrepeated win is
noise and a rule made of it pins a shape to what may be the slower kernel.  The entry's default variant is -1 (the
library's own choice by shape).  Needs an MI355X; refuses to run without one."""
import argparse
import json
import os
import sys

SHAPES_NK = [(14336, 4096), (4096, 14336), (4096, 4096), (1024, 4096), (28672, 4096)]
BATCHES = [1, 2, 4, 8, 16, 32, 64, 128, 256, 512, 1024, 2048]
FORMATS = ["Q4_K", "Q6_K", "Q8_0"]


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--output", default=os.path.join(os.path.dirname(os.path.abspath(__file__)), "tuning_data.json"))
    ap.add_argument("--reps", type=int, default=20)
    ap.add_argument("--sweeps", type=int, default=2, help="complete passes; a rule needs the same winner in all of them")
    ap.add_argument("--min-gain", type=float, default=0.06, help="a rule needs the winner faster by this fraction in every pass")
    ap.add_argument("--formats", default=",".join(FORMATS))
    ap.add_argument("--batches", default=",".join(str(b) for b in BATCHES), help="rows of activations to sweep (comma separated)")
    ap.add_argument("--measurements", default=None, help="also write every timing of the sweep to this JSON file")
    ap.add_argument("--with-vendor", action="store_true",
                    help="let rules name the dequantize + hipBLASLt variant too (it is timed and logged either way)")
    args = ap.parse_args()
    import numpy as np
    import torch
    if not torch.cuda.is_available():
        sys.exit("autotune: no GPU")
    from cut_amd import lib, ops, quantize as Q
    lib.check(lib.load().cuthip_init(0))
    dev = torch.device("cuda:0")
    names = [v["name"] for v in lib.variants(lib.OP_MATMUL_GGUF)]
    def sweep(fmt, log):
        """One pass over the shapes of a format: {(M, K, N): (winner, its us, the library's choice us)}."""
        wins = {}
        for (N, K) in SHAPES_NK:
            tile = Q.quantize(fmt, np.random.default_rng(0).standard_normal(1024 * K, dtype=np.float32) * np.float32(0.02))
            w = torch.from_numpy(tile).to(dev).repeat(N // 1024)
            copies = [w.clone() for _ in range(max(2, min(8, int(3e8 // w.numel()))))]
            for M in [int(b) for b in args.batches.split(",")]:
                a = torch.randn((M, K), dtype=torch.float16, device=dev)
                c = torch.empty((M, N), dtype=torch.float16, device=dev)
                ws = ops.matmul_gguf_workspace(fmt, M, K, N, a.dtype, dev)
                best, auto_us = None, None
                for v in [-1] + list(range(len(names))) + [-1]:   # the library's choice first and last: the faster one counts
                    try:
                        for i in range(2):
                            ops.matmul_gguf(a, copies[i % len(copies)], fmt, N, K, out=c, variant=v, workspace=ws)
                        torch.cuda.synchronize()
                    except lib.CutHipError:
                        continue          # the variant does not take this shape
                    # the launches are replayed as one HIP graph: timed eagerly, anything under ~10 us would
                    # measure the host's launch rate instead of the kernel
                    g = torch.cuda.CUDAGraph()
                    with torch.cuda.graph(g):
                        for i in range(args.reps):
                            ops.matmul_gguf(a, copies[i % len(copies)], fmt, N, K, out=c, variant=v, workspace=ws)
                    g.replay()
                    torch.cuda.synchronize()
                    us = float("inf")
                    for _ in range(3):    # the fastest of three replays: the first ones on fresh buffers run slow
                        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
                        e0.record()
                        g.replay()
                        e1.record()
                        torch.cuda.synchronize()
                        us = min(us, e0.elapsed_time(e1) * 1e3 / args.reps)
                    del g
                    if v == -1:
                        if auto_us is not None:   # second pass: keep the faster timing, one log entry
                            auto_us = min(auto_us, us)
                            next(e for e in reversed(log) if e["shape"] == [M, K, N] and e["variant"] == -1)["us"] = round(auto_us, 2)
                            if auto_us <= best[1]:
                                best = (-1, auto_us)
                            continue
                        auto_us = us
                    log.append({"shape": [M, K, N], "variant": v, "us": round(us, 2)})
                    if names[v] == "MatMulGgufDequantBlasLt" and v >= 0 and not args.with_vendor:
                        continue
                    if best is None or us < best[1]:
                        best = (v, us)
                print(f"{fmt} M={M} K={K} N={N}: variant {best[0]} {best[1]:.1f} us (library's choice {auto_us:.1f})", flush=True)
                wins[(M, K, N)] = (best[0], best[1], auto_us)
                del ws
            del copies, w
            torch.cuda.empty_cache()
        return wins

    operators, measurements = {}, {}
    for fmt in args.formats.split(","):
        log = []
        passes = [sweep(fmt, log) for _ in range(args.sweeps)]
        rules = []
        for shape, (v, _us, _auto) in passes[0].items():
            # a rule only where the same named variant beats the library's own choice clearly in every pass
            if v >= 0 and all(p[shape][0] == v and p[shape][1] <= (1.0 - args.min_gain) * p[shape][2] for p in passes):
                rules.append({"variant": v, "conditions": {"shape": list(shape)}})
                print(f"rule: {fmt} {list(shape)} -> variant {v} ({names[v]}): " +
                      ", ".join(f"{p[shape][1]:.1f} against {p[shape][2]:.1f} us" for p in passes), flush=True)
        operators[f"MatMulGguf{fmt}"] = {"backends": {"hip": {"default_variant": -1, "rules": rules}}}
        measurements[f"MatMulGguf{fmt}"] = log
    info = lib.device_info()
    out = {"device": info["name"], "arch": info["arch"], "variant_names": names, "operators": operators}
    with open(args.output, "w") as fh:
        json.dump(out, fh, separators=(",", ":"))
        fh.write("\n")
    print(f"wrote {args.output}")
    if args.measurements:
        with open(args.measurements, "w") as fh:
            json.dump(measurements, fh, separators=(",", ":"))
            fh.write("\n")


if __name__ == "__main__":
    main()
