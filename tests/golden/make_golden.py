"""Writes tests/golden/dequant_golden.npz from the reference's own GGUF reader.

Runs only where the reference tree is mounted: it calls oracle/_ref
(libcut_ref.so = the reference's gguf_reader.cpp compiled where it lies,
behind oracle/ref_driver.cpp) on seeded block bytes and stores inputs and the
fp32 bit patterns the reference produced.  The fixture is data only.

    python tests/golden/make_golden.py
"""
import os
import sys

import numpy as np

sys.path.insert(0, os.path.join(os.path.dirname(__file__), "..", ".."))
import oracle  # noqa: E402

ROWS, COLS = 8, 1024  # 8 rows of 4 (K-quant) / 32 (32-wide) blocks


def finite_random_blocks(fmt, rng, n_elems):
    """Uniformly random block bytes with the fp16 scale fields forced finite."""
    nb = oracle.n_bytes(fmt, n_elems)
    b = rng.integers(0, 256, nb, dtype=np.uint8)
    bb = oracle.BLOCK_BYTES[fmt]
    blocks = b.reshape(-1, bb)
    offs = {oracle.Q8_0: [0], oracle.Q4_0: [0], oracle.Q4_K: [0, 2], oracle.Q6_K: [208]}[fmt]
    for off in offs:
        hi = blocks[:, off + 1]
        bad = (hi & 0x7C) == 0x7C  # exponent all ones -> Inf/NaN
        hi[bad] &= 0xFB
    return blocks.reshape(-1)


def main():
    if not oracle.have_ref():
        oracle.build()
    rng = np.random.default_rng(20240607)
    out = {}
    for name, fmt in oracle.FORMATS.items():
        n = ROWS * COLS
        rnd = finite_random_blocks(fmt, rng, n)
        gauss = oracle.quantize(fmt, rng.standard_normal(n).astype(np.float32) * 0.02)
        for tag, blocks in (("random", rnd), ("gauss", gauss)):
            ref = oracle.ref_dequant(fmt, blocks, ROWS, COLS)
            out[f"{name}_{tag}_blocks"] = blocks
            out[f"{name}_{tag}_f32bits"] = ref.view(np.uint32)
    # separated readers (gguf_reader.cpp:389-501)
    q8 = out["Q8_0_random_blocks"]
    v, s = oracle.ref_split_q8(q8, ROWS, COLS)
    out["Q8_0_split_values"], out["Q8_0_split_scales"] = v, s
    q4 = out["Q4_0_random_blocks"]
    v, s = oracle.ref_split_q4(q4, ROWS, COLS)
    out["Q4_0_split_packed"], out["Q4_0_split_scales"] = v, s
    path = os.path.join(os.path.dirname(__file__), "dequant_golden.npz")
    np.savez_compressed(path, rows=ROWS, cols=COLS, **out)
    print("wrote", path, os.path.getsize(path), "bytes")


if __name__ == "__main__":
    main()
