"""Shared test helpers (CPU side): seeded inputs and error metrics."""
import numpy as np

import oracle


def stl_uniform(n: int, seed: int, a: float, b: float) -> np.ndarray:
    """std::mt19937(seed) + std::uniform_real_distribution<float>(a, b) as
    libstdc++ evaluates it (one 32-bit draw per value, canonical = raw/2^32 in
    float, clamped below 1) -- the generator behind generateTestData<float>
    (OpRefs.h:241-264) and the Mistral-geometry test (RuntimeTests.cpp:2865-2868).
    Pinned by test_oracle_matmul.test_stl_uniform_known_values."""
    rs = np.random.RandomState(seed)  # init_genrand(seed), like std::mt19937
    raw = rs.randint(0, 2 ** 32, size=n, dtype=np.uint64).astype(np.uint32)
    c = raw.astype(np.float32) / np.float32(4294967296.0)
    c = np.where(c >= 1.0, np.nextafter(np.float32(1), np.float32(0)), c).astype(np.float32)
    return (c * (np.float32(b) - np.float32(a)) + np.float32(a)).astype(np.float32)


def generate_test_data(n: int, seed: int = 42) -> np.ndarray:
    return stl_uniform(n, seed, 0.1, 10.0)


def gauss_weights(n_elems: int, seed: int = 0, sigma: float = 0.02) -> np.ndarray:
    """fp32 N(0, sigma) from numpy's PCG64 stream (same on every box)."""
    return (np.random.default_rng(seed).standard_normal(n_elems, dtype=np.float32) * np.float32(sigma))


def gauss_acts(shape, seed: int = 1, dtype=np.float32) -> np.ndarray:
    return np.random.default_rng(seed).standard_normal(shape, dtype=np.float32).astype(dtype)


def quantized_weights(fmt: int, N: int, K: int, seed: int = 0) -> np.ndarray:
    return oracle.quantize(fmt, gauss_weights(N * K, seed))


def finite_random_blocks(fmt: int, n_blocks: int, seed: int) -> np.ndarray:
    """Uniformly random block bytes with finite fp16 scale fields."""
    rng = np.random.default_rng(seed)
    b = rng.integers(0, 256, (n_blocks, oracle.BLOCK_BYTES[fmt]), dtype=np.uint8)
    for off in {oracle.Q8_0: [0], oracle.Q4_0: [0], oracle.Q4_K: [0, 2], oracle.Q6_K: [208]}[fmt]:
        bad = (b[:, off + 1] & 0x7C) == 0x7C
        b[bad, off + 1] &= 0xFB
    return b.reshape(-1)


def normwise_rel_err(got, ref) -> float:
    got = np.asarray(got, np.float64).reshape(-1)
    ref = np.asarray(ref, np.float64).reshape(-1)
    return float(np.linalg.norm(got - ref) / max(np.linalg.norm(ref), 1e-300))


def write_gguf(path, metadata: dict, tensors: list, alignment: int = 32, version: int = 3):
    """Minimal GGUF writer for tests (the reference ships none): metadata values are (type_code, value) pairs
    with type codes of gguf_types.hpp:56-70; tensors are (name, dims_innermost_first, ggml_type, bytes)."""
    import struct

    def s(b):
        b = b.encode() if isinstance(b, str) else b
        return struct.pack("<Q", len(b)) + b
    fmt = {0: "B", 1: "b", 2: "H", 3: "h", 4: "I", 5: "i", 6: "f", 7: "?", 10: "Q", 11: "q", 12: "d"}

    def val(t, v):
        if t in fmt:
            return struct.pack("<" + fmt[t], v)
        if t == 8:
            return s(v)
        et, items = v   # array: (element type, list)
        return struct.pack("<IQ", et, len(items)) + b"".join(val(et, x) for x in items)
    out = struct.pack("<IIQQ", 0x46554747, version, len(tensors), len(metadata))
    for k, (t, v) in metadata.items():
        out += s(k) + struct.pack("<I", t) + val(t, v)
    offset, blobs = 0, []
    for name, dims, gt, data in tensors:
        data = bytes(data)
        out += s(name) + struct.pack("<I", len(dims)) + b"".join(struct.pack("<Q", d) for d in dims)
        out += struct.pack("<IQ", gt, offset)
        blobs.append((offset, data))
        offset = (offset + len(data) + alignment - 1) // alignment * alignment
    pad = (len(out) + alignment - 1) // alignment * alignment - len(out)
    out += b"\0" * pad
    body = bytearray(offset)
    for off, data in blobs:
        body[off:off + len(data)] = data
    with open(path, "wb") as f:
        f.write(out + bytes(body))
