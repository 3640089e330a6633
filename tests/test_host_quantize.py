"""Host-side numpy encoders (cut_amd.quantize) against the oracle (CPU only)."""
import numpy as np
import pytest

import oracle
from cut_amd import quantize as Q


def test_f16_narrowing_matches_reference_rounding():
    rng = np.random.default_rng(1)
    u = rng.integers(0, 1 << 32, 1 << 18, dtype=np.uint64).astype(np.uint32)
    e = (rng.integers(95, 146, 1 << 18, dtype=np.uint64).astype(np.uint32) << 23)
    ties = e | (rng.integers(0, 1024, 1 << 18, dtype=np.uint64).astype(np.uint32) << 13) | 0x1000
    x = np.concatenate([u, e | (u & 0x7FFFFF), ties, ties | 0x80000000]).view(np.float32)
    assert np.array_equal(Q.f32_to_f16_bits(x), oracle.f32_to_f16_array(x))


def test_q8_0_is_the_reference_quantizer():
    x = (np.random.default_rng(0).standard_normal(32 * 4096).astype(np.float32) * np.float32(0.02))
    x[:32] = 0
    assert np.array_equal(Q.quantize("Q8_0", x), oracle.quantize(oracle.Q8_0, x))


@pytest.mark.parametrize("name,tol", [("Q4_0", 0.12), ("Q4_K", 0.10), ("Q6_K", 0.03), ("Q8_0", 0.01)])
def test_encoders_give_valid_blocks(name, tol):
    fmt = oracle.FORMATS[name]
    x = (np.random.default_rng(2).standard_normal(256 * 512).astype(np.float32) * np.float32(0.02))
    blocks = Q.quantize(name, x)
    assert blocks.size == oracle.n_bytes(fmt, x.size)
    y = oracle.dequant(fmt, blocks, x.size)
    assert np.linalg.norm(y - x) / np.linalg.norm(x) < tol
