"""GPU parity: block dequantization through the C ABI, bit-exact against the
CPU oracle and the committed golden vectors of the reference reader."""
import numpy as np
import pytest

import oracle
from helpers import finite_random_blocks, quantized_weights

torch = pytest.importorskip("torch")
pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def ops():
    from cut_amd import lib, ops as _ops
    lib.check(lib.load().cuthip_init(0))
    return _ops


def run(ops, fmt, blocks, rows, cols, dtype, stride=None):
    raw = torch.from_numpy(np.ascontiguousarray(blocks)).cuda()
    if stride is None:
        out = ops.dequantize(raw, fmt, rows, cols, dtype)
    else:
        buf = torch.full((rows, stride), -1.0, dtype=dtype, device="cuda")
        out = ops.dequantize(raw, fmt, rows, cols, dtype, out=buf[:, :cols])
        assert torch.all(buf[:, cols:] == -1.0)  # padding untouched
    torch.cuda.synchronize()
    return out.cpu().numpy()


def check(fmt, got, blocks, n, dtype):
    if dtype == torch.float32:
        want = oracle.dequant(fmt, blocks, n)
        assert np.array_equal(got.reshape(-1).view(np.uint32), want.view(np.uint32))
    else:
        want = oracle.dequant_f16(fmt, blocks, n)
        assert np.array_equal(got.reshape(-1).view(np.uint16), want)


@pytest.mark.parametrize("name", list(oracle.FORMATS))
@pytest.mark.parametrize("dtype", ["float32", "float16"])
def test_golden_vectors(ops, golden, name, dtype):
    fmt = oracle.FORMATS[name]
    dt = getattr(torch, dtype)
    rows, cols = int(golden["rows"]), int(golden["cols"])
    for tag in ("random", "gauss"):
        blocks = golden[f"{name}_{tag}_blocks"]
        got = run(ops, fmt, blocks, rows, cols, dt)
        if dt == torch.float32:
            assert np.array_equal(got.reshape(-1).view(np.uint32), golden[f"{name}_{tag}_f32bits"])
        else:
            check(fmt, got, blocks, rows * cols, dt)


@pytest.mark.parametrize("name", list(oracle.FORMATS))
@pytest.mark.parametrize("dtype", ["float32", "float16"])
def test_random_bytes_bit_exact(ops, name, dtype):
    """Uniformly random block bytes (finite scales): every bit pattern class,
    including subnormal scales, signed zeros and fp16 ties."""
    fmt = oracle.FORMATS[name]
    dt = getattr(torch, dtype)
    rows, cols = 37, 2048
    blocks = finite_random_blocks(fmt, rows * cols // oracle.BLOCK_ELEMS[fmt], seed=100 + fmt)
    got = run(ops, fmt, blocks, rows, cols, dt)
    check(fmt, got, blocks, rows * cols, dt)


@pytest.mark.parametrize("name", list(oracle.FORMATS))
def test_gaussian_weights_and_small_scales(ops, name):
    """N(0, 0.02) weights through the quantizer, plus a copy scaled into the
    fp16-subnormal output range (exercises the tie and subnormal rounding)."""
    fmt = oracle.FORMATS[name]
    rows, cols = 16, 4096
    for scale in (1.0, 2.0 ** -9):
        w = np.random.default_rng(5).standard_normal(rows * cols).astype(np.float32) * np.float32(0.02 * scale)
        blocks = oracle.quantize(fmt, w)
        for dt in (torch.float32, torch.float16):
            got = run(ops, fmt, blocks, rows, cols, dt)
            check(fmt, got, blocks, rows * cols, dt)


@pytest.mark.parametrize("name,rows,cols,stride", [("Q8_0", 5, 96, 100), ("Q4_0", 3, 32, 36), ("Q4_K", 4, 256, 264),
                                                   ("Q6_K", 2, 512, 520), ("Q8_0", 1, 32, 32), ("Q6_K", 1, 256, 256)])
def test_ragged_shapes_and_strides(ops, name, rows, cols, stride):
    fmt = oracle.FORMATS[name]
    blocks = finite_random_blocks(fmt, rows * cols // oracle.BLOCK_ELEMS[fmt], seed=7)
    for dt in (torch.float32, torch.float16):
        got = run(ops, fmt, blocks, rows, cols, dt, stride=stride)
        check(fmt, np.ascontiguousarray(got), blocks, rows * cols, dt)


def test_reference_fixtures(ops):
    # dequant/q4k and dequant/q6k of the reference harness (OpRegistry.h:1929-1978)
    blk = np.zeros(144, np.uint8)
    blk[0:2] = np.array([0x3C00], np.uint16).view(np.uint8)
    blk[4:8] = 1
    blk[12:16] = 1
    qs = np.array([(i % 8) | ((i % 8 + 1) << 4) for i in range(128)], np.uint8)
    blk[16:] = qs
    out = run(ops, oracle.Q4_K, blk, 1, 256, torch.float32).reshape(-1)
    assert np.all(np.isfinite(out)) and np.array_equal(out[:32], (qs[:32] & 15).astype(np.float32))
    blk = np.zeros(210, np.uint8)
    blk[0:128] = 0x55
    blk[192:208] = 1
    blk[208:210] = np.array([0x3C00], np.uint16).view(np.uint8)
    out = run(ops, oracle.Q6_K, blk, 1, 256, torch.float32).reshape(-1)
    assert np.array_equal(out, np.full(256, -27.0, np.float32))


def test_nonfinite_scales_keep_their_class(ops):
    """Inf/NaN block scales never occur in GGUF files; outputs must still be
    NaN where the reference's are NaN and +-Inf where it gives +-Inf (NaN
    payload and sign are host-FPU specific and not compared)."""
    for name, fmt in oracle.FORMATS.items():
        rng = np.random.default_rng(3)
        n = 256 * 8
        blocks = rng.integers(0, 256, oracle.n_bytes(fmt, n), dtype=np.uint8)
        got = run(ops, fmt, blocks, 1, n, torch.float32).reshape(-1)
        want = oracle.dequant(fmt, blocks, n)
        assert np.array_equal(np.isnan(got), np.isnan(want)), name
        fin = ~np.isnan(want)
        assert np.array_equal(got[fin].view(np.uint32), want[fin].view(np.uint32)), name


@pytest.mark.parametrize("name", list(oracle.FORMATS))
def test_full_size_properties(ops, name):
    """256 Mi elements (BASELINE config 2) -> fp16, every format: tiled weights, so every
    repeat of the tile must dequantize to the same bits as the first, which is
    checked against the oracle; plus a checksum over the whole output."""
    fmt = oracle.FORMATS[name]
    tile_rows, cols, reps = 1024, 4096, 64  # 64 x 4 Mi = 256 Mi elements
    tile = quantized_weights(fmt, tile_rows, cols, seed=0)
    raw = torch.from_numpy(tile).cuda().repeat(reps)
    out = ops.dequantize(raw, fmt, tile_rows * reps, cols, torch.float16)
    torch.cuda.synchronize()
    first = out[:tile_rows].cpu().numpy()
    want = oracle.dequant_f16(fmt, tile, tile_rows * cols)
    assert np.array_equal(first.reshape(-1).view(np.uint16), want)
    v = out.view(torch.int16).view(reps, -1)
    assert torch.equal(v, v[0:1].expand_as(v))
