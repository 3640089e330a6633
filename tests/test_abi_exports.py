"""CPU checks of the C-ABI library: it loads, exports every symbol that
include/cut_hip.h declares, and its host-only entry points behave (variant
tables, argument validation).  No compute call is made here."""
import ctypes as C
import os
import re

import pytest

from cut_amd import lib as L

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def declared_symbols():
    text = open(os.path.join(ROOT, "include", "cut_hip.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(cuthip_[a-z0-9_]+)\s*\(", text)))


def test_header_and_binding_agree():
    assert declared_symbols() == sorted(L.EXPORTS)


def test_library_exports_every_declared_symbol():
    lib = L.load()
    for name in declared_symbols():
        assert hasattr(lib, name), name


def test_variant_tables():
    v = L.variants(L.OP_MATMUL_GGUF)
    assert [x["name"] for x in v][:2] == ["MatMulGgufGemvMfma", "MatMulGgufSkinnyMfma"]
    assert all(x["effTileN"] == 32 for x in v[:2])
    lib = L.load()
    assert lib.cuthip_variant_lookup(L.OP_MATMUL_GGUF, b"MatMulGgufGemvMfma") == 0
    # unknown names are hard errors, never a skipped dispatch
    assert lib.cuthip_variant_lookup(L.OP_MATMUL_GGUF, b"NoSuchKernel") == -4
    assert b"NoSuchKernel" in lib.cuthip_last_error()
    assert L.variants(L.OP_DEQUANT)[0]["name"] == "DequantGguf8"


# The reference's tables (operators/impl/matmul/MatMulQ8Variants.generated.h:20-32, MatMulQ4Variants.generated.h:20-29):
# name, wgX, wgY, effTileM, effTileN at each index, and the defaults kMatMulQ8DefaultVariant / kMatMulQ4DefaultVariant.
REF_Q8 = [("MatMulQ8T16R4x4", 16, 16, 64, 64), ("MatMulQ8Gemv", 256, 1, 1, 256), ("MatMulQ8VecT16R4x4", 16, 16, 64, 64),
          ("MatMulQ8GemvKPar", 32, 1, 1, 4), ("MatMulQ8GemvKPar8", 32, 8, 1, 8), ("MatMulQ8GemvDot", 32, 1, 1, 4),
          ("MatMulQ8TiledDot", 256, 1, 32, 64), ("MatMulQ8CoopMatTiled", 128, 1, 32, 32)]
REF_Q4 = [("MatMulQ4T16R4x4", 16, 16, 64, 64), ("MatMulQ4Gemv", 256, 1, 1, 256), ("MatMulQ4GemvKPar", 32, 1, 1, 4),
          ("MatMulQ4GemvKPar8", 32, 8, 1, 8), ("MatMulQ4CoopMatTiled", 128, 1, 32, 32)]


@pytest.mark.parametrize("op,ref,default", [(L.OP_MATMUL_Q8, REF_Q8, 2), (L.OP_MATMUL_Q4, REF_Q4, 0)])
def test_separated_layout_tables_hold_the_reference_names_at_the_reference_indices(op, ref, default):
    lib = L.load()
    v = L.variants(op)
    assert [(x["name"], x["wgX"], x["wgY"], x["effTileM"], x["effTileN"]) for x in v] == ref
    assert lib.cuthip_variant_count(op) == len(ref)
    assert lib.cuthip_variant_default(op) == default
    for i, row in enumerate(ref):
        assert lib.cuthip_variant_lookup(op, row[0].encode()) == i
        assert lib.cuthip_variant_available(op, i) == 1
    assert lib.cuthip_variant_available(op, len(ref)) == -4


def test_separated_layout_entry_points_take_the_variant_index():
    """Unknown indices are refused before anything touches the GPU (no device is needed to see that)."""
    lib = L.load()
    one = C.c_void_p(256)
    common = (one, one, one, None, one, 1, 64, 4, 64, 4, 4, 4, 0, 0)
    assert lib.cuthip_matmul_q8_sep(*common, 8, None, 0, None) == -4
    assert b"unknown variant index 8" in lib.cuthip_last_error()
    assert lib.cuthip_matmul_q8_sep(*common, -2, None, 0, None) == -4
    assert lib.cuthip_matmul_q4_sep(*common, 0, 5, None, 0, None) == -4
    # the cooperative-matrix indices need K a multiple of 128 and a workspace: refused with a message, not skipped
    assert lib.cuthip_matmul_q8_sep(*common, 7, None, 0, None) == -1
    assert b"multiple of 128" in lib.cuthip_last_error()
    assert lib.cuthip_matmul_q4_sep(*common, 0, 4, None, 0, None) == -1
    # sizing follows the route of the index: a GEMV index never asks for the fp16 copy of the weights
    small = lib.cuthip_matmul_sep_workspace_bytes_for(L.OP_MATMUL_Q8, 4, 32, 4096, 4096)
    big = lib.cuthip_matmul_sep_workspace_bytes_for(L.OP_MATMUL_Q8, 7, 32, 4096, 4096)
    auto = lib.cuthip_matmul_sep_workspace_bytes_for(L.OP_MATMUL_Q8, -1, 32, 4096, 4096)
    assert big >= 4096 * 4096 * 2 > small and auto == lib.cuthip_matmul_sep_workspace_bytes(32, 4096, 4096) == big
    assert lib.cuthip_matmul_sep_workspace_bytes_for(L.OP_MATMUL_Q4, 4, 1, 4096, 4096) >= 4096 * 4096 * 2


def test_batched_gemv_workspace_covers_the_k_ranges_its_lds_budget_forces():
    """Host logic of the workspace sizing for 2..8 batch rows (no device needed): the K split of the 8-row GEMV takes
    enough ranges for one workgroup of eight waves per CU, and beyond that as many as it needs for the activations of
    one range (8 batch rows x 576 + 32 bytes per 256 elements; 640 for Q6_K) to fit 96 KB of LDS; the workspace holds
    one fp32 [M, N] per range.  Ranges are a power of two."""
    lib = L.load()
    Q4_K, Q6_K = L.FORMATS["Q4_K"], L.FORMATS["Q6_K"]

    def ranges(fmt, M, K, N):
        b = lib.cuthip_matmul_gguf_workspace_bytes(fmt, M, K, N, L.F16)
        assert b % (M * N * 4) == 0
        return b // (M * N * 4)
    # few weight rows: the occupancy rule alone (16 ranges at most from it), 4096 x 14336 at batch 8: 4 ranges of 14 steps
    assert ranges(Q4_K, 8, 14336, 4096) == 4
    # many weight rows on K = 8192: the chip is full without a split, but 8 rows x 32 steps x 608 B = 152 KB: 2 ranges
    assert ranges(Q4_K, 8, 8192, 28672) == 2
    assert ranges(Q6_K, 8, 8192, 28672) == 2
    # 4 rows of K = 8192 fit (76 / 80 KB): no K split is preferred for that many weight rows, the workspace is the
    # prefill one (fp16 copy of the weights) as for any other shape
    assert lib.cuthip_matmul_gguf_workspace_bytes(Q4_K, 4, 8192, 28672, L.F16) >= 28672 * 8192 * 2
    # very long rows on few weight rows: 16 ranges from the occupancy rule leave 22 steps each, 8 x 22 x 608 B = 107 KB:
    # doubled once more
    assert ranges(Q4_K, 8, 90112, 16) == 32
    # two rows of K = 28672 (2 x 112 x 608 B = 136 KB)
    assert ranges(Q4_K, 2, 28672, 8192) >= 2


def test_default_variant_of_the_gguf_table_is_valid_for_every_m():
    lib = L.load()
    assert lib.cuthip_variant_default(L.OP_MATMUL_GGUF) == 0
    assert lib.cuthip_variant_default(77) == -1
    assert lib.cuthip_variant_available(L.OP_MATMUL_GGUF, 4) == 1
    assert lib.cuthip_variant_available(L.OP_MATMUL_GGUF, 5) in (0, 1)


def test_fusion_operator_codes_are_the_reference_codes():
    """OP_UNARY_* / OP_BINARY_* of operators/runtime/ComputeOpsShared.h:22-40, 118-167 for the operators that
    cut_writeOutput implements (MatMulQ8Common.cuh:58-109)."""
    assert L.UNARY == {"neg": 100, "abs": 101, "sqrt": 102, "square": 103, "reciprocal": 104, "exp": 106, "log": 109,
                       "tanh": 121, "floor": 122, "ceil": 123, "round": 124, "relu": 130, "sigmoid": 131, "gelu": 132,
                       "gelu_tanh": 132, "silu": 133, "softplus": 134, "relu6": 137, "mish": 141, "hardswish": 142,
                       "hardsigmoid": 143, "rsqrt": 148}
    assert L.BINARY == {"add": 0, "sub": 1, "mul": 2, "div": 3, "mod": 4, "pow": 5, "floor_div": 6, "min": 13, "max": 14}
    lib = L.load()
    assert sum(lib.cuthip_epilogue_op_supported(L.EPI_UNARY, c) for c in range(0, 200)) == 21
    assert sum(lib.cuthip_epilogue_op_supported(L.EPI_BINARY, c) for c in range(0, 200)) == 9
    header = open(os.path.join(ROOT, "include", "cut_hip.h")).read()
    for name, code in list(L.UNARY.items()) + list(L.BINARY.items()):
        kind = "UNARY" if name in L.UNARY and code >= 100 else "BINARY"
        assert re.search(rf"CUTHIP_{kind}_{name.upper()} = {code}\b", header), (name, code)


def test_argument_validation_without_a_device():
    lib = L.load()
    one = C.c_void_p(16)
    # bad format / dtype / shapes are refused before anything touches the GPU
    assert lib.cuthip_dequant(9, one, one, L.F32, 1, 256, 256, None) == -1
    assert lib.cuthip_dequant(L.Q4_K, one, one, L.F32, 1, 100, 100, None) == -1
    assert b"multiple of the block size" in lib.cuthip_last_error()
    assert lib.cuthip_dequant(L.Q4_K, one, one, 7, 1, 256, 256, None) == -1
    assert lib.cuthip_dequant(L.Q4_K, one, one, L.F32, 1, 256, 128, None) == -1
    assert lib.cuthip_dequant(L.Q4_K, None, one, L.F32, 1, 256, 256, None) == -1
    mm = lib.cuthip_matmul_gguf
    assert mm(L.Q4_K, one, one, L.F32, one, L.F32, 1, 100, 32, 100, 32, 0, 0, None, -1, None) == -1
    assert mm(L.Q4_K, one, one, L.F32, one, L.F32, 1, 256, 32, 128, 32, 0, 0, None, -1, None) == -1
    assert mm(L.Q4_K, one, one, L.F32, one, L.F32, 1, 256, 32, 256, 32, L.EPI_BINARY, 0, None, -1, None) == -1
    assert mm(L.Q4_K, one, one, L.F32, one, L.F32, 1, 256, 32, 256, 32, 0, 0, None, 99, None) == -4
    # empty problems are a no-op
    assert mm(L.Q4_K, one, one, L.F32, one, L.F32, 0, 256, 32, 256, 32, 0, 0, None, -1, None) == 0
    assert lib.cuthip_dequant(L.Q4_K, one, one, L.F32, 0, 256, 256, None) == 0


def test_attention_halves_validate_without_a_device():
    lib = L.load()
    one = C.c_void_p(16)
    assert lib.cuthip_attn_partial_splits(2048) == 8 and lib.cuthip_attn_partial_splits(65) == 2
    assert lib.cuthip_attn_partial_splits(64) == 1 and lib.cuthip_attn_partial_splits(1 << 16) == 8
    assert lib.cuthip_attn_partial_bytes(32, 128, 2048) == 32 * 8 * 130 * 4
    part = lib.cuthip_attn_decode_partial
    # a head dimension the wide-split kernel is not built for; records too small; heads that do not divide
    assert part(one, L.F32, one, one, one, 8, 2, 64, 128, 0.125, 64, one, 1 << 20, None) == -1
    assert b"head_dim" in lib.cuthip_last_error()
    assert part(one, L.F32, one, one, one, 8, 2, 128, 256, 0.1, 2048, one, 100, None) == -1
    assert b"records" in lib.cuthip_last_error()
    assert part(one, L.F32, one, one, one, 8, 3, 128, 384, 0.1, 2048, one, 1 << 20, None) == -1
    assert lib.cuthip_attn_merge(one, 0, 8, 128, one, L.F32, None) == -1
    assert lib.cuthip_attn_merge(one, 8, 8, 136, one, L.F32, None) == -1
    mm = lib.cuthip_matmul_gguf_attn_merge
    assert mm(L.Q4_K, one, one, 9, 8, 128, one, L.F32, 64, 0, 0, None, None, None) == -1    # more than 8 records per head
    assert b"splits" in lib.cuthip_last_error()
    assert mm(L.Q4_K, one, one, 8, 3, 100, one, L.F32, 64, 0, 0, None, None, None) == -1    # K = 300 is no multiple of 256
    assert mm(L.Q4_K, one, one, 8, 8, 128, one, L.F32, 64, L.EPI_BINARY, 0, None, None, None) == -1   # binary epilogue without D
    assert mm(L.Q4_K, one, C.c_void_p(12), 8, 8, 128, one, L.F32, 64, 0, 0, None, None, None) == -1   # records not 8-byte aligned


def test_missing_library_fails_loudly(monkeypatch):
    monkeypatch.setattr(L, "_lib", None)
    monkeypatch.setattr(L, "LIB_PATH", "/nonexistent/libcut_hip.so")
    with pytest.raises(L.CutHipError):
        L.load()
