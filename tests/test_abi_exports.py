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


def test_missing_library_fails_loudly(monkeypatch):
    monkeypatch.setattr(L, "_lib", None)
    monkeypatch.setattr(L, "LIB_PATH", "/nonexistent/libcut_hip.so")
    with pytest.raises(L.CutHipError):
        L.load()
