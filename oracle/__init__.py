"""ctypes/numpy front end of the CPU oracle -- TEST INFRASTRUCTURE ONLY.

Loads ``oracle/liboracle.so`` (the C restatement in ``cut_oracle.c``) and, when
it has been built, ``oracle/_ref/libcut_ref.so`` (the reference's own GGUF
reader behind ``ref_driver.cpp``).  Only tests, the smoke check and the bench's
``cpu_baseline`` leg may import this package; the product never does.
"""
from __future__ import annotations

import ctypes as C
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "liboracle.so")
_REF_PATH = os.path.join(_HERE, "_ref", "libcut_ref.so")

Q8_0, Q4_0, Q4_K, Q6_K = 0, 1, 2, 3
FORMATS = {"Q8_0": Q8_0, "Q4_0": Q4_0, "Q4_K": Q4_K, "Q6_K": Q6_K}
BLOCK_ELEMS = {Q8_0: 32, Q4_0: 32, Q4_K: 256, Q6_K: 256}
BLOCK_BYTES = {Q8_0: 34, Q4_0: 18, Q4_K: 144, Q6_K: 210}
GGML_TYPE = {Q4_0: 2, Q8_0: 8, Q4_K: 12, Q6_K: 14}  # gguf_types.hpp:16-53


def build(force: bool = False) -> None:
    """Compile liboracle.so (and _ref when the reference tree is mounted)."""
    args = ["make", "-C", _HERE] + (["-B"] if force else [])
    subprocess.check_call(args + ["all"], stdout=subprocess.DEVNULL)
    if os.path.isdir("/root/reference/interface/loader/gguf"):
        subprocess.check_call(args + ["ref"], stdout=subprocess.DEVNULL)


def embedding_col(indices, matrix, scales, emb_dim: int, fmt: int) -> np.ndarray:
    """EmbeddingCol: matrix [emb_dim, vocab] column-wise (fmt 0: fp16 bits as uint16; fmt 1: int8 with fp16 scales
    [emb_dim / 32, vocab]); returns fp32 [len(indices), emb_dim]."""
    idx = _c(indices, np.uint32).reshape(-1)
    m = _c(matrix, np.uint16 if fmt == 0 else np.int8)
    sc = _c(scales, np.uint16) if fmt == 1 else np.zeros((1, 1), np.uint16)
    out = np.empty((idx.size, emb_dim), np.float32)
    _lib.orc_embedding_col(_p(idx), _p(m), _p(sc), idx.size, emb_dim, m.shape[1], sc.shape[1], emb_dim, fmt, _p(out))
    return out


def repetition_penalty(logits, factors) -> np.ndarray:
    lg, f = _c(logits, np.float32).reshape(-1), _c(factors, np.float32).reshape(-1)
    out = np.empty_like(lg)
    _lib.orc_repetition_penalty(_p(lg), _p(f), lg.size, _p(out))
    return out


def penalty_factors(recent, penalty: float, vocab: int) -> np.ndarray:
    r = _c(recent, np.int32).reshape(-1)
    out = np.empty(vocab, np.float32)
    _lib.orc_penalty_factors(_p(r), r.size, penalty, vocab, _p(out))
    return out


def _load():
    if not os.path.exists(_LIB_PATH):
        build()
    lib = C.CDLL(_LIB_PATH)
    u8p, f32p, u16p, i8p, f64p = (C.c_void_p,) * 5
    sz, u32 = C.c_size_t, C.c_uint32
    sig = {
        "orc_f16_to_f32": (C.c_float, [C.c_uint16]),
        "orc_f32_to_f16": (C.c_uint16, [C.c_float]),
        "orc_runner_f16_to_f32": (C.c_float, [C.c_uint16]),
        "orc_harness_f32_to_f16": (C.c_uint16, [C.c_float]),
        "orc_f16_to_f32_array": (None, [u16p, sz, f32p]),
        "orc_f32_to_f16_array": (None, [f32p, sz, u16p]),
        "orc_runner_f16_to_f32_array": (None, [u16p, sz, f32p]),
        "orc_get_scale_min_k4": (None, [C.c_int, u8p, u8p, u8p]),
        "orc_dequant": (C.c_int, [C.c_int, u8p, f32p, sz]),
        "orc_dequant_f16": (C.c_int, [C.c_int, u8p, u16p, sz]),
        "orc_quantize_rows_q8_0": (None, [f32p, sz, i8p, u16p]),
        "orc_pack_q8_0": (None, [i8p, u16p, sz, u8p]),
        "orc_split_q8_0": (None, [u8p, u32, u32, i8p, u16p]),
        "orc_split_q4_0": (None, [u8p, u32, u32, u8p, u16p]),
        "orc_requantize_q4k_to_affine": (C.c_int, [u8p, sz, u32, u32, u8p, u16p]),
        "orc_decode_affine_q4": (None, [u8p, u16p, u32, u32, f32p]),
        "orc_transpose_q4_nibble": (None, [u8p, u32, u32, u8p]),
        "orc_matmul_sep_q8_f32": (None, [f32p, i8p, f32p, u32, u32, u32, f32p]),
        "orc_matmul_sep_q4_f32": (None, [f32p, u8p, f32p, u32, u32, u32, C.c_int, f32p]),
        "orc_matmul_sep_q8_f64": (None, [f32p, i8p, f32p, u32, u32, u32, f32p]),
        "orc_matmul_gguf_f32": (C.c_int, [C.c_int, u8p, f32p, u32, u32, u32, f32p]),
        "orc_matmul_gguf_f64": (C.c_int, [C.c_int, u8p, f32p, u32, u32, u32, f64p]),
        "orc_matmul_dense_f32": (None, [f32p, f32p, u32, u32, u32, f32p]),
        "orc_quantize_act_q8": (None, [f32p, sz, i8p, f32p]),
        "orc_matmul_q8_i8": (C.c_int, [u8p, f32p, u32, u32, u32, f32p, f64p]),
        "orc_quantize": (C.c_int, [C.c_int, f32p, sz, u8p]),
        "orc_rmsnorm": (None, [f32p, f32p, u32, u32, C.c_float, f32p]),
        "orc_rope_kv_write": (None, [f32p, f32p, f32p, u32, f32p, f32p, u32, u32, u32, u32, f32p, u16p, u16p]),
        "orc_attention_decode": (None, [f32p, u16p, u16p, u32, u32, u32, u32, u32, C.c_float, f32p]),
        "orc_silu_mul": (None, [f32p, u32, f32p]),
        "orc_embedding_col": (None, [u8p, u8p, u16p, u32, u32, u32, u32, u32, C.c_int, f32p]),
        "orc_repetition_penalty": (None, [f32p, f32p, u32, f32p]),
        "orc_penalty_factors": (None, [u8p, u32, C.c_float, u32, f32p]),
    }
    for name, (res, args) in sig.items():
        fn = getattr(lib, name)
        fn.restype, fn.argtypes = res, args
    return lib


_lib = _load()


def _p(a: np.ndarray):
    return a.ctypes.data_as(C.c_void_p)


def _c(a, dtype):
    return np.ascontiguousarray(a, dtype=dtype)


# ---- scalars / element-wise ------------------------------------------------

def f16_to_f32(h: int) -> float:
    return _lib.orc_f16_to_f32(int(h))


def f32_to_f16(v: float) -> int:
    return _lib.orc_f32_to_f16(float(np.float32(v)))


def f32_to_f16_bits(v: float) -> int:
    """f32_to_f16 on an exact fp32 bit pattern carried in a Python float."""
    return _lib.orc_f32_to_f16(v)


def f16_to_f32_array(h, runner: bool = False) -> np.ndarray:
    h = _c(h, np.uint16).reshape(-1)
    out = np.empty(h.size, np.float32)
    fn = _lib.orc_runner_f16_to_f32_array if runner else _lib.orc_f16_to_f32_array
    fn(_p(h), h.size, _p(out))
    return out


def f32_to_f16_array(v) -> np.ndarray:
    v = _c(v, np.float32).reshape(-1)
    out = np.empty(v.size, np.uint16)
    _lib.orc_f32_to_f16_array(_p(v), v.size, _p(out))
    return out


def runner_f16_to_f32(h: int) -> float:
    return _lib.orc_runner_f16_to_f32(int(h))


def harness_f32_to_f16(v: float) -> int:
    return _lib.orc_harness_f32_to_f16(float(np.float32(v)))


def get_scale_min_k4(j: int, q12) -> tuple[int, int]:
    q = _c(q12, np.uint8)
    sc, m = C.c_uint8(), C.c_uint8()
    _lib.orc_get_scale_min_k4(j, _p(q), C.byref(sc), C.byref(m))
    return sc.value, m.value


# ---- block formats ---------------------------------------------------------

def n_bytes(fmt: int, n_elems: int) -> int:
    assert n_elems % BLOCK_ELEMS[fmt] == 0
    return n_elems // BLOCK_ELEMS[fmt] * BLOCK_BYTES[fmt]


def dequant(fmt: int, blocks, n_elems: int) -> np.ndarray:
    b = _c(blocks, np.uint8).reshape(-1)
    assert n_elems % BLOCK_ELEMS[fmt] == 0 and b.size >= n_bytes(fmt, n_elems)
    out = np.empty(n_elems, np.float32)
    rc = _lib.orc_dequant(fmt, _p(b), _p(out), n_elems)
    assert rc == 0
    return out


def dequant_f16(fmt: int, blocks, n_elems: int) -> np.ndarray:
    """fp16 BITS (uint16) after the reference's host narrowing."""
    b = _c(blocks, np.uint8).reshape(-1)
    assert n_elems % BLOCK_ELEMS[fmt] == 0 and b.size >= n_bytes(fmt, n_elems)
    out = np.empty(n_elems, np.uint16)
    rc = _lib.orc_dequant_f16(fmt, _p(b), _p(out), n_elems)
    assert rc == 0
    return out


def quantize(fmt: int, x) -> np.ndarray:
    x = _c(x, np.float32).reshape(-1)
    out = np.empty(n_bytes(fmt, x.size), np.uint8)
    rc = _lib.orc_quantize(fmt, _p(x), x.size, _p(out))
    assert rc == 0
    return out


def quantize_rows_q8_0(x):
    x = _c(x, np.float32).reshape(-1)
    assert x.size % 32 == 0
    v = np.empty(x.size, np.int8)
    s = np.empty(x.size // 32, np.uint16)
    _lib.orc_quantize_rows_q8_0(_p(x), x.size, _p(v), _p(s))
    return v, s


def split_q8_0(blocks, rows: int, cols: int):
    b = _c(blocks, np.uint8).reshape(-1)
    v = np.empty((rows, cols), np.int8)
    s = np.empty((rows, cols // 32), np.uint16)
    _lib.orc_split_q8_0(_p(b), rows, cols, _p(v), _p(s))
    return v, s


def split_q4_0(blocks, rows: int, cols: int):
    b = _c(blocks, np.uint8).reshape(-1)
    v = np.empty((rows, cols // 2), np.uint8)
    s = np.empty((rows, cols // 32), np.uint16)
    _lib.orc_split_q4_0(_p(b), rows, cols, _p(v), _p(s))
    return v, s


def requantize_q4k_to_affine(raw, N: int, K: int):
    b = _c(raw, np.uint8).reshape(-1)
    packed = np.empty((K, N // 2), np.uint8)
    scales = np.empty((2 * (K // 32), N), np.uint16)
    ok = _lib.orc_requantize_q4k_to_affine(_p(b), b.size, N, K, _p(packed), _p(scales))
    return (packed, scales) if ok else None


def decode_affine_q4(packed, scales, N: int, K: int) -> np.ndarray:
    p, s = _c(packed, np.uint8), _c(scales, np.uint16)
    out = np.empty((N, K), np.float32)
    _lib.orc_decode_affine_q4(_p(p), _p(s), N, K, _p(out))
    return out


def transpose_q4_nibble(packed, N: int, K: int) -> np.ndarray:
    p = _c(packed, np.uint8)
    out = np.empty((K, N // 2), np.uint8)
    _lib.orc_transpose_q4_nibble(_p(p), N, K, _p(out))
    return out


# ---- matmul references -----------------------------------------------------

def matmul_sep_q8(A, B, S, f64: bool = False) -> np.ndarray:
    A, B, S = _c(A, np.float32), _c(B, np.int8), _c(S, np.float32)
    M, K = A.reshape(-1, A.shape[-1]).shape
    N = B.shape[1]
    out = np.empty((M, N), np.float32)
    fn = _lib.orc_matmul_sep_q8_f64 if f64 else _lib.orc_matmul_sep_q8_f32
    fn(_p(A), _p(B), _p(S), M, K, N, _p(out))
    return out


def matmul_sep_q4(A, Bp, S, affine: bool = False) -> np.ndarray:
    A, Bp, S = _c(A, np.float32), _c(Bp, np.uint8), _c(S, np.float32)
    M, K = A.reshape(-1, A.shape[-1]).shape
    N = S.shape[1]
    out = np.empty((M, N), np.float32)
    _lib.orc_matmul_sep_q4_f32(_p(A), _p(Bp), _p(S), M, K, N, int(affine), _p(out))
    return out


def matmul_gguf(fmt: int, W, A, N: int, f64: bool = False) -> np.ndarray:
    """A [M,K] times dequant(W)[N,K] transposed; fp32 sequential or double."""
    W, A = _c(W, np.uint8).reshape(-1), _c(A, np.float32)
    A2 = A.reshape(-1, A.shape[-1])
    M, K = A2.shape
    assert W.size >= N * n_bytes(fmt, K)
    if f64:
        out = np.empty((M, N), np.float64)
        rc = _lib.orc_matmul_gguf_f64(fmt, _p(W), _p(A2), M, K, N, _p(out))
    else:
        out = np.empty((M, N), np.float32)
        rc = _lib.orc_matmul_gguf_f32(fmt, _p(W), _p(A2), M, K, N, _p(out))
    assert rc == 0
    return out


def quantize_act_q8(a):
    a = _c(a, np.float32).reshape(-1)
    q = np.empty(a.size, np.int8)
    s = np.empty(a.size // 32, np.float32)
    _lib.orc_quantize_act_q8(_p(a), a.size, _p(q), _p(s))
    return q, s


def matmul_q8_i8(W, A, N: int, f64: bool = False) -> np.ndarray:
    """The reference's int8-activation arithmetic (MatMulQ8GemvDot.cu:60-85) on Q8_0 blocks W [N][K/32]."""
    A = _c(A, np.float32)
    A = A.reshape(1, -1) if A.ndim == 1 else A
    M, K = A.shape
    W = _c(W, np.uint8).reshape(-1)
    assert W.size == N * (K // 32) * 34
    c32 = np.empty((M, N), np.float32)
    c64 = np.empty((M, N), np.float64)
    rc = _lib.orc_matmul_q8_i8(_p(W), _p(A), M, K, N, _p(c32), _p(c64))
    assert rc == 0
    return c64 if f64 else c32


# ---- the reference's own reader (only where oracle/_ref was built) ----------

def rmsnorm(x, weight, eps: float) -> np.ndarray:
    x = _c(x, np.float32)
    x2 = x.reshape(-1, x.shape[-1])
    w = _c(weight, np.float32)
    out = np.empty_like(x2)
    _lib.orc_rmsnorm(_p(x2), _p(w), x2.shape[0], x2.shape[1], eps, _p(out))
    return out.reshape(x.shape)


def rope_kv_write(q, k, v, pos: int, cos_t, sin_t, head_dim: int, k_cache, v_cache) -> np.ndarray:
    """Rotates q (returned) and k; writes k, v into row `pos` of the uint16 (fp16 bits) caches in place."""
    q, k, v = _c(q, np.float32).reshape(-1), _c(k, np.float32).reshape(-1), _c(v, np.float32).reshape(-1)
    cos_t, sin_t = _c(cos_t, np.float32), _c(sin_t, np.float32)
    assert k_cache.dtype == np.uint16 and v_cache.dtype == np.uint16 and k_cache.flags.c_contiguous
    q_out = np.empty_like(q)
    _lib.orc_rope_kv_write(_p(q), _p(k), _p(v), pos, _p(cos_t), _p(sin_t), q.size, k.size, head_dim,
                           k_cache.shape[1], _p(q_out), _p(k_cache), _p(v_cache))
    return q_out


def attention_decode(q, k_cache, v_cache, seq_len: int, n_heads: int, n_kv_heads: int, head_dim: int,
                     scale: float) -> np.ndarray:
    q = _c(q, np.float32).reshape(-1)
    assert k_cache.dtype == np.uint16 and v_cache.dtype == np.uint16
    out = np.empty(n_heads * head_dim, np.float32)
    _lib.orc_attention_decode(_p(q), _p(k_cache), _p(v_cache), seq_len, n_heads, n_kv_heads, head_dim,
                              k_cache.shape[1], scale, _p(out))
    return out


def silu_mul(gate_up) -> np.ndarray:
    g = _c(gate_up, np.float32).reshape(-1)
    out = np.empty(g.size // 2, np.float32)
    _lib.orc_silu_mul(_p(g), g.size // 2, _p(out))
    return out


def have_ref() -> bool:
    return os.path.exists(_REF_PATH)


_ref = None


def _load_ref():
    global _ref
    if _ref is None:
        _ref = C.CDLL(_REF_PATH)
        _ref.ref_dequant.restype = C.c_int
        _ref.ref_dequant.argtypes = [C.c_uint32, C.c_void_p, C.c_size_t,
                                     C.c_uint64, C.c_uint64, C.c_void_p]
        for fn in (_ref.ref_split_q8, _ref.ref_split_q4):
            fn.restype = C.c_int
            fn.argtypes = [C.c_void_p, C.c_size_t, C.c_uint64, C.c_uint64,
                           C.c_void_p, C.c_void_p]
    return _ref


def ref_dequant(fmt: int, blocks, rows: int, cols: int) -> np.ndarray:
    b = _c(blocks, np.uint8).reshape(-1)
    out = np.empty(rows * cols, np.float32)
    rc = _load_ref().ref_dequant(GGML_TYPE[fmt], _p(b), b.size, rows, cols, _p(out))
    assert rc == 0, rc
    return out


def ref_split_q8(blocks, rows: int, cols: int):
    b = _c(blocks, np.uint8).reshape(-1)
    v = np.empty((rows, cols), np.int8)
    s = np.empty((rows, cols // 32), np.uint16)
    assert _load_ref().ref_split_q8(_p(b), b.size, rows, cols, _p(v), _p(s)) == 0
    return v, s


def ref_split_q4(blocks, rows: int, cols: int):
    b = _c(blocks, np.uint8).reshape(-1)
    v = np.empty((rows, cols // 2), np.uint8)
    s = np.empty((rows, cols // 32), np.uint16)
    assert _load_ref().ref_split_q4(_p(b), b.size, rows, cols, _p(v), _p(s)) == 0
    return v, s
