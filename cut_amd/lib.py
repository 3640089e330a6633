"""ctypes binding of libcut_hip.so (the C ABI declared in include/cut_hip.h).

The library is built in-tree by ``__graft_entry__.build()`` / ``make -C
cut_amd/csrc``.  There is no CPU fallback: if the shared object is missing or a
call fails, an exception is raised.
"""
from __future__ import annotations

import ctypes as C
import os

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "libcut_hip.so")

Q8_0, Q4_0, Q4_K, Q6_K = 0, 1, 2, 3
F32, F16 = 0, 1
OP_DEQUANT, OP_MATMUL_GGUF, OP_MATMUL_Q8, OP_MATMUL_Q4 = 0, 1, 2, 3
EPI_NONE, EPI_UNARY, EPI_BINARY, EPI_SWIGLU_PAIRS = 0, 1, 2, 3
# epilogue operators: the reference's OP_UNARY_* / OP_BINARY_* codes (operators/runtime/ComputeOpsShared.h), the set of
# cut_writeOutput (operators/impl/matmul/MatMulQ8Common.cuh:58-109)
UNARY = {"neg": 100, "abs": 101, "sqrt": 102, "square": 103, "reciprocal": 104, "exp": 106, "log": 109, "tanh": 121,
         "floor": 122, "ceil": 123, "round": 124, "relu": 130, "sigmoid": 131, "gelu": 132, "gelu_tanh": 132, "silu": 133,
         "softplus": 134, "relu6": 137, "mish": 141, "hardswish": 142, "hardsigmoid": 143, "rsqrt": 148}
BINARY = {"add": 0, "sub": 1, "mul": 2, "div": 3, "mod": 4, "pow": 5, "floor_div": 6, "min": 13, "max": 14}
FORMATS = {"Q8_0": Q8_0, "Q4_0": Q4_0, "Q4_K": Q4_K, "Q6_K": Q6_K}
BLOCK_ELEMS = {Q8_0: 32, Q4_0: 32, Q4_K: 256, Q6_K: 256}
BLOCK_BYTES = {Q8_0: 34, Q4_0: 18, Q4_K: 144, Q6_K: 210}

# every symbol include/cut_hip.h declares
EXPORTS = [
    "cuthip_init", "cuthip_last_error", "cuthip_device_info", "cuthip_set_tuning",
    "cuthip_malloc", "cuthip_free", "cuthip_memcpy_h2d", "cuthip_memcpy_d2h", "cuthip_memcpy_d2d", "cuthip_memset",
    "cuthip_stream_create", "cuthip_stream_destroy", "cuthip_stream_sync",
    "cuthip_event_create", "cuthip_event_destroy", "cuthip_event_record", "cuthip_event_sync", "cuthip_event_elapsed_ms",
    "cuthip_read_probe", "cuthip_debug_fill_lds", "cuthip_epilogue_op_supported",
    "cuthip_graph_begin_capture", "cuthip_graph_end_capture", "cuthip_graph_launch", "cuthip_graph_destroy",
    "cuthip_variant_count", "cuthip_variant_default", "cuthip_variant_available", "cuthip_variant_info", "cuthip_variant_lookup",
    "cuthip_dequant", "cuthip_matmul_gguf", "cuthip_matmul_gguf_pro",
    "cuthip_matmul_gguf_workspace_bytes", "cuthip_matmul_gguf_ws", "cuthip_matmul_gguf_pair", "cuthip_matmul_gguf_carry",
    "cuthip_rmsnorm", "cuthip_rope_kv_write", "cuthip_attn_decode_workspace_bytes", "cuthip_attn_decode",
    "cuthip_attn_decode_static_max_bytes", "cuthip_attn_decode_static",
    "cuthip_attn_partial_splits", "cuthip_attn_partial_bytes", "cuthip_attn_decode_partial", "cuthip_attn_merge",
    "cuthip_matmul_gguf_attn_merge",
    "cuthip_silu_mul", "cuthip_argmax", "cuthip_repetition_penalty", "cuthip_argmax_penalized",
    "cuthip_matmul_gguf_argmax_workspace_bytes", "cuthip_matmul_gguf_argmax", "cuthip_embedding_rows", "cuthip_embedding_col",
    "cuthip_matmul_sep_workspace_bytes", "cuthip_matmul_sep_workspace_bytes_for", "cuthip_matmul_q8_sep", "cuthip_matmul_q4_sep",
    "cuthip_prepare_sep", "cuthip_transpose_q4_nibble", "cuthip_quantize_rows_q8_0",
    "cuthip_matmul_q8_i8_workspace_bytes", "cuthip_matmul_q8_i8",
    "cuthip_matmul_dense_f16_workspace_bytes", "cuthip_matmul_dense_f16",
]


class NormCarry(C.Structure):
    """cuthip_norm_carry_t: device pointers as integers (0 = NULL)."""
    _fields_ = [("sumsq_parts", C.c_void_p), ("eps", C.c_float), ("next_norm_weight", C.c_void_p), ("next_x16", C.c_void_p),
                ("next_sumsq_parts", C.c_void_p)]


class RopeAppend(C.Structure):
    """cuthip_rope_append_t: device pointers as integers."""
    _fields_ = [("runtime_params", C.c_void_p), ("cos_table", C.c_void_p), ("sin_table", C.c_void_p), ("q_out", C.c_void_p),
                ("q_out_dtype", C.c_int), ("k_cache", C.c_void_p), ("v_cache", C.c_void_p), ("q_dim", C.c_uint32),
                ("head_dim", C.c_uint32), ("aligned_kv_dim", C.c_uint32), ("max_positions", C.c_uint32)]


class CutHipError(RuntimeError):
    """A C-ABI call returned non-zero (the reference throws std::runtime_error)."""


class DeviceInfo(C.Structure):
    _fields_ = [("name", C.c_char * 64), ("arch", C.c_char * 32), ("compute_units", C.c_int),
                ("wave_size", C.c_int), ("lds_bytes_per_workgroup", C.c_int), ("clock_khz", C.c_int),
                ("memory_clock_khz", C.c_int), ("memory_bus_bits", C.c_int), ("hbm_bytes", C.c_size_t),
                ("l2_bytes", C.c_size_t)]


class VariantInfo(C.Structure):
    _fields_ = [("name", C.c_char_p), ("wgX", C.c_uint32), ("wgY", C.c_uint32), ("effTileM", C.c_uint32),
                ("effTileN", C.c_uint32), ("description", C.c_char_p)]


_lib = None


def load() -> C.CDLL:
    """Loads the shared object; raises if it has not been built."""
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(LIB_PATH):
        raise CutHipError(f"{LIB_PATH} is missing: build it with `python -c 'import __graft_entry__ as g; g.build()'` "
                          "or `make -C cut_amd/csrc` (there is no CPU fallback)")
    lib = C.CDLL(LIB_PATH)
    vp, u32, i = C.c_void_p, C.c_uint32, C.c_int
    lib.cuthip_last_error.restype = C.c_char_p
    lib.cuthip_last_error.argtypes = []
    lib.cuthip_init.argtypes = [i]
    lib.cuthip_device_info.argtypes = [C.POINTER(DeviceInfo)]
    lib.cuthip_set_tuning.argtypes = [C.c_char_p, C.c_char_p]
    lib.cuthip_malloc.argtypes = [C.POINTER(vp), C.c_size_t]
    lib.cuthip_free.argtypes = [vp]
    for n in ("cuthip_memcpy_h2d", "cuthip_memcpy_d2h", "cuthip_memcpy_d2d"):
        getattr(lib, n).argtypes = [vp, vp, C.c_size_t, vp]
    lib.cuthip_memset.argtypes = [vp, i, C.c_size_t, vp]
    lib.cuthip_stream_create.argtypes = [C.POINTER(vp)]
    lib.cuthip_stream_destroy.argtypes = [vp]
    lib.cuthip_stream_sync.argtypes = [vp]
    lib.cuthip_event_create.argtypes = [C.POINTER(vp)]
    lib.cuthip_event_destroy.argtypes = [vp]
    lib.cuthip_event_record.argtypes = [vp, vp]
    lib.cuthip_event_sync.argtypes = [vp]
    lib.cuthip_event_elapsed_ms.argtypes = [vp, vp, C.POINTER(C.c_float)]
    lib.cuthip_read_probe.argtypes = [vp, C.c_size_t, vp, vp]
    lib.cuthip_debug_fill_lds.argtypes = [C.c_uint32, vp]
    lib.cuthip_epilogue_op_supported.argtypes = [i, i]
    lib.cuthip_graph_begin_capture.argtypes = [vp]
    lib.cuthip_graph_end_capture.argtypes = [vp, C.POINTER(vp)]
    lib.cuthip_graph_launch.argtypes = [vp, vp]
    lib.cuthip_graph_destroy.argtypes = [vp]
    lib.cuthip_variant_count.argtypes = [i]
    lib.cuthip_variant_default.argtypes = [i]
    lib.cuthip_variant_available.argtypes = [i, i]
    lib.cuthip_variant_info.argtypes = [i, i, C.POINTER(VariantInfo)]
    lib.cuthip_variant_lookup.argtypes = [i, C.c_char_p]
    lib.cuthip_dequant.argtypes = [i, vp, vp, i, u32, u32, u32, vp]
    lib.cuthip_matmul_gguf.argtypes = [i, vp, vp, i, vp, i, u32, u32, u32, u32, u32, i, i, vp, i, vp]
    lib.cuthip_matmul_gguf_workspace_bytes.argtypes = [i, u32, u32, u32, i]
    lib.cuthip_matmul_gguf_ws.argtypes = [i, vp, vp, i, vp, i, u32, u32, u32, u32, u32, i, i, vp, i, vp, C.c_size_t, vp]
    lib.cuthip_matmul_gguf_pair.argtypes = [i, vp, u32, vp, i, vp, u32, vp, vp, i, i, u32, C.POINTER(NormCarry),
                                            C.POINTER(RopeAppend), vp]
    lib.cuthip_matmul_gguf_carry.argtypes = [i, vp, vp, i, vp, i, u32, u32, i, i, vp, C.POINTER(NormCarry), vp]
    f32 = C.c_float
    lib.cuthip_matmul_gguf_pro.argtypes = [i, vp, vp, i, vp, i, u32, u32, i, i, vp, i, vp, f32, vp]
    lib.cuthip_rmsnorm.argtypes = [vp, i, vp, vp, i, u32, u32, u32, f32, vp]
    lib.cuthip_rope_kv_write.argtypes = [vp, vp, vp, i, vp, vp, vp, vp, vp, vp, i, u32, u32, u32, u32, u32, vp]
    lib.cuthip_attn_decode_workspace_bytes.argtypes = [u32, u32, u32]
    lib.cuthip_attn_decode.argtypes = [vp, i, vp, vp, vp, vp, i, u32, u32, u32, u32, f32, u32, vp, C.c_size_t, vp]
    lib.cuthip_attn_decode_static_max_bytes.argtypes = []
    lib.cuthip_attn_partial_splits.argtypes = [u32]
    lib.cuthip_attn_partial_bytes.argtypes = [u32, u32, u32]
    lib.cuthip_attn_decode_partial.argtypes = [vp, i, vp, vp, vp, u32, u32, u32, u32, f32, u32, vp, C.c_size_t, vp]
    lib.cuthip_attn_merge.argtypes = [vp, u32, u32, u32, vp, i, vp]
    lib.cuthip_matmul_gguf_attn_merge.argtypes = [i, vp, vp, u32, u32, u32, vp, i, u32, i, i, vp, C.POINTER(NormCarry), vp]
    lib.cuthip_attn_decode_static.argtypes = [vp, i, vp, vp, vp, vp, i, u32, u32, u32, u32, f32, u32, vp]
    lib.cuthip_silu_mul.argtypes = [vp, i, vp, i, u32, vp]
    lib.cuthip_argmax.argtypes = [vp, i, u32, vp, vp]
    lib.cuthip_repetition_penalty.argtypes = [vp, vp, vp, u32, vp]
    lib.cuthip_argmax_penalized.argtypes = [vp, i, u32, vp, vp, u32, vp, vp]
    lib.cuthip_matmul_gguf_argmax_workspace_bytes.argtypes = [u32]
    lib.cuthip_matmul_gguf_argmax.argtypes = [i, vp, vp, i, vp, i, u32, u32, C.POINTER(NormCarry), vp, vp, u32, vp, C.c_size_t,
                                              vp, vp]
    lib.cuthip_embedding_rows.argtypes = [i, vp, vp, u32, u32, u32, vp, i, u32, vp]
    lib.cuthip_embedding_col.argtypes = [vp, vp, vp, vp, u32, u32, u32, u32, u32, u32, i, vp]
    lib.cuthip_matmul_sep_workspace_bytes.argtypes = [u32, u32, u32]
    lib.cuthip_matmul_sep_workspace_bytes_for.argtypes = [i, i, u32, u32, u32]
    lib.cuthip_matmul_q8_sep.argtypes = [vp, vp, vp, vp, vp, u32, u32, u32, u32, u32, u32, u32, i, i, i, vp, C.c_size_t, vp]
    lib.cuthip_matmul_q4_sep.argtypes = [vp, vp, vp, vp, vp, u32, u32, u32, u32, u32, u32, u32, i, i, i, i, vp, C.c_size_t, vp]
    lib.cuthip_prepare_sep.argtypes = [i, vp, u32, u32, vp, u32, vp, u32, vp]
    lib.cuthip_transpose_q4_nibble.argtypes = [vp, vp, u32, u32, u32, u32, vp]
    lib.cuthip_quantize_rows_q8_0.argtypes = [vp, C.c_uint64, vp, vp]
    lib.cuthip_matmul_dense_f16_workspace_bytes.argtypes = [u32, u32, u32, i]
    lib.cuthip_matmul_dense_f16.argtypes = [vp, vp, i, vp, i, u32, u32, u32, u32, u32, i, i, vp, vp, C.c_size_t, vp]
    lib.cuthip_matmul_q8_i8_workspace_bytes.argtypes = [u32, u32]
    lib.cuthip_matmul_q8_i8.argtypes = [vp, vp, i, vp, i, u32, u32, u32, u32, u32, i, i, vp, vp, C.c_size_t, vp]
    sized = ("cuthip_attn_decode_workspace_bytes", "cuthip_matmul_sep_workspace_bytes", "cuthip_matmul_sep_workspace_bytes_for",
             "cuthip_matmul_gguf_workspace_bytes", "cuthip_matmul_q8_i8_workspace_bytes",
             "cuthip_matmul_dense_f16_workspace_bytes", "cuthip_attn_decode_static_max_bytes",
             "cuthip_matmul_gguf_argmax_workspace_bytes", "cuthip_attn_partial_bytes")
    for n in EXPORTS:
        if n != "cuthip_last_error" and n not in sized:
            getattr(lib, n).restype = i
    for n in sized:
        getattr(lib, n).restype = C.c_size_t
    lib.cuthip_attn_partial_splits.restype = u32
    _lib = lib
    return lib


def check(rc: int) -> None:
    if rc != 0:
        raise CutHipError(f"cut_hip error {rc}: {load().cuthip_last_error().decode()}")


def variants(op: int) -> list[dict]:
    lib = load()
    out = []
    for idx in range(lib.cuthip_variant_count(op)):
        v = VariantInfo()
        check(lib.cuthip_variant_info(op, idx, C.byref(v)))
        out.append({"index": idx, "name": v.name.decode(), "wgX": v.wgX, "wgY": v.wgY, "effTileM": v.effTileM,
                    "effTileN": v.effTileN, "description": v.description.decode()})
    return out


def device_info() -> dict:
    d = DeviceInfo()
    check(load().cuthip_device_info(C.byref(d)))
    return {f: (getattr(d, f).decode() if isinstance(getattr(d, f), bytes) else getattr(d, f)) for f, _ in d._fields_}


def set_tuning(key: str, value: str | None) -> None:
    """Forces a launch shape (tests, sweeps); value None restores the library's own choice (cuthip_set_tuning)."""
    check(load().cuthip_set_tuning(key.encode(), value.encode() if value is not None else None))
