"""Host-side mirror (Python) of the reference's operator interface for the
quantized-matmul path, over torch device tensors.

Same names and argument meaning as ``Operations::dequantize(raw, fmt, rows,
cols)`` (runtime/Operations.cpp:1354-1361) and ``Operations::matmul(a, packedB,
scales)`` (runtime/Operations.cpp:226-231), with the weights kept as GGUF
blocks.  torch only supplies device memory and the current stream; every call
goes through the C ABI of libcut_hip.so.  Shape errors raise, as the
reference's constructors do (MatMulOp.cpp:288-329).
"""
from __future__ import annotations

import ctypes as C

import torch

from . import lib as _l


def _stream_ptr() -> int:
    return torch.cuda.current_stream().cuda_stream


def _fmt(fmt) -> int:
    if isinstance(fmt, str):
        if fmt not in _l.FORMATS:
            raise _l.CutHipError(f"unknown quantization format {fmt!r}")
        return _l.FORMATS[fmt]
    return int(fmt)


def n_bytes(fmt, rows: int, cols: int) -> int:
    f = _fmt(fmt)
    if cols % _l.BLOCK_ELEMS[f]:
        raise _l.CutHipError(f"cols ({cols}) must be a multiple of the block size {_l.BLOCK_ELEMS[f]}")
    return rows * (cols // _l.BLOCK_ELEMS[f]) * _l.BLOCK_BYTES[f]


def dequantize(raw: torch.Tensor, fmt, rows: int, cols: int, dtype: torch.dtype = torch.float32,
               out: torch.Tensor | None = None) -> torch.Tensor:
    """raw: 1-D uint8/int8 device tensor of GGUF blocks -> [rows, cols]."""
    f = _fmt(fmt)
    if not raw.is_cuda or raw.element_size() != 1 or not raw.is_contiguous():
        raise _l.CutHipError("dequantize: raw must be a contiguous 1-byte device tensor")
    need = n_bytes(f, rows, cols)
    if raw.numel() < need:
        raise _l.CutHipError(f"dequantize: raw holds {raw.numel()} bytes, {need} needed")
    if dtype not in (torch.float32, torch.float16):
        raise _l.CutHipError("dequantize: output dtype must be float32 or float16")
    if out is None:
        out = torch.empty((rows, cols), dtype=dtype, device=raw.device)
    stride = out.stride(0) if out.dim() == 2 else cols
    _l.check(_l.load().cuthip_dequant(f, raw.data_ptr(), out.data_ptr(), _l.F16 if dtype == torch.float16 else _l.F32,
                                      rows, cols, stride, _stream_ptr()))
    return out


_FMT_NAMES = {_l.Q8_0: "Q8_0", _l.Q4_0: "Q4_0", _l.Q4_K: "Q4_K", _l.Q6_K: "Q6_K"}
_tuning = None


def enable_tuning(path: str | None = None) -> bool:
    """Lets matmul_gguf consult shape rules (cut_amd/tuning_data.json by default, the "hip" backend section) when it
    is called with variant = -1, no epilogue and a workspace: the reference's VariantSelector mechanism
    (MatMulOp.cpp:242-246).  Returns False, and changes nothing, if the file cannot be loaded."""
    global _tuning
    from . import variant_selector as _vs
    sel = _vs.VariantSelector()
    if not sel.load(path or _vs.DEFAULT_PATH):
        return False
    _tuning = sel
    return True


def disable_tuning() -> None:
    global _tuning
    _tuning = None


def matmul_gguf(a: torch.Tensor, w_blocks: torch.Tensor, fmt, N: int, K: int, out_dtype: torch.dtype | None = None,
                out: torch.Tensor | None = None, unary: str | None = None, binary: str | None = None,
                d: torch.Tensor | None = None, variant: int = -1, workspace: torch.Tensor | None = None,
                swiglu_pairs: bool = False) -> torch.Tensor:
    """C = A . dequant(W)^T.  a: [M, K] or [K] (fp32 or fp16); w_blocks: N rows
    of K/blk GGUF blocks as a 1-byte device tensor.  With `workspace` (a device
    byte tensor from matmul_gguf_workspace) the call goes through
    cuthip_matmul_gguf_ws, which opens variant 4 (dequantize once, dense GEMM).
    swiglu_pairs: weight rows 2i / 2i+1 are gate_i / up_i and the result is [M, N/2] = silu(gate) * up (M <= 8)."""
    f = _fmt(fmt)
    if a.dim() == 1:
        a2 = a.unsqueeze(0)
    elif a.dim() == 2:
        a2 = a
    else:
        raise _l.CutHipError("matmul: A must be 1D or 2D")
    M = a2.shape[0]
    if a2.shape[1] != K:
        raise _l.CutHipError(f"matmul: B rows ({K}) must match A cols ({a2.shape[1]})")
    if a2.dtype not in (torch.float32, torch.float16) or a2.stride(1) != 1:
        raise _l.CutHipError("matmul: A must be float32/float16 with unit inner stride")
    if w_blocks.numel() < n_bytes(f, N, K):
        raise _l.CutHipError("matmul: weight tensor too small for [N, K]")
    odt = out_dtype or a2.dtype
    if out is None:
        out = torch.empty((M, N // 2 if swiglu_pairs else N), dtype=odt, device=a.device)
    epi, op, dptr = _l.EPI_NONE, 0, None
    if swiglu_pairs:
        epi = _l.EPI_SWIGLU_PAIRS
    elif unary is not None:
        epi, op = _l.EPI_UNARY, _l.UNARY[unary]
    elif binary is not None:
        if d is None or d.shape != out.shape or d.dtype != out.dtype or d.stride(0) != out.stride(0):
            raise _l.CutHipError("matmul: binary epilogue needs D with the shape, dtype and stride of C")
        epi, op, dptr = _l.EPI_BINARY, _l.BINARY[binary], d.data_ptr()
    adt = _l.F16 if a2.dtype == torch.float16 else _l.F32
    cdt = _l.F16 if out.dtype == torch.float16 else _l.F32
    if _tuning is not None and variant == -1 and epi == _l.EPI_NONE and workspace is not None:
        variant = _tuning.select("MatMulGguf" + _FMT_NAMES[f], [M, K, N], -1)
        # a rule may name a variant this process cannot run (the vendor-GEMM variant without its library): the
        # hand-written two-pass GEMM takes its place
        if variant >= 0 and _l.load().cuthip_variant_available(_l.OP_MATMUL_GGUF, variant) != 1:
            variant = 4 if variant == 5 else -1
    if workspace is not None:
        _l.check(_l.load().cuthip_matmul_gguf_ws(
            f, w_blocks.data_ptr(), a2.data_ptr(), adt, out.data_ptr(), cdt, M, K, N, a2.stride(0), out.stride(0), epi, op,
            dptr, variant, workspace.data_ptr(), workspace.numel() * workspace.element_size(), _stream_ptr()))
    else:
        _l.check(_l.load().cuthip_matmul_gguf(
            f, w_blocks.data_ptr(), a2.data_ptr(), adt, out.data_ptr(), cdt, M, K, N, a2.stride(0), out.stride(0), epi, op,
            dptr, variant, _stream_ptr()))
    return out


def norm_carry(sumsq_parts: torch.Tensor | None = None, eps: float = 0.0, next_norm_weight: torch.Tensor | None = None,
               next_x16: torch.Tensor | None = None, next_sumsq_parts: torch.Tensor | None = None) -> "_l.NormCarry":
    """cuthip_norm_carry_t from device tensors (float32 [K/8] / [N] / [N/8], fp16 [N] output)."""
    def ptr(t, dtype):
        if t is None:
            return None
        if t.dtype != dtype or not t.is_contiguous():
            raise _l.CutHipError("norm_carry: wrong dtype or non-contiguous tensor")
        return t.data_ptr()
    return _l.NormCarry(ptr(sumsq_parts, torch.float32), eps, ptr(next_norm_weight, torch.float32), ptr(next_x16, torch.float16),
                        ptr(next_sumsq_parts, torch.float32))


def matmul_gguf_carry(a: torch.Tensor, w_blocks: torch.Tensor, fmt, N: int, K: int, out: torch.Tensor, carry, binary: str | None = None,
                      d: torch.Tensor | None = None, swiglu_pairs: bool = False) -> torch.Tensor:
    """Batch-1 matmul taking part in a carried RMSNorm (cuthip_matmul_gguf_carry); a [K], out [N] (or [N/2])."""
    f = _fmt(fmt)
    if a.numel() != K or a.dtype not in (torch.float32, torch.float16) or not a.is_contiguous() or not out.is_contiguous():
        raise _l.CutHipError("matmul_carry: A must be a contiguous float32/float16 vector of K elements, out contiguous")
    if w_blocks.numel() < n_bytes(f, N, K) or out.numel() != (N // 2 if swiglu_pairs else N):
        raise _l.CutHipError("matmul_carry: weight tensor too small or output of the wrong size")
    epi, op, dptr = _l.EPI_NONE, 0, None
    if swiglu_pairs:
        epi = _l.EPI_SWIGLU_PAIRS
    elif binary is not None:
        if d is None or d.numel() != N or d.dtype != out.dtype:
            raise _l.CutHipError("matmul_carry: binary epilogue needs D with the size and dtype of C")
        epi, op, dptr = _l.EPI_BINARY, _l.BINARY[binary], d.data_ptr()
    import ctypes
    _l.check(_l.load().cuthip_matmul_gguf_carry(f, w_blocks.data_ptr(), a.data_ptr(), _dt(a), out.data_ptr(), _dt(out), K, N, epi,
                                                op, dptr, ctypes.byref(carry) if carry is not None else None, _stream_ptr()))
    return out


def rope_append(runtime_params: torch.Tensor, cos_t: torch.Tensor, sin_t: torch.Tensor, q_out: torch.Tensor, k_cache: torch.Tensor,
                v_cache: torch.Tensor, q_dim: int, head_dim: int) -> "_l.RopeAppend":
    """cuthip_rope_append_t for matmul_gguf_pair: rotated q to q_out, rotated k and v to the cache row of the position."""
    if k_cache.dtype != torch.float16 or v_cache.dtype != torch.float16 or k_cache.stride(0) != v_cache.stride(0):
        raise _l.CutHipError("rope_append: caches must be fp16 with one row stride")
    return _l.RopeAppend(runtime_params.data_ptr(), cos_t.data_ptr(), sin_t.data_ptr(), q_out.data_ptr(), _dt(q_out),
                         k_cache.data_ptr(), v_cache.data_ptr(), q_dim, head_dim, k_cache.stride(0),
                         min(k_cache.shape[0], cos_t.shape[0]))


def interleave_rope_rows(w_blocks: torch.Tensor, n_rows: int, head_dim: int) -> torch.Tensor:
    """Rows of [heads * head_dim, K] GGUF blocks re-ordered inside every head to d = 0, half, 1, half + 1, ...: the
    layout the RoPE epilogue of matmul_gguf_pair reads (a permutation of whole block rows)."""
    rb = w_blocks.numel() // n_rows
    half = head_dim // 2
    w = w_blocks.view(n_rows // head_dim, 2, half, rb)
    return w.permute(0, 2, 1, 3).reshape(-1).contiguous()


def matmul_gguf_pair(a: torch.Tensor, wa: torch.Tensor, fmt_a, Na: int, out_a: torch.Tensor | None, wb: torch.Tensor, fmt_b,
                     Nb: int, out_b: torch.Tensor | None, K: int, carry=None, rope=None) -> None:
    """out_a = a . dequant(wa)^T and out_b = a . dequant(wb)^T for one activation vector a [K], in one launch where the
    formats allow it (cuthip_matmul_gguf_pair)."""
    fa, fb = _fmt(fmt_a), _fmt(fmt_b)
    if a.numel() != K or a.dtype not in (torch.float32, torch.float16) or not a.is_contiguous():
        raise _l.CutHipError("matmul_pair: A must be a contiguous float32/float16 vector of K elements")
    if wa.numel() < n_bytes(fa, Na, K) or wb.numel() < n_bytes(fb, Nb, K):
        raise _l.CutHipError("matmul_pair: weight tensor too small for [N, K]")
    import ctypes
    if rope is not None:   # the epilogue writes q_out and the caches; the plain outputs are not used
        _l.check(_l.load().cuthip_matmul_gguf_pair(
            fa, wa.data_ptr(), Na, None, fb, wb.data_ptr(), Nb, None, a.data_ptr(), _dt(a), _l.F32, K,
            ctypes.byref(carry) if carry is not None else None, ctypes.byref(rope), _stream_ptr()))
        return
    if out_a.dtype != out_b.dtype or out_a.numel() != Na or out_b.numel() != Nb or not (out_a.is_contiguous() and out_b.is_contiguous()):
        raise _l.CutHipError("matmul_pair: outputs must be contiguous [Na] and [Nb] of one dtype")
    _l.check(_l.load().cuthip_matmul_gguf_pair(
        fa, wa.data_ptr(), Na, out_a.data_ptr(), fb, wb.data_ptr(), Nb, out_b.data_ptr(), a.data_ptr(), _dt(a), _dt(out_a), K,
        ctypes.byref(carry) if carry is not None else None, None, _stream_ptr()))


def matmul_gguf_workspace(fmt, M: int, K: int, N: int, a_dtype: torch.dtype, device) -> torch.Tensor:
    """Scratch for the two-pass prefill matmul (variant 4): N*K fp16 (+ M*K fp16 for fp32 activations)."""
    n = _l.load().cuthip_matmul_gguf_workspace_bytes(_fmt(fmt), M, K, N, _l.F16 if a_dtype == torch.float16 else _l.F32)
    return torch.empty(max(int(n), 256), dtype=torch.uint8, device=device)


# ---- operators between the matmuls of a decode step ---------------------------------------------------
def _dt(t: torch.Tensor) -> int:
    if t.dtype == torch.float16:
        return _l.F16
    if t.dtype == torch.float32:
        return _l.F32
    raise _l.CutHipError(f"activations must be float16 or float32, got {t.dtype}")


def rmsnorm(x: torch.Tensor, weight: torch.Tensor, eps: float, out: torch.Tensor | None = None,
            out_dtype: torch.dtype | None = None) -> torch.Tensor:
    """x: [rows, dim] or [dim]; weight: fp32 [dim] (RMSNormOpNode of the reference)."""
    x2 = x if x.dim() == 2 else x.reshape(1, -1)
    if weight.dtype != torch.float32 or weight.numel() != x2.shape[1] or x2.stride(1) != 1:
        raise _l.CutHipError("rmsnorm: weight must be fp32 [dim] and x rows contiguous")
    if out is None:
        out = torch.empty(x2.shape, dtype=out_dtype or x.dtype, device=x.device)
    _l.check(_l.load().cuthip_rmsnorm(x2.data_ptr(), _dt(x2), weight.data_ptr(), out.data_ptr(), _dt(out), x2.shape[0],
                                      x2.shape[1], x2.stride(0), eps, _stream_ptr()))
    return out


def rope_kv_write(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, runtime_params: torch.Tensor, cos_t: torch.Tensor,
                  sin_t: torch.Tensor, k_cache: torch.Tensor, v_cache: torch.Tensor, head_dim: int,
                  q_out: torch.Tensor) -> torch.Tensor:
    """q [q_dim], k, v [kv_dim] (same dtype); caches fp16 [max_ctx, aligned_kv_dim]; runtime_params int32/uint32[2] on device."""
    if k_cache.dtype != torch.float16 or v_cache.dtype != torch.float16 or k.dtype != q.dtype or v.dtype != q.dtype:
        raise _l.CutHipError("rope_kv_write: caches must be fp16 and q, k, v of one dtype")
    _l.check(_l.load().cuthip_rope_kv_write(q.data_ptr(), k.data_ptr(), v.data_ptr(), _dt(q), runtime_params.data_ptr(),
                                            cos_t.data_ptr(), sin_t.data_ptr(), k_cache.data_ptr(), v_cache.data_ptr(),
                                            q_out.data_ptr(), _dt(q_out), q.numel(), k.numel(), head_dim, k_cache.stride(0),
                                            min(k_cache.shape[0], cos_t.shape[0]), _stream_ptr()))
    return q_out


def attn_decode_workspace(n_heads: int, head_dim: int, max_seq_len: int, device) -> torch.Tensor:
    n = _l.load().cuthip_attn_decode_workspace_bytes(n_heads, head_dim, max_seq_len)
    return torch.empty(n, dtype=torch.uint8, device=device)


def attn_decode(q: torch.Tensor, k_cache: torch.Tensor, v_cache: torch.Tensor, runtime_params: torch.Tensor, n_heads: int,
                n_kv_heads: int, head_dim: int, scale: float, workspace: torch.Tensor, out: torch.Tensor,
                max_seq_len: int | None = None) -> torch.Tensor:
    _l.check(_l.load().cuthip_attn_decode(q.data_ptr(), _dt(q), k_cache.data_ptr(), v_cache.data_ptr(),
                                          runtime_params.data_ptr(), out.data_ptr(), _dt(out), n_heads, n_kv_heads, head_dim,
                                          k_cache.stride(0), scale, max_seq_len or k_cache.shape[0], workspace.data_ptr(),
                                          workspace.numel(), _stream_ptr()))
    return out


def attn_decode_static(q: torch.Tensor, k_cache: torch.Tensor, v_cache: torch.Tensor, runtime_params: torch.Tensor, n_heads: int,
                       n_kv_heads: int, head_dim: int, scale: float, out: torch.Tensor,
                       max_seq_len: int | None = None) -> torch.Tensor:
    """attn_decode on the library's built-in scratch (no workspace, no allocation; shapes up to 4 MiB of partials)."""
    _l.check(_l.load().cuthip_attn_decode_static(q.data_ptr(), _dt(q), k_cache.data_ptr(), v_cache.data_ptr(),
                                                 runtime_params.data_ptr(), out.data_ptr(), _dt(out), n_heads, n_kv_heads,
                                                 head_dim, k_cache.stride(0), scale, max_seq_len or k_cache.shape[0],
                                                 _stream_ptr()))
    return out


def attn_partial_records(n_heads: int, head_dim: int, max_seq_len: int, device) -> torch.Tensor:
    """Records of attn_decode_partial: [n_heads, splits, 2 + head_dim] fp32 (max, sum, un-normalised output)."""
    splits = _l.load().cuthip_attn_partial_splits(max_seq_len)
    return torch.empty((n_heads, splits, 2 + head_dim), dtype=torch.float32, device=device)


def attn_decode_partial(q: torch.Tensor, k_cache: torch.Tensor, v_cache: torch.Tensor, runtime_params: torch.Tensor, n_heads: int,
                        n_kv_heads: int, head_dim: int, scale: float, records: torch.Tensor,
                        max_seq_len: int | None = None) -> torch.Tensor:
    """The attention up to the per-split records (cuthip_attn_decode_partial); attn_merge or matmul_gguf_attn_merge
    folds them.  records: attn_partial_records() for the same max_seq_len."""
    _l.check(_l.load().cuthip_attn_decode_partial(q.data_ptr(), _dt(q), k_cache.data_ptr(), v_cache.data_ptr(),
                                                  runtime_params.data_ptr(), n_heads, n_kv_heads, head_dim, k_cache.stride(0),
                                                  scale, max_seq_len or k_cache.shape[0], records.data_ptr(),
                                                  records.numel() * records.element_size(), _stream_ptr()))
    return records


def attn_merge(records: torch.Tensor, out: torch.Tensor) -> torch.Tensor:
    """out[h, :] from records [n_heads, splits, 2 + head_dim] (cuthip_attn_merge)."""
    if records.dtype != torch.float32 or records.dim() != 3 or not records.is_contiguous() or not out.is_contiguous():
        raise _l.CutHipError("attn_merge: records must be a contiguous float32 [heads, splits, 2 + head_dim] tensor")
    n_heads, splits, rec = records.shape
    if out.numel() != n_heads * (rec - 2):
        raise _l.CutHipError("attn_merge: out must hold heads x head_dim elements")
    _l.check(_l.load().cuthip_attn_merge(records.data_ptr(), splits, n_heads, rec - 2, out.data_ptr(), _dt(out), _stream_ptr()))
    return out


def matmul_gguf_attn_merge(records: torch.Tensor, w_blocks: torch.Tensor, fmt, N: int, out: torch.Tensor, carry=None,
                           binary: str | None = None, d: torch.Tensor | None = None) -> torch.Tensor:
    """out [N] = merge(records) . dequant(W)^T with K = heads x head_dim (cuthip_matmul_gguf_attn_merge): the merge of the
    attention splits rides in the staging of the matmul's activations."""
    f = _fmt(fmt)
    if records.dtype != torch.float32 or records.dim() != 3 or not records.is_contiguous() or not out.is_contiguous():
        raise _l.CutHipError("matmul_gguf_attn_merge: records must be a contiguous float32 [heads, splits, 2 + head_dim] tensor")
    n_heads, splits, rec = records.shape
    K = n_heads * (rec - 2)
    if w_blocks.numel() < n_bytes(f, N, K) or out.numel() != N:
        raise _l.CutHipError("matmul_gguf_attn_merge: weight tensor too small or output of the wrong size")
    epi, op, dptr = _l.EPI_NONE, 0, None
    if binary is not None:
        if d is None or d.numel() != N or d.dtype != out.dtype:
            raise _l.CutHipError("matmul_gguf_attn_merge: binary epilogue needs D with the size and dtype of C")
        epi, op, dptr = _l.EPI_BINARY, _l.BINARY[binary], d.data_ptr()
    import ctypes
    _l.check(_l.load().cuthip_matmul_gguf_attn_merge(f, w_blocks.data_ptr(), records.data_ptr(), splits, n_heads, rec - 2,
                                                     out.data_ptr(), _dt(out), N, epi, op, dptr,
                                                     ctypes.byref(carry) if carry is not None else None, _stream_ptr()))
    return out


def silu_mul(gate_up: torch.Tensor, out: torch.Tensor) -> torch.Tensor:
    _l.check(_l.load().cuthip_silu_mul(gate_up.data_ptr(), _dt(gate_up), out.data_ptr(), _dt(out), out.numel(), _stream_ptr()))
    return out


def argmax(x: torch.Tensor, out_index: torch.Tensor) -> torch.Tensor:
    _l.check(_l.load().cuthip_argmax(x.data_ptr(), _dt(x), x.numel(), out_index.data_ptr(), _stream_ptr()))
    return out_index


def repetition_penalty(logits: torch.Tensor, factors: torch.Tensor, out: torch.Tensor | None = None) -> torch.Tensor:
    """RepetitionPenaltyOpNode on the dense fp32 factor vector (1 for tokens that are not penalised)."""
    if logits.dtype != torch.float32 or factors.dtype != torch.float32 or logits.numel() != factors.numel():
        raise _l.CutHipError("RepetitionPenalty: logits and penaltyFactors must be fp32 tensors of the same shape")
    out = torch.empty_like(logits) if out is None else out
    _l.check(_l.load().cuthip_repetition_penalty(logits.data_ptr(), factors.data_ptr(), out.data_ptr(), logits.numel(), _stream_ptr()))
    return out


def _pen_args(pen_tokens, pen_factors):
    if pen_tokens is None:
        return None, None, 0
    if pen_tokens.dtype != torch.int32 or pen_factors.dtype != torch.float32 or pen_tokens.numel() != pen_factors.numel():
        raise _l.CutHipError("penalised tokens are int32 ids with one fp32 factor each")
    return pen_tokens.data_ptr(), pen_factors.data_ptr(), pen_tokens.numel()


def argmax_penalized(logits: torch.Tensor, out_index: torch.Tensor, pen_tokens: torch.Tensor | None = None,
                     pen_factors: torch.Tensor | None = None) -> torch.Tensor:
    """Repetition penalty on the listed tokens (in place), then the arg-max (cuthip_argmax_penalized)."""
    pt, pf, n = _pen_args(pen_tokens, pen_factors)
    _l.check(_l.load().cuthip_argmax_penalized(logits.data_ptr(), _dt(logits), logits.numel(), pt, pf, n, out_index.data_ptr(),
                                               _stream_ptr()))
    return out_index


def lm_head_workspace(N: int, device) -> torch.Tensor:
    return torch.empty(max(int(_l.load().cuthip_matmul_gguf_argmax_workspace_bytes(N)), 8), dtype=torch.uint8, device=device)


def matmul_gguf_argmax(a: torch.Tensor, w_blocks: torch.Tensor, fmt, N: int, K: int, logits: torch.Tensor, out_index: torch.Tensor,
                       carry=None, pen_tokens: torch.Tensor | None = None, pen_factors: torch.Tensor | None = None,
                       workspace: torch.Tensor | None = None) -> torch.Tensor:
    """The output head with the sampling folded in: logits = a . dequant(W)^T, penalty on the listed tokens, arg-max."""
    f = _fmt(fmt)
    if a.numel() != K or not a.is_contiguous() or logits.numel() != N or not logits.is_contiguous():
        raise _l.CutHipError("matmul_gguf_argmax: a is a contiguous vector of K elements, logits one of N")
    pt, pf, n = _pen_args(pen_tokens, pen_factors)
    _l.check(_l.load().cuthip_matmul_gguf_argmax(f, w_blocks.data_ptr(), a.data_ptr(), _dt(a), logits.data_ptr(), _dt(logits), K, N,
                                                 C.byref(carry) if carry is not None else None, pt, pf, n,
                                                 workspace.data_ptr() if workspace is not None else None,
                                                 workspace.numel() if workspace is not None else 0, out_index.data_ptr(),
                                                 _stream_ptr()))
    return out_index


def embedding_rows(w_blocks: torch.Tensor, fmt, token_ids: torch.Tensor, n_rows: int, dim: int, out: torch.Tensor) -> torch.Tensor:
    """out[i] = dequant(row token_ids[i]) of a GGUF table [n_rows, dim]; token_ids int32/uint32 on the device."""
    if token_ids.dtype not in (torch.int32, torch.uint32) or out.stride(-1) != 1 or out.numel() < token_ids.numel() * dim:
        raise _l.CutHipError("embedding_rows: token ids are 32-bit integers, out holds one row of dim per id")
    out2 = out if out.dim() == 2 else out.view(token_ids.numel(), -1)
    _l.check(_l.load().cuthip_embedding_rows(_fmt(fmt), w_blocks.data_ptr(), token_ids.data_ptr(), token_ids.numel(), n_rows, dim,
                                             out2.data_ptr(), _dt(out2), out2.stride(0), _stream_ptr()))
    return out


def embedding_col(indices: torch.Tensor, matrix: torch.Tensor, scales: torch.Tensor | None, emb_dim: int, vocab: int,
                  out: torch.Tensor | None = None) -> torch.Tensor:
    """EmbeddingColOpNode: matrix [emb_dim, vocab_stride] column-wise, fp16 (scales None) or int8 with fp16 scales
    [emb_dim / 32, scale_stride]; returns fp32 [len(indices), emb_dim]."""
    fmt = 0 if scales is None else 1
    if matrix.dim() != 2 or matrix.dtype != (torch.float16 if fmt == 0 else torch.int8) or indices.dtype not in (torch.int32, torch.uint32):
        raise _l.CutHipError("embedding_col: matrix is 2-D fp16 (no scales) or int8 (fp16 scales), indices 32-bit integers")
    if out is None:
        out = torch.empty((indices.numel(), emb_dim), dtype=torch.float32, device=matrix.device)
    _l.check(_l.load().cuthip_embedding_col(indices.data_ptr(), matrix.data_ptr(), scales.data_ptr() if fmt else None, out.data_ptr(),
                                            indices.numel(), emb_dim, matrix.stride(0), scales.stride(0) if fmt else 0, out.stride(0),
                                            vocab, fmt, _stream_ptr()))
    return out


# ---- the reference's separated weight layout ----------------------------------------------------------
def matmul_sep(a: torch.Tensor, b: torch.Tensor, scales: torch.Tensor, N: int, q4: bool = False, affine: bool = False,
               out: torch.Tensor | None = None, unary: str | None = None, binary: str | None = None,
               d: torch.Tensor | None = None, variant: int = -1) -> torch.Tensor:
    """Operations::matmul(a, packedB, scalesB) of the reference on its own layout: a fp32 [M, K]; b int8 [K, N]
    (q4: uint8 [K, N/2], even column in the low nibble); scales fp16 [K/32, N] ([2K/32, N] when affine).
    variant: the reference's `spec` (an index of its MatMulQ8 / MatMulQ4 variant tables), -1 = by shape."""
    a2 = a if a.dim() == 2 else a.reshape(1, -1)
    M, K = a2.shape
    if a2.dtype != torch.float32 or scales.dtype != torch.float16 or b.element_size() != 1 or b.dim() != 2 or scales.dim() != 2:
        raise _l.CutHipError("matmul_sep: a must be fp32, b a 2-D 1-byte tensor and scales a 2-D fp16 tensor")
    rows_s = (2 if affine else 1) * (K // 32)
    if b.shape[0] != K or scales.shape[0] != rows_s or b.shape[1] < ((N + 1) // 2 if q4 else N) or scales.shape[1] < N:
        raise _l.CutHipError(f"matmul_sep: shapes do not match K = {K}, N = {N} (b {tuple(b.shape)}, scales {tuple(scales.shape)})")
    if out is None:
        out = torch.empty((M, N), dtype=torch.float32, device=a.device)
    epi, op, dptr = _l.EPI_NONE, 0, None
    if unary is not None:
        epi, op = _l.EPI_UNARY, _l.UNARY[unary]
    elif binary is not None:
        if d is None or d.shape != out.shape or d.dtype != torch.float32 or d.stride(0) != out.stride(0):
            raise _l.CutHipError("matmul_sep: binary epilogue needs an fp32 D with the shape and stride of C")
        epi, op, dptr = _l.EPI_BINARY, _l.BINARY[binary], d.data_ptr()
    lib = _l.load()
    ws_bytes = lib.cuthip_matmul_sep_workspace_bytes_for(_l.OP_MATMUL_Q4 if q4 else _l.OP_MATMUL_Q8, variant, M, K, N)
    ws = torch.empty(max(ws_bytes, 1), dtype=torch.uint8, device=a.device)
    common = (a2.data_ptr(), b.data_ptr(), scales.data_ptr(), dptr, out.data_ptr(), M, K, N, a2.stride(0), b.stride(0),
              out.stride(0), scales.stride(0), epi, op)
    if q4:
        _l.check(lib.cuthip_matmul_q4_sep(*common, int(affine), variant, ws.data_ptr(), ws_bytes, _stream_ptr()))
    else:
        _l.check(lib.cuthip_matmul_q8_sep(*common, variant, ws.data_ptr(), ws_bytes, _stream_ptr()))
    return out


def matmul_dense_f16(a: torch.Tensor, w16: torch.Tensor, out_dtype: torch.dtype | None = None, out: torch.Tensor | None = None,
                     unary: str | None = None, binary: str | None = None, d: torch.Tensor | None = None,
                     workspace: torch.Tensor | None = None) -> torch.Tensor:
    """Prefill matmul on resident dequantized weights: w16 fp16 [N, K] (from dequantize(..., torch.float16)), a [M, K]
    fp16 or fp32; C = a . w16^T.  The quantized blocks stay the operand of the decode GEMV; this copy serves prefill."""
    a2 = a if a.dim() == 2 else a.reshape(1, -1)
    M, K = a2.shape
    if w16.dtype != torch.float16 or w16.dim() != 2 or w16.shape[1] != K or not w16.is_contiguous():
        raise _l.CutHipError(f"matmul_dense_f16: w16 must be a contiguous fp16 [N, {K}] tensor")
    N = w16.shape[0]
    if a2.dtype not in (torch.float32, torch.float16) or a2.stride(1) != 1:
        raise _l.CutHipError("matmul_dense_f16: a must be fp32 / fp16 with contiguous rows")
    if out is None:
        out = torch.empty((M, N), dtype=out_dtype or a2.dtype, device=a.device)
    epi, op, dptr = _l.EPI_NONE, 0, None
    if unary is not None:
        epi, op = _l.EPI_UNARY, _l.UNARY[unary]
    elif binary is not None:
        if d is None or d.shape != out.shape or d.dtype != out.dtype or d.stride(0) != out.stride(0):
            raise _l.CutHipError("matmul_dense_f16: binary epilogue needs a D with the dtype, shape and stride of C")
        epi, op, dptr = _l.EPI_BINARY, _l.BINARY[binary], d.data_ptr()
    lib = _l.load()
    if workspace is None:
        workspace = torch.empty(max(lib.cuthip_matmul_dense_f16_workspace_bytes(M, K, N, _dt(a2)), 256), dtype=torch.uint8,
                                device=a.device)
    _l.check(lib.cuthip_matmul_dense_f16(w16.data_ptr(), a2.data_ptr(), _dt(a2), out.data_ptr(), _dt(out), M, K, N,
                                         a2.stride(0), out.stride(0), epi, op, dptr, workspace.data_ptr(), workspace.numel(),
                                         _stream_ptr()))
    return out


def matmul_q8_i8(a: torch.Tensor, w_blocks: torch.Tensor, N: int, K: int, out_dtype: torch.dtype | None = None,
                 out: torch.Tensor | None = None, unary: str | None = None, binary: str | None = None,
                 d: torch.Tensor | None = None, workspace: torch.Tensor | None = None) -> torch.Tensor:
    """Q8_0 weights (GGUF blocks [N][K/32]) x activations quantized to int8 per 32 elements, on the int8 matrix
    core: the arithmetic of the reference's MatMulQ8GemvDot for any M.  Opt-in: about 5e-3 from the fp32 path."""
    a2 = a if a.dim() == 2 else a.reshape(1, -1)
    M = a2.shape[0]
    if a2.shape[1] != K or a2.dtype not in (torch.float32, torch.float16) or a2.stride(1) != 1:
        raise _l.CutHipError(f"matmul_q8_i8: a must be fp32 / fp16 [M, {K}] with contiguous rows")
    if out is None:
        out = torch.empty((M, N), dtype=out_dtype or a2.dtype, device=a.device)
    epi, op, dptr = _l.EPI_NONE, 0, None
    if unary is not None:
        epi, op = _l.EPI_UNARY, _l.UNARY[unary]
    elif binary is not None:
        if d is None or d.shape != out.shape or d.dtype != out.dtype or d.stride(0) != out.stride(0):
            raise _l.CutHipError("matmul_q8_i8: binary epilogue needs a D with the dtype, shape and stride of C")
        epi, op, dptr = _l.EPI_BINARY, _l.BINARY[binary], d.data_ptr()
    lib = _l.load()
    need = lib.cuthip_matmul_q8_i8_workspace_bytes(M, K)
    if workspace is None:
        workspace = torch.empty(max(need, 16), dtype=torch.uint8, device=a.device)
    _l.check(lib.cuthip_matmul_q8_i8(w_blocks.data_ptr(), a2.data_ptr(), _dt(a2), out.data_ptr(), _dt(out), M, K, N,
                                     a2.stride(0), out.stride(0), epi, op, dptr, workspace.data_ptr(), workspace.numel(),
                                     _stream_ptr()))
    return out


def prepare_sep(w_blocks: torch.Tensor, fmt, N: int, K: int, stride_b: int | None = None, scale_stride: int | None = None):
    """GGUF blocks [N rows of K/blk blocks] on the device -> (B, scales) in the reference's separated [K, N] layout:
    Q8_0 -> int8 [K, N] + fp16 [K/32, N]; Q4_0 -> nibbles uint8 [K, N/2] + fp16 [K/32, N]; Q4_K -> affine Q4, nibbles
    + fp16 [2K/32, N] (scales then minima: requantizeQ4KToAffine).  Row strides default to the reference's padding
    to multiples of 4 elements (MatMulOp.cpp:514-541)."""
    f = _fmt(fmt)
    if f not in (_l.Q8_0, _l.Q4_0, _l.Q4_K):
        raise _l.CutHipError("prepare_sep: only Q8_0, Q4_0 and Q4_K have a separated layout")
    q4 = f != _l.Q8_0
    width = (N // 2) if q4 else N
    sb = stride_b if stride_b is not None else (width + 3) & ~3
    ss = scale_stride if scale_stride is not None else (N + 3) & ~3
    rows_s = (2 if f == _l.Q4_K else 1) * (K // 32)
    B = torch.zeros((K, sb), dtype=torch.uint8 if q4 else torch.int8, device=w_blocks.device)
    S = torch.zeros((rows_s, ss), dtype=torch.float16, device=w_blocks.device)
    _l.check(_l.load().cuthip_prepare_sep(f, w_blocks.data_ptr(), N, K, B.data_ptr(), sb, S.data_ptr(), ss, _stream_ptr()))
    return B, S


def transpose_q4_nibble(packed: torch.Tensor, N: int, K: int) -> torch.Tensor:
    """Operations::transposeQ4(packed, N, K) of the reference: GGML-order nibbles [N, K/2] -> [K, N/2]."""
    if packed.dim() != 2 or packed.element_size() != 1 or packed.stride(1) != 1:
        raise _l.CutHipError("transpose_q4_nibble: packed must be a 2-D 1-byte tensor with contiguous rows")
    so = (N // 2 + 3) & ~3
    out = torch.zeros((K, so), dtype=torch.uint8, device=packed.device)
    _l.check(_l.load().cuthip_transpose_q4_nibble(packed.data_ptr(), out.data_ptr(), N, K, packed.stride(0), so, _stream_ptr()))
    return out


def quantize_rows_q8_0(x: torch.Tensor) -> torch.Tensor:
    """quantizeRowsQ8_0 of the reference's runner on the device: fp32 [n] -> Q8_0 blocks (uint8 [n/32 * 34])."""
    if x.dtype != torch.float32 or not x.is_contiguous():
        raise _l.CutHipError("quantize_rows_q8_0: x must be a contiguous fp32 tensor")
    n = x.numel()
    out = torch.empty(max(n // 32, 1) * 34, dtype=torch.uint8, device=x.device)
    _l.check(_l.load().cuthip_quantize_rows_q8_0(x.data_ptr(), n, out.data_ptr(), _stream_ptr()))
    return out


def matmul_gguf_pro(a: torch.Tensor, w_blocks: torch.Tensor, fmt, N: int, K: int, out: torch.Tensor, prologue: str,
                    norm_weight: torch.Tensor | None = None, eps: float = 0.0, unary: str | None = None,
                    binary: str | None = None, d: torch.Tensor | None = None) -> torch.Tensor:
    """Batch-1 matmul with the preceding operator fused into the activation staging:
    prologue "rmsnorm": a = x [K] (fp32 or fp16), norm_weight fp32 [K];  "swiglu": a = [gate | up] fp16 [2K]."""
    pro = {"rmsnorm": 1, "swiglu": 2}[prologue]
    need = K if pro == 1 else 2 * K
    if a.numel() != need or not a.is_contiguous() or out.numel() != N:
        raise _l.CutHipError(f"matmul_gguf_pro: a must hold {need} contiguous elements and out {N}")
    epi, op, dptr = _l.EPI_NONE, 0, None
    if unary is not None:
        epi, op = _l.EPI_UNARY, _l.UNARY[unary]
    elif binary is not None:
        if d is None or d.numel() != N or d.dtype != out.dtype:
            raise _l.CutHipError("matmul_gguf_pro: binary epilogue needs D like C")
        epi, op, dptr = _l.EPI_BINARY, _l.BINARY[binary], d.data_ptr()
    _l.check(_l.load().cuthip_matmul_gguf_pro(_fmt(fmt), w_blocks.data_ptr(), a.data_ptr(), _dt(a), out.data_ptr(), _dt(out), K, N,
                                              epi, op, dptr, pro, norm_weight.data_ptr() if norm_weight is not None else None,
                                              eps, _stream_ptr()))
    return out
