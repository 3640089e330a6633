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


def matmul_gguf(a: torch.Tensor, w_blocks: torch.Tensor, fmt, N: int, K: int, out_dtype: torch.dtype | None = None,
                out: torch.Tensor | None = None, unary: str | None = None, binary: str | None = None,
                d: torch.Tensor | None = None, variant: int = -1) -> torch.Tensor:
    """C = A . dequant(W)^T.  a: [M, K] or [K] (fp32 or fp16); w_blocks: N rows
    of K/blk GGUF blocks as a 1-byte device tensor."""
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
        out = torch.empty((M, N), dtype=odt, device=a.device)
    epi, op, dptr = _l.EPI_NONE, 0, None
    if unary is not None:
        epi, op = _l.EPI_UNARY, _l.UNARY[unary]
    elif binary is not None:
        if d is None or d.shape != out.shape or d.dtype != out.dtype or d.stride(0) != out.stride(0):
            raise _l.CutHipError("matmul: binary epilogue needs D with the shape, dtype and stride of C")
        epi, op, dptr = _l.EPI_BINARY, _l.BINARY[binary], d.data_ptr()
    _l.check(_l.load().cuthip_matmul_gguf(
        f, w_blocks.data_ptr(), a2.data_ptr(), _l.F16 if a2.dtype == torch.float16 else _l.F32, out.data_ptr(),
        _l.F16 if out.dtype == torch.float16 else _l.F32, M, K, N, a2.stride(0), out.stride(0), epi, op, dptr,
        variant, _stream_ptr()))
    return out if a.dim() == 2 else out
