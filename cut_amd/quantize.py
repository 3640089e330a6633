"""Host-side (numpy) encoders producing GGUF blocks from fp32 weights.

Q8_0 follows the reference's ``quantizeRowsQ8_0`` (interface/runner/llama/
llama.cpp:488-505: d = amax/127, q = round-half-away(x * (1/d)), stored scale
narrowed with round-half-away).  The reference has no encoder for Q4_0, Q4_K
and Q6_K; the ones here are simple min/max fits that produce valid blocks for
synthetic weights (benchmarks, examples).  Decoding is defined over the block
bytes alone, so any valid encoder serves.
"""
from __future__ import annotations

import numpy as np


def f32_to_f16_bits(x: np.ndarray) -> np.ndarray:
    """fp32 -> binary16 bits, round half away from zero, subnormals kept,
    overflow and NaN -> +-Inf (the host narrowing of llama.cpp:445-482)."""
    x = np.ascontiguousarray(x, np.float32)
    u = x.view(np.uint32)
    sign = ((u >> 16) & 0x8000).astype(np.uint16)
    # setting the lowest mantissa bit breaks every tie upward in magnitude and
    # moves no other value across a rounding boundary; then round to nearest even
    with np.errstate(over="ignore", invalid="ignore"):
        h = (u | np.uint32(1)).view(np.float32).astype(np.float16).view(np.uint16)
    nonfinite = (u & 0x7F800000) == 0x7F800000
    return np.where(nonfinite, sign | np.uint16(0x7C00), h).astype(np.uint16)


def _round_half_away(v: np.ndarray) -> np.ndarray:
    return np.where(v >= 0, np.floor(v + np.float32(0.5)), np.ceil(v - np.float32(0.5)))


def quantize_q8_0(x: np.ndarray) -> np.ndarray:
    xb = np.ascontiguousarray(x, np.float32).reshape(-1, 32)
    amax = np.abs(xb).max(axis=1)
    d = (amax / np.float32(127.0)).astype(np.float32)
    inv = np.where(d != 0, np.float32(1.0) / np.where(d != 0, d, np.float32(1)), np.float32(0)).astype(np.float32)
    prod = (xb * inv[:, None]).astype(np.float32)
    q = _round_half_away(prod.astype(np.float64)).astype(np.int8)
    out = np.empty((xb.shape[0], 34), np.uint8)
    out[:, 0:2] = f32_to_f16_bits(d).view(np.uint8).reshape(-1, 2)
    out[:, 2:] = q.view(np.uint8)
    return out.reshape(-1)


def quantize_q4_0(x: np.ndarray) -> np.ndarray:
    xb = np.ascontiguousarray(x, np.float32).reshape(-1, 32)
    idx = np.abs(xb).argmax(axis=1)
    mx = xb[np.arange(xb.shape[0]), idx]
    d = (mx / np.float32(-8.0)).astype(np.float32)
    inv = np.where(d != 0, np.float32(1.0) / np.where(d != 0, d, np.float32(1)), np.float32(0)).astype(np.float32)
    q = np.clip((xb * inv[:, None] + np.float32(8.5)).astype(np.int32), 0, 15).astype(np.uint8)
    out = np.empty((xb.shape[0], 18), np.uint8)
    out[:, 0:2] = f32_to_f16_bits(d).view(np.uint8).reshape(-1, 2)
    out[:, 2:] = q[:, :16] | (q[:, 16:] << 4)
    return out.reshape(-1)


def _f16_bits_to_f32(h: np.ndarray) -> np.ndarray:
    return h.view(np.float16).astype(np.float32)


def quantize_q4_k(x: np.ndarray) -> np.ndarray:
    xb = np.ascontiguousarray(x, np.float32).reshape(-1, 8, 32)
    nb = xb.shape[0]
    lo = np.minimum(xb.min(axis=2), 0.0).astype(np.float32)
    hi = xb.max(axis=2)
    scales = ((hi - lo) / np.float32(15.0)).astype(np.float32)
    mins = (-lo).astype(np.float32)
    max_scale, max_min = scales.max(axis=1), mins.max(axis=1)
    dh = f32_to_f16_bits((max_scale / np.float32(63.0)).astype(np.float32))
    dmh = f32_to_f16_bits((max_min / np.float32(63.0)).astype(np.float32))
    inv_s = np.where(max_scale > 0, np.float32(63.0) / np.where(max_scale > 0, max_scale, 1), 0).astype(np.float32)
    inv_m = np.where(max_min > 0, np.float32(63.0) / np.where(max_min > 0, max_min, 1), 0).astype(np.float32)
    ls = np.minimum(np.rint(inv_s[:, None] * scales), 63).astype(np.uint8)
    lm = np.minimum(np.rint(inv_m[:, None] * mins), 63).astype(np.uint8)
    d, dmin = _f16_bits_to_f32(dh), _f16_bits_to_f32(dmh)
    dj = (d[:, None] * ls.astype(np.float32)).astype(np.float32)
    mj = (dmin[:, None] * lm.astype(np.float32)).astype(np.float32)
    with np.errstate(divide="ignore", invalid="ignore"):
        q = np.where(dj[:, :, None] != 0, np.rint((xb + mj[:, :, None]) / dj[:, :, None]), 0)
    L = np.clip(q, 0, 15).astype(np.uint8)
    out = np.zeros((nb, 144), np.uint8)
    out[:, 0:2] = dh.view(np.uint8).reshape(-1, 2)
    out[:, 2:4] = dmh.view(np.uint8).reshape(-1, 2)
    sc = out[:, 4:16]
    sc[:, 0:4] = ls[:, 0:4] | ((ls[:, 4:8] >> 4) << 6)
    sc[:, 4:8] = lm[:, 0:4] | ((lm[:, 4:8] >> 4) << 6)
    sc[:, 8:12] = (ls[:, 4:8] & 0xF) | ((lm[:, 4:8] & 0xF) << 4)
    Lg = L.reshape(nb, 4, 2, 32)
    out[:, 16:] = (Lg[:, :, 0, :] | (Lg[:, :, 1, :] << 4)).reshape(nb, 128)
    return out.reshape(-1)


def quantize_q6_k(x: np.ndarray) -> np.ndarray:
    xb = np.ascontiguousarray(x, np.float32).reshape(-1, 16, 16)
    nb = xb.shape[0]
    idx = np.abs(xb).argmax(axis=2)
    mx = np.take_along_axis(xb, idx[:, :, None], axis=2)[:, :, 0]
    scales = (mx / np.float32(-32.0)).astype(np.float32)
    j = np.abs(scales).argmax(axis=1)
    max_scale = scales[np.arange(nb), j]
    iscale = np.where(max_scale != 0, np.float32(-128.0) / np.where(max_scale != 0, max_scale, 1), 0).astype(np.float32)
    dh = f32_to_f16_bits(np.where(iscale != 0, np.float32(1.0) / np.where(iscale != 0, iscale, 1), 0).astype(np.float32))
    sc = np.clip(np.rint(iscale[:, None] * scales), -128, 127).astype(np.int8)
    d = _f16_bits_to_f32(dh)
    dj = (d[:, None] * sc.astype(np.float32)).astype(np.float32)
    with np.errstate(divide="ignore", invalid="ignore"):
        q = np.where(dj[:, :, None] != 0, np.rint(xb / dj[:, :, None]), 0)
    L = (np.clip(q, -32, 31) + 32).astype(np.uint8).reshape(nb, 2, 4, 32)  # [H][s][l]
    out = np.zeros((nb, 210), np.uint8)
    ql = out[:, 0:128].reshape(nb, 2, 2, 32)  # [H][sigma][l]
    ql[:, :, 0, :] = (L[:, :, 0, :] & 0xF) | ((L[:, :, 2, :] & 0xF) << 4)
    ql[:, :, 1, :] = (L[:, :, 1, :] & 0xF) | ((L[:, :, 3, :] & 0xF) << 4)
    out[:, 128:192] = ((L[:, :, 0, :] >> 4) | ((L[:, :, 1, :] >> 4) << 2) | ((L[:, :, 2, :] >> 4) << 4) |
                       ((L[:, :, 3, :] >> 4) << 6)).reshape(nb, 64)
    out[:, 192:208] = sc.view(np.uint8)
    out[:, 208:210] = dh.view(np.uint8).reshape(-1, 2)
    return out.reshape(-1)


_ENCODERS = {0: quantize_q8_0, 1: quantize_q4_0, 2: quantize_q4_k, 3: quantize_q6_k}
_NAMES = {"Q8_0": 0, "Q4_0": 1, "Q4_K": 2, "Q6_K": 3}


def quantize(fmt, x: np.ndarray) -> np.ndarray:
    """fmt: 0..3 or 'Q8_0' | 'Q4_0' | 'Q4_K' | 'Q6_K'; x: fp32, size a multiple of the block."""
    f = _NAMES[fmt] if isinstance(fmt, str) else int(fmt)
    return _ENCODERS[f](x)
