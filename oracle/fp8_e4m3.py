"""OCP FP8 E4M3 ("e4m3fn": no infinities, one NaN code per sign) in integer numpy.

Test infrastructure only (see ``oracle/__init__.py``).

The reference's hot path has no FP8 KV; the only FP8 code in its tree is the
vLLM-derived legacy prefix-prefill kernel, whose convention is
``dequant = fp8.to(float32) * scale`` with one scalar scale per tensor
(diffulex_legacy/layers/attention/ops/prefix_prefill.py:126-129,166-169).
This file fixes the matching quantiser used by this build:

    code = RNE_e4m3fn( clamp( float32(x) / scale[h], -448, +448 ) )

with a true fp32 division (not a reciprocal multiply), one fp32 scale per KV
head, K and V separately.
"""
from __future__ import annotations

import numpy as np

E4M3_MAX = 448.0


def encode_e4m3fn(x: np.ndarray) -> np.ndarray:
    """Round-to-nearest-even float32 -> e4m3fn code (uint8).

    Values whose magnitude rounds above 448 become NaN (0x7f | sign), as the
    library cast does; callers that want saturation clamp first.
    """
    x = np.ascontiguousarray(x, dtype=np.float32)
    bits = x.view(np.uint32)
    sign = ((bits >> 24) & 0x80).astype(np.uint8)
    mag = bits & 0x7FFFFFFF
    out = np.zeros(x.shape, dtype=np.uint32)

    is_nan = mag > 0x7F800000
    # smallest fp32 magnitude that is a *normal* e4m3 number: 2**-6
    normal = mag >= np.uint32(np.float32(2.0 ** -6).view(np.uint32))

    # normal range: keep 3 mantissa bits, round half to even on the 20 dropped
    lsb = (mag >> 20) & 1
    rounded = (mag.astype(np.uint64) + 0x7FFFF + lsb) >> 20  # exp8<<3 | m3
    code_n = rounded.astype(np.int64) - ((127 - 7) << 3)
    over = code_n > 0x7E  # 0x7e == 448, 0x7f is NaN
    code_n = np.where(over, 0x7F, code_n)

    # subnormal range: multiples of 2**-9; scaling by 512 is exact in fp32
    mag_f = np.where(normal, np.float32(0), mag.view(np.float32))
    code_d = np.rint(mag_f.astype(np.float64) * 512.0).astype(np.int64)  # 0..8

    out = np.where(normal, code_n, code_d).astype(np.uint8)
    out = np.where(is_nan, np.uint8(0x7F), out)
    return (out | sign).astype(np.uint8)


def decode_e4m3fn(code: np.ndarray) -> np.ndarray:
    """e4m3fn code (uint8) -> float32 (exact)."""
    code = np.asarray(code, dtype=np.uint8)
    sign = np.where(code & 0x80, -1.0, 1.0).astype(np.float32)
    e = ((code >> 3) & 0xF).astype(np.int32)
    m = (code & 0x7).astype(np.int32)
    sub = m.astype(np.float32) * np.float32(2.0 ** -9)
    nor = (8 + m).astype(np.float32) * np.exp2((e - 10).astype(np.float32))
    val = np.where(e == 0, sub, nor).astype(np.float32)
    val = np.where((e == 15) & (m == 7), np.float32(np.nan), val)
    return (sign * val).astype(np.float32)


def quantize_per_head(x_f32: np.ndarray, scale: np.ndarray) -> np.ndarray:
    """x: [..., H, hd] float32 (the exact value of a bf16 tensor), scale: [H] float32."""
    x = np.asarray(x_f32, dtype=np.float32)
    s = np.asarray(scale, dtype=np.float32).reshape((1,) * (x.ndim - 2) + (-1, 1))
    with np.errstate(invalid="ignore", divide="ignore", over="ignore"):
        y = (x / s).astype(np.float32)  # IEEE fp32 division
        y = np.where(np.isnan(y), y, np.clip(y, np.float32(-E4M3_MAX), np.float32(E4M3_MAX)))
    return encode_e4m3fn(y.astype(np.float32))


def dequantize_per_head(code: np.ndarray, scale: np.ndarray) -> np.ndarray:
    """code: [..., H, hd] uint8 -> float32 = decode(code) * scale[h]."""
    v = decode_e4m3fn(code)
    s = np.asarray(scale, dtype=np.float32).reshape((1,) * (v.ndim - 2) + (-1, 1))
    return (v * s).astype(np.float32)


def amax_scale(x_f32: np.ndarray) -> np.ndarray:
    """Per-KV-head scale amax_h / 448 over a [..., H, hd] tensor (fp32)."""
    x = np.asarray(x_f32, dtype=np.float32)
    red = tuple(i for i in range(x.ndim) if i != x.ndim - 2)
    amax = np.max(np.abs(x), axis=red).astype(np.float32)
    return (amax / np.float32(E4M3_MAX)).astype(np.float32)
