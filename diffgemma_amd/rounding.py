"""Storage rounding conventions, as numpy bit operations.

The reference rounds by truncation on the host (src/shaders/common/bf16.rs:9-11,
src/shaders/common/f16.rs:28-47: clamp to +-65504, flush subnormals, mantissa >> 13) and
its bf16 arena store truncates too (src/shaders/include/common.metal:16-18).  The HIP
kernels round to nearest even unless asked to truncate.
"""
from __future__ import annotations

import numpy as np


def f32_to_bf16_bits_trunc(x: np.ndarray) -> np.ndarray:
    u = np.ascontiguousarray(x, dtype=np.float32).view(np.uint32)
    return (u >> 16).astype(np.uint16)


def f32_to_bf16_bits_rne(x: np.ndarray) -> np.ndarray:
    u = np.ascontiguousarray(x, dtype=np.float32).view(np.uint32)
    nan = (u & np.uint32(0x7FFFFFFF)) > np.uint32(0x7F800000)
    with np.errstate(over="ignore"):  # only NaN patterns can wrap, and those are replaced below
        r = (u + np.uint32(0x7FFF) + ((u >> np.uint32(16)) & np.uint32(1))) >> np.uint32(16)
    if nan.any():
        r = np.where(nan, (u >> np.uint32(16)) | np.uint32(0x40), r)
    return r.astype(np.uint16)


def bf16_bits_to_f32(b: np.ndarray) -> np.ndarray:
    return (np.ascontiguousarray(b, dtype=np.uint16).astype(np.uint32) << 16).view(np.float32)


def f32_to_f16_bits_trunc(x: np.ndarray) -> np.ndarray:
    """Reference host conversion: clamp, flush subnormals to signed zero, truncate."""
    v = np.ascontiguousarray(x, dtype=np.float32)
    c = np.where(np.isnan(v), v, np.clip(v, -65504.0, 65504.0)).astype(np.float32)
    bits = c.view(np.uint32)
    sign = ((bits >> 16) & 0x8000).astype(np.uint32)
    exp = ((bits >> 23) & 0xFF).astype(np.int64)
    mant = bits & 0x7FFFFF
    new_exp = exp - 127 + 15
    out = sign | (np.clip(new_exp, 0, 0x1F).astype(np.uint32) << 10) | (mant >> 13)
    out = np.where(new_exp >= 0x1F, sign | 0x7C00, out)
    out = np.where(new_exp <= 0, sign, out)
    out = np.where(exp == 0, sign, out)
    out = np.where(exp == 0xFF, sign | np.where(mant == 0, 0, 0x7E00).astype(np.uint32), out)
    return out.astype(np.uint16)


def f32_to_f16_bits_rne(x: np.ndarray) -> np.ndarray:
    with np.errstate(over="ignore"):
        return np.ascontiguousarray(x, dtype=np.float32).astype(np.float16).view(np.uint16)


def f16_bits_to_f32(b: np.ndarray) -> np.ndarray:
    return np.ascontiguousarray(b, dtype=np.uint16).view(np.float16).astype(np.float32)


def to_bits(x: np.ndarray, dtype: str, truncate: bool) -> np.ndarray:
    if dtype == "bf16":
        return f32_to_bf16_bits_trunc(x) if truncate else f32_to_bf16_bits_rne(x)
    if dtype == "f16":
        return f32_to_f16_bits_trunc(x) if truncate else f32_to_f16_bits_rne(x)
    raise ValueError(dtype)


def from_bits(b: np.ndarray, dtype: str) -> np.ndarray:
    return bf16_bits_to_f32(b) if dtype == "bf16" else f16_bits_to_f32(b)
