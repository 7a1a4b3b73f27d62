"""Software OCP FP8 encoders/decoders in numpy integer arithmetic (test oracle).

The reference relies on ``Tensor.to(torch.float8_e4m3fn)`` /
``Tensor.to(torch.float8_e5m2)`` (gemm/FP8/m_grouped_gemm_channel_expert.py:217-261,
quant/trans_per_block_quant_expand_128x.py:216-219): round-to-nearest-even,
non-saturating (e4m3fn overflow -> NaN 0x7F, e5m2 overflow -> inf 0x7C).
These functions restate that conversion from the bit layout of the formats so
the HIP quantizers can be checked bit for bit without trusting a library cast.
"""
from __future__ import annotations

import numpy as np


def _f32_bits(x: np.ndarray) -> np.ndarray:
    return np.ascontiguousarray(x, dtype=np.float32).view(np.uint32)


def encode_e4m3fn(x: np.ndarray) -> np.ndarray:
    """fp32 -> e4m3fn code (uint8). RNE; |x| that rounds above 448 -> NaN (0x7F)."""
    bits = _f32_bits(x)
    sign = ((bits >> 24) & 0x80).astype(np.uint8)
    mag = bits & np.uint32(0x7FFFFFFF)
    absx = mag.view(np.float32)
    nan = mag > np.uint32(0x7F800000)
    # normal range of the target: |x| >= 2^-6
    lsb = (mag >> 20) & np.uint32(1)
    rounded = mag.astype(np.uint64) + np.uint64(0x7FFFF) + lsb.astype(np.uint64)
    exp = (rounded >> np.uint64(23)).astype(np.int64) - 127 + 7
    man = ((rounded >> np.uint64(20)) & np.uint64(7)).astype(np.int64)
    code_norm = (exp << 3) | man
    # subnormal range: multiples of 2^-9, RNE on the exact quotient
    code_sub = np.rint(absx.astype(np.float64) * 512.0).astype(np.int64)
    is_sub = absx < np.float32(2.0 ** -6)
    code = np.where(is_sub, code_sub, code_norm)
    code = np.where((code > 0x7E) | nan, 0x7F, code)
    return (code.astype(np.uint8) | sign).astype(np.uint8)


def decode_e4m3fn(code: np.ndarray) -> np.ndarray:
    c = np.asarray(code, dtype=np.uint8).astype(np.int64)
    sign = np.where(c & 0x80, -1.0, 1.0)
    e = (c >> 3) & 0xF
    m = c & 7
    val = np.where(e == 0, m * 2.0 ** -9, (8 + m) * np.exp2((e - 10).astype(np.float64)))
    val = np.where((c & 0x7F) == 0x7F, np.nan, val)
    return (sign * val).astype(np.float32)


def encode_e5m2(x: np.ndarray) -> np.ndarray:
    """fp32 -> e5m2 code (uint8). RNE; finite overflow -> inf (0x7C), NaN -> 0x7F."""
    bits = _f32_bits(x)
    sign = ((bits >> 24) & 0x80).astype(np.uint8)
    mag = bits & np.uint32(0x7FFFFFFF)
    absx = mag.view(np.float32)
    nan = mag > np.uint32(0x7F800000)
    lsb = (mag >> 21) & np.uint32(1)
    rounded = mag.astype(np.uint64) + np.uint64(0xFFFFF) + lsb.astype(np.uint64)
    exp = (rounded >> np.uint64(23)).astype(np.int64) - 127 + 15
    man = ((rounded >> np.uint64(21)) & np.uint64(3)).astype(np.int64)
    code_norm = (exp << 2) | man
    with np.errstate(over="ignore", invalid="ignore"):
        code_sub = np.rint(np.minimum(absx.astype(np.float64), 1.0) * 65536.0).astype(np.int64)
    is_sub = absx < np.float32(2.0 ** -14)
    code = np.where(is_sub, code_sub, code_norm)
    code = np.where(code > 0x7C, 0x7C, code)
    code = np.where(nan, 0x7F, code)
    return (code.astype(np.uint8) | sign).astype(np.uint8)


def decode_e5m2(code: np.ndarray) -> np.ndarray:
    c = np.asarray(code, dtype=np.uint8).astype(np.int64)
    sign = np.where(c & 0x80, -1.0, 1.0)
    e = (c >> 2) & 0x1F
    m = c & 3
    val = np.where(e == 0, m * 2.0 ** -16, (4 + m) * np.exp2((e - 17).astype(np.float64)))
    val = np.where(e == 31, np.where(m == 0, np.inf, np.nan), val)
    return (sign * val).astype(np.float32)


def bf16_bits_to_f32(bits16: np.ndarray) -> np.ndarray:
    """uint16 bf16 bit patterns -> float32 values (exact)."""
    return (np.asarray(bits16, dtype=np.uint16).astype(np.uint32) << 16).view(np.float32)


def f32_to_bf16_bits(x: np.ndarray) -> np.ndarray:
    """float32 -> bf16 bit patterns, round-to-nearest-even (NaN kept quiet)."""
    bits = _f32_bits(x)
    lsb = (bits >> 16) & np.uint32(1)
    rounded = (bits.astype(np.uint64) + np.uint64(0x7FFF) + lsb.astype(np.uint64)) >> np.uint64(16)
    out = rounded.astype(np.uint16)
    nan = (bits & np.uint32(0x7FFFFFFF)) > np.uint32(0x7F800000)
    return np.where(nan, ((bits >> 16) | 0x40).astype(np.uint16), out)
