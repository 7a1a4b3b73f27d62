"""numpy restatement of the reference's FP8 quantizers (test oracle).

All arithmetic is done in IEEE fp32 with numpy scalars/arrays so that the HIP
kernels can be compared bit for bit.  Inputs are float32 arrays that hold
bf16-representable values (the reference quantizes bf16 tensors).

Follows:
* quant/trans_per_block_quant_expand_128x.py:91-131,159-208 (kernel semantics:
  scale clamped to [1e-12, 3e38], rows beyond a group's end read as zero,
  tail columns up to M_EXPAND zero) and its torch oracle :216-273
  (``scale = amax.float()/fmax``; ``to_fp8_saturated(x / scale)``).
* gemm/FP8/m_grouped_gemm_channel_expert.py:217-222 (``per_token_cast_to_fp8``)
  and :237-245 (``per_block_cast_to_fp8``).
"""
from __future__ import annotations

import numpy as np

from . import fp8_soft

_F32 = np.float32
_FMAX = {"e4m3fn": _F32(448.0), "e5m2": _F32(57344.0)}
_ENC = {"e4m3fn": fp8_soft.encode_e4m3fn, "e5m2": fp8_soft.encode_e5m2}


def _rdiv(scalar, t: np.ndarray) -> np.ndarray:
    """``python_float / tensor`` as torch evaluates it: ``tensor.reciprocal() * scalar`` -- two fp32
    roundings, not one division (the recipes' ``448.0 / x_amax``)."""
    return ((_F32(1.0) / t).astype(_F32) * _F32(scalar)).astype(_F32)


def m_expand(M: int, G: int, group_size: int = 128) -> int:
    """quant/trans_per_block_quant_expand_128x.py:172."""
    return M + group_size * G - M % group_size


def trans_per_block_quant_expand_128x(x: np.ndarray, sizes, fmt: str = "e4m3fn"):
    """Returns (codes uint8 [N, M_EXPAND], scales f32 [N/128, M_EXPAND/128], padded sizes)."""
    x = np.asarray(x, dtype=_F32)
    M, N = x.shape
    assert N % 128 == 0
    sizes = [int(s) for s in sizes]
    G = len(sizes)
    ME = m_expand(M, G)
    fmax = _FMAX[fmt]
    enc = _ENC[fmt]
    codes = np.zeros((N, ME), dtype=np.uint8)
    scales = np.zeros((N // 128, ME // 128), dtype=_F32)
    padded = [(s + 127) // 128 * 128 for s in sizes]
    src = 0
    dst = 0
    for size, pad in zip(sizes, padded):
        for bm in range(pad // 128):
            r0 = src + bm * 128
            r1 = min(r0 + 128, src + size)
            blk_rows = np.zeros((128, N), dtype=_F32)
            blk_rows[: r1 - r0] = x[r0:r1]
            for bn in range(N // 128):
                blk = blk_rows[:, bn * 128:(bn + 1) * 128]
                amax = _F32(np.max(np.abs(blk)))
                scale = _F32(amax / fmax)
                scale = _F32(min(max(scale, _F32(1e-12)), _F32(3e38)))
                q = np.clip((blk / scale).astype(_F32), -fmax, fmax)
                codes[bn * 128:(bn + 1) * 128, dst + bm * 128: dst + (bm + 1) * 128] = enc(q).T
                scales[bn, (dst + bm * 128) // 128] = scale
        src += size
        dst += pad
    return codes, scales, np.asarray(padded, dtype=np.int64)


def per_token_cast_to_fp8(x: np.ndarray, fmt: str = "e4m3fn"):
    """1x128 recipe: codes uint8 [M, K], scales f32 [M, K/128]."""
    x = np.asarray(x, dtype=_F32)
    M, K = x.shape
    assert K % 128 == 0
    fmax = _FMAX[fmt]
    v = x.reshape(M, K // 128, 128)
    amax = np.maximum(np.max(np.abs(v), axis=2), _F32(1e-4)).astype(_F32)
    mult = _rdiv(fmax, amax)
    prod = (v * mult[:, :, None]).astype(_F32)
    return _ENC[fmt](prod).reshape(M, K), (amax / fmax).astype(_F32)


def per_block_cast_to_fp8(x: np.ndarray, fmt: str = "e4m3fn"):
    """128x128 recipe: codes uint8 [M, N], scales f32 [ceil(M/128), ceil(N/128)]."""
    x = np.asarray(x, dtype=_F32)
    M, N = x.shape
    Mp, Np = (M + 127) // 128 * 128, (N + 127) // 128 * 128
    fmax = _FMAX[fmt]
    xp = np.zeros((Mp, Np), dtype=_F32)
    xp[:M, :N] = x
    v = xp.reshape(Mp // 128, 128, Np // 128, 128)
    amax = np.maximum(np.max(np.abs(v), axis=(1, 3), keepdims=True), _F32(1e-4)).astype(_F32)
    prod = (v * _rdiv(fmax, amax)).astype(_F32)
    codes = _ENC[fmt](prod).reshape(Mp, Np)[:M, :N]
    return np.ascontiguousarray(codes), (amax / fmax).astype(_F32).reshape(Mp // 128, Np // 128)


def per_row_cast_to_fp8(x: np.ndarray, fmt: str = "e4m3fn"):
    """Whole-row ("per channel") recipe, m_grouped_gemm_channel_expert.py:224-234."""
    x = np.asarray(x, dtype=_F32)
    fmax = _FMAX[fmt]
    amax = np.maximum(np.max(np.abs(x), axis=1, keepdims=True), _F32(1e-4)).astype(_F32)
    prod = (x * _rdiv(fmax, amax)).astype(_F32)
    return _ENC[fmt](prod), (amax / fmax).astype(_F32)


def per_expert_cast_to_fp8(x: np.ndarray, fmt: str = "e4m3fn"):
    """One scale per expert matrix, m_grouped_gemm_channel_expert.py:247-261. x: [G, N, K]."""
    x = np.asarray(x, dtype=_F32)
    fmax = _FMAX[fmt]
    amax = np.maximum(np.max(np.abs(x), axis=(1, 2), keepdims=True), _F32(1e-4)).astype(_F32)
    prod = (x * _rdiv(fmax, amax)).astype(_F32)
    return _ENC[fmt](prod), (amax / fmax).astype(_F32).reshape(-1, 1)


def dequant(codes: np.ndarray, fmt: str = "e4m3fn") -> np.ndarray:
    return (fp8_soft.decode_e4m3fn if fmt == "e4m3fn" else fp8_soft.decode_e5m2)(codes)
