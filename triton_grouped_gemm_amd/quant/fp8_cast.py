"""GPU versions of the reference's FP8 cast recipes
(gemm/FP8/m_grouped_gemm_channel_expert.py:217-245): ``amax.clamp(1e-4)``, codes
``fp8(x * (fmax / amax))``, scales ``amax / fmax``, all in IEEE fp32."""
from __future__ import annotations

from typing import Tuple

import torch

from .. import _native


def per_token_cast_to_fp8(x: torch.Tensor, dtype: torch.dtype = torch.float8_e4m3fn,
                          scales_mn_major: bool = False) -> Tuple[torch.Tensor, torch.Tensor]:
    """1x128 groups along the last dim: x ``[M, K]`` bf16 -> (codes ``[M, K]``, scales ``[M, K/128]``).
    With ``scales_mn_major`` the scales keep that shape but are stored K-block-major (strides ``(1, M)``),
    the layout the block-scaled GEMM consumes without a copy."""
    assert x.dim() == 2 and x.size(1) % 128 == 0
    assert x.dtype == torch.bfloat16, f"data type {x.dtype} not supported"
    _native.require_gpu(x)
    x = x.contiguous()
    m, k = x.shape
    codes = torch.empty((m, k), device=x.device, dtype=dtype)
    if scales_mn_major:
        scales = torch.empty((k // 128, m), device=x.device, dtype=torch.float32).t()
    else:
        scales = torch.empty((m, k // 128), device=x.device, dtype=torch.float32)
    _native.call("tgg_per_token_cast_to_fp8", x.data_ptr(), codes.data_ptr(), scales.data_ptr(), m, k,
                 _native.FP8_CODE[dtype], int(scales_mn_major), _native.stream_of(x))
    return codes, scales


def per_block_cast_to_fp8(x: torch.Tensor, dtype: torch.dtype = torch.float8_e4m3fn) -> Tuple[torch.Tensor, torch.Tensor]:
    """128x128 blocks: x ``[R, C]`` (or a batch ``[G, R, C]``) bf16 -> (codes of the same shape,
    scales ``[ceil(R/128), ceil(C/128)]`` (with a leading G for a batch))."""
    assert x.dim() in (2, 3)
    assert x.dtype == torch.bfloat16, f"data type {x.dtype} not supported"
    _native.require_gpu(x)
    x = x.contiguous()
    batch = 1 if x.dim() == 2 else x.shape[0]
    r, c = x.shape[-2:]
    codes = torch.empty(x.shape, device=x.device, dtype=dtype)
    sshape = ((r + 127) // 128, (c + 127) // 128)
    scales = torch.empty(sshape if x.dim() == 2 else (batch, *sshape), device=x.device, dtype=torch.float32)
    _native.call("tgg_per_block_cast_to_fp8", x.data_ptr(), codes.data_ptr(), scales.data_ptr(), batch, r, c,
                 _native.FP8_CODE[dtype], _native.stream_of(x))
    return codes, scales
