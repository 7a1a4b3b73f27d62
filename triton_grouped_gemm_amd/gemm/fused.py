"""M-grouped GEMM with the 1x128 FP8 quantisation of its output fused into the epilogue.

In an FP8 MoE layer the first expert GEMM's output is quantised (``per_token_cast_to_fp8``,
gemm/FP8/m_grouped_gemm_channel_expert.py:217-222) before it enters the block-scaled second GEMM
(gemm/deep_gemm_ops.py:60-100).  ``m_grouped_gemm_fp8_out`` produces exactly the bits of

    per_token_cast_to_fp8(m_grouped_gemm(A, B, size_per_group, trans_b), dtype, scales_mn_major)

without writing and re-reading the 16-bit intermediate.  Shapes the fused kernel does not take run as those two
launches.
"""
from typing import Tuple

import torch

from .. import _native
from ..quant.fp8_cast import per_token_cast_to_fp8
from .BF16.m_grouped_gemm import _sizes_on_device, m_grouped_gemm

MAX_FUSED_GROUPS = 512


def m_grouped_gemm_fp8_out(A: torch.Tensor, B: torch.Tensor, size_per_group: torch.Tensor, trans_b: bool = False,
                           dtype: torch.dtype = torch.float8_e4m3fn, scales_mn_major: bool = False,
                           numSM: int = -1) -> Tuple[torch.Tensor, torch.Tensor]:
    """Returns ``(codes [M, N] fp8, scales [M, N/128] fp32)``; rows past ``sum(size_per_group)`` are left
    uninitialised in both, as in ``m_grouped_gemm``."""
    assert A.dim() == 2 and B.dim() == 3, "A must be [M, K] and B [G, N, K] or [G, K, N]"
    assert A.dtype == torch.bfloat16 and B.dtype == A.dtype, f"data type {A.dtype} not supported"
    M, K = A.shape
    G = B.shape[0]
    N = B.shape[1] if trans_b else B.shape[2]
    assert (B.shape[2] if trans_b else B.shape[1]) == K, "K of A and B must match"
    assert N % 128 == 0, "N must be a multiple of 128 (whole 1x128 quantisation groups)"
    assert size_per_group.numel() == G
    _native.require_gpu(A, B)
    fused = G <= MAX_FUSED_GROUPS and K % 8 == 0 and K * 512 < 2 ** 30 and N * 128 < 2 ** 30
    if not fused:
        return per_token_cast_to_fp8(m_grouped_gemm(A, B, size_per_group, trans_b, numSM), dtype, scales_mn_major)
    A, B = A.contiguous(), B.contiguous()
    codes = torch.empty((M, N), device=A.device, dtype=dtype)
    if scales_mn_major:
        scales = torch.empty((N // 128, M), device=A.device, dtype=torch.float32).t()
    else:
        scales = torch.empty((M, N // 128), device=A.device, dtype=torch.float32)
    sizes, is64 = _sizes_on_device(size_per_group, A.device)
    _native.call("tgg_m_grouped_gemm_fp8_out", A.data_ptr(), B.data_ptr(), codes.data_ptr(), scales.data_ptr(),
                 sizes.data_ptr(), is64, G, M, N, K, int(bool(trans_b)), _native.DTYPE_CODE[A.dtype],
                 _native.FP8_CODE[dtype], int(scales_mn_major), int(numSM), _native.stream_of(A))
    return codes, scales
