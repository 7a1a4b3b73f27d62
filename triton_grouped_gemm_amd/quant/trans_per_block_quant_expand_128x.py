"""Per-128x128-block FP8 quantiser that also transposes and pads every expert to 128 tokens.

Mirror of quant/trans_per_block_quant_expand_128x.py:135-213.  One streaming HIP kernel reads
each 128x128 bf16 block once (rows past an expert's end count as zero), computes
``scale = clamp(amax / fmax, 1e-12, 3e38)`` and ``q = fp8(clamp(x / scale, -fmax, fmax))`` in
IEEE fp32, transposes through LDS and writes 128-byte rows of codes; the tail up to
``M_EXPAND`` gets zero codes and zero scales.
"""
from __future__ import annotations

from typing import Tuple

import torch

from .. import _native
from ..gemm.BF16.m_grouped_gemm import _sizes_on_device


def trans_per_block_quant_expand_128x(input_tensor: torch.Tensor, size_per_group: torch.Tensor,
                                      group_size: int = 128, dtype: torch.dtype = torch.float8_e4m3fn
                                      ) -> Tuple[torch.Tensor, torch.Tensor, torch.Tensor]:
    """input ``[M, N]`` bf16 -> (codes ``[N, M_EXPAND]``, scales ``[N/128, M_EXPAND/128]`` fp32,
    per-expert sizes rounded up to 128) with ``M_EXPAND = M + 128*G - M % 128``."""
    assert input_tensor.dim() == 2
    M, N = input_tensor.shape
    assert group_size == 128, "only group_size=128 is implemented"
    assert N % group_size == 0
    assert input_tensor.dtype == torch.bfloat16, f"data type {input_tensor.dtype} not supported"
    assert dtype in _native.FP8_CODE, f"data type {dtype} not supported"
    num_experts = size_per_group.shape[0]
    assert size_per_group.dim() == 1 and 1 <= num_experts <= _native.MAX_GROUPS
    _native.require_gpu(input_tensor)
    assert input_tensor.is_contiguous(), "input_tensor must be contiguous"
    sizes, is64 = _sizes_on_device(size_per_group, input_tensor.device)
    size_per_group_padding = torch.div(sizes + (group_size - 1), group_size, rounding_mode="floor") * group_size
    M_EXPAND = M + group_size * num_experts - M % group_size
    output_tensor = input_tensor.new_empty((N, M_EXPAND), dtype=dtype)
    output_scales = input_tensor.new_empty((N // group_size, M_EXPAND // group_size), dtype=torch.float32)
    _native.call("tgg_trans_per_block_quant_expand_128x", input_tensor.data_ptr(), output_tensor.data_ptr(),
                 output_scales.data_ptr(), sizes.data_ptr(), is64, num_experts, M, N, M_EXPAND,
                 _native.FP8_CODE[dtype], _native.stream_of(input_tensor))
    return output_tensor, output_scales, size_per_group_padding


def trans_quant(input_tensor: torch.Tensor, size_per_group: torch.Tensor):
    return trans_per_block_quant_expand_128x(input_tensor, size_per_group)
