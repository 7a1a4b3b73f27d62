"""FP8 K-grouped (weight-gradient) GEMM with per-(row, expert) scales.

Mirror of ``matmul`` in gemm/FP8/k_grouped_gemm_channel_expert.py:143-181:
``out[g] = (x[:, seg_g] @ y[:, seg_g]^T) * x_scale[:, g] (x) y_scale[:, g]`` in bf16, where the
token segments are the prefix sums of ``tokens_per_expert`` (the caller pads every expert's
tokens to a multiple of 128 with zeros, as the reference requires).
"""
from __future__ import annotations

from typing import Optional

import torch
from torch import Tensor

from ... import _native

_FMT = {1: _native.E4M3, 2: _native.E5M2}


def _expert_major(scale: Tensor, rows: int, groups: int) -> Tensor:
    """fp32 buffer with element (row, g) at ``g*rows + row`` -- the layout the reference kernel
    indexes (:121-124) and its data generator produces (:262-266).  Zero-copy when the
    ``[rows, G]`` tensor already has strides ``(1, rows)``."""
    assert tuple(scale.shape) == (rows, groups), f"scale must have shape ({rows}, {groups})"
    s = scale.to(torch.float32)
    if s.stride() == (1, rows) or groups == 1:
        return s
    return s.t().contiguous().t()


def matmul(x_fp8: Tensor, x_scale: Tensor, y_fp8: Tensor, y_scale: Tensor, tokens_per_expert: Tensor,
           M: int, N: int, K: int, num_groups: int, dtype_a: int = 1, dtype_b: int = 1, *,
           queue: Optional[Tensor] = None) -> Tensor:
    """x ``[M, K]``, y ``[N, K]`` fp8 with the token dimension contiguous; dtype codes 1 = e4m3fn,
    anything else = e5m2 (reference :83-84).  Returns ``[num_groups, M, N]`` bf16.  ``queue`` (not in the
    reference): caller-owned tile counters, see ``k_grouped_gemm``."""
    assert x_fp8.dim() == 2 and tuple(x_fp8.shape) == (M, K), "x_fp8 must be [M, K]"
    assert y_fp8.dim() == 2 and tuple(y_fp8.shape) == (N, K), "y_fp8 must be [N, K]"
    assert x_fp8.element_size() == 1 and y_fp8.element_size() == 1, "x_fp8 and y_fp8 must hold 8-bit codes"
    assert tokens_per_expert.dim() == 1 and tokens_per_expert.shape[0] == num_groups
    assert 1 <= num_groups <= _native.MAX_GROUPS_OTHER, f"between 1 and {_native.MAX_GROUPS_OTHER} groups are supported"
    _native.require_gpu(x_fp8, x_scale, y_fp8, y_scale)
    assert x_fp8.is_contiguous() and y_fp8.is_contiguous(), "x_fp8 and y_fp8 must be contiguous"
    xs = _expert_major(x_scale, M, num_groups)
    ys = _expert_major(y_scale, N, num_groups)
    tokens = tokens_per_expert.to(device=x_fp8.device, dtype=torch.int32).contiguous()
    output = torch.empty((num_groups, M, N), dtype=torch.bfloat16, device=x_fp8.device)
    # tile-id counter of the kernel's work queue (a tile costs what its group has tokens; see include/tgg_amd.h)
    queue = _native.work_queue(x_fp8.device, queue)
    _native.call("tgg_k_grouped_gemm_fp8_channel_queued", x_fp8.data_ptr(), xs.data_ptr(), y_fp8.data_ptr(),
                 ys.data_ptr(), output.data_ptr(), tokens.data_ptr(), num_groups, M, N, K,
                 _FMT.get(int(dtype_a), _native.E5M2), _FMT.get(int(dtype_b), _native.E5M2), -1, queue.data_ptr(),
                 _native.stream_of(x_fp8))
    return output
