"""BF16/FP16 K-grouped (weight-gradient) GEMM: ``C[g] = A[s_g:e_g]^T @ B[s_g:e_g]``.

Mirror of gemm/BF16/k_grouped_gemm_TMA.py:183-294 (SM80 twin gemm/BF16/k_grouped_gemm.py:142-216).
An empty group yields a zero matrix (the TMA kernel's behaviour).  The native kernel has no
tile-divisibility requirement on M_DIM / N_DIM beyond 16-byte rows.
"""
from __future__ import annotations

from typing import Optional, Tuple

import torch
from torch import Tensor

from ... import _native


def _dtype_code(dtype: torch.dtype) -> int:
    code = _native.DTYPE_CODE.get(dtype, -1)
    assert code >= 0, f"data type {dtype} not supported"
    return code


def _check_k_grouped_gemm_inputs(A: Tensor, B: Tensor, size_per_group: Tensor, trans_b: bool = False
                                 ) -> Tuple[int, int, int, int]:
    """Same checks and messages as the reference (:183-214)."""
    assert not trans_b, \
        'trans_b=True path has been removed; pass B as contiguous [K_TOTAL, N_DIM] and trans_b=False'
    assert A.is_cuda and B.is_cuda and size_per_group.is_cuda, 'A, B, and size_per_group must be CUDA tensors'
    assert A.dim() == 2, 'A must be 2D'
    assert B.dim() == 2, 'B must be 2D'
    assert A.is_contiguous(), 'A must be contiguous [K_TOTAL, M_DIM]'
    assert B.is_contiguous(), 'B must be contiguous [K_TOTAL, N_DIM]'
    assert size_per_group.dim() == 1, 'size_per_group must be 1D'
    assert size_per_group.dtype in (torch.int32, torch.int64), 'size_per_group must be int32 or int64'
    K_TOTAL, M_DIM = A.shape
    K_B, N_DIM = B.shape
    assert K_TOTAL == K_B, f'A K_TOTAL={K_TOTAL} must equal B K_TOTAL={K_B}'
    _dtype_code(A.dtype)
    _dtype_code(B.dtype)
    assert A.dtype == B.dtype, f'A dtype {A.dtype} and B dtype {B.dtype} should match'
    assert A.data_ptr() % 16 == 0, 'A base pointer must be 16-byte aligned for TMA path'
    assert B.data_ptr() % 16 == 0, 'B base pointer must be 16-byte aligned for TMA path'
    assert (M_DIM * A.element_size()) % 16 == 0, 'A row stride must be 16-byte aligned for TMA path'
    assert (N_DIM * B.element_size()) % 16 == 0, 'B row stride must be 16-byte aligned for TMA path'
    return K_TOTAL, M_DIM, N_DIM, int(size_per_group.numel())


def k_grouped_gemm(A: Tensor, B: Tensor, size_per_group: Tensor, group_start: Optional[Tensor] = None,
                   group_end: Optional[Tensor] = None, trans_b: bool = False, numSM: int = -1,
                   use_fixed_sm90_config: bool = True, *, queue: Optional[Tensor] = None) -> Tensor:
    """A ``[K_TOTAL, M_DIM]``, B ``[K_TOTAL, N_DIM]`` -> C ``[G, M_DIM, N_DIM]`` (fp32 accumulation over
    the whole segment, one rounding to the input dtype).

    ``queue`` (not in the reference): the kernel's tile counters, ``_native.QUEUE_WORDS`` zeroed int32 on A's device
    that the caller owns -- for callers that must not allocate inside the call (graph capture); the kernel hands them
    back zeroed.  By default the library keeps one such tensor per device and stream."""
    K_TOTAL, M_DIM, N_DIM, num_groups = _check_k_grouped_gemm_inputs(A, B, size_per_group, trans_b)
    assert 1 <= num_groups <= _native.MAX_GROUPS, f"between 1 and {_native.MAX_GROUPS} groups are supported"
    C = A.new_empty(num_groups, M_DIM, N_DIM)
    if group_start is None or group_end is None:
        group_end = size_per_group.cumsum(0)
        group_start = group_end - size_per_group
    group_start = group_start.to(device=A.device, dtype=torch.int32).contiguous()
    group_end = group_end.to(device=A.device, dtype=torch.int32).contiguous()
    # tile-id counter of the kernel's work queue (a tile costs what its group has tokens; see include/tgg_amd.h)
    queue = _native.work_queue(A.device, queue)
    _native.call("tgg_k_grouped_gemm_queued", A.data_ptr(), B.data_ptr(), C.data_ptr(), group_start.data_ptr(),
                 group_end.data_ptr(), num_groups, M_DIM, N_DIM, K_TOTAL, _dtype_code(A.dtype), int(numSM),
                 queue.data_ptr(), _native.stream_of(A))
    return C
