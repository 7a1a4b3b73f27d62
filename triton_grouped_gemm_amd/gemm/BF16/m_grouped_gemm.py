"""BF16/FP16 M-grouped GEMM over expert-contiguous rows.

Host-side mirror of the reference operator ``moe::m_grouped_gemm``
(gemm/BF16/m_grouped_gemm_TMA.py:297-462; SM80 twin gemm/BF16/m_grouped_gemm.py:220-292):
same names, arguments and assertion messages.  Underneath there is one native
implementation: the call crosses the C ABI (``tgg_m_grouped_gemm``) into a persistent
gfx950 MFMA kernel that derives its tile schedule from ``size_per_group`` on the device,
so no tile->group map, no ``.item()`` and no side stream are involved; the launch goes
to the caller's current stream.
"""
from __future__ import annotations

from typing import Optional, Tuple

import torch
from torch import Tensor

from ... import _native

BLOCK_M = 128


def _sizes_on_device(size_per_group: Tensor, device) -> Tuple[Tensor, int]:
    """int32/int64 contiguous sizes on `device`; returns (tensor, is_int64)."""
    s = size_per_group
    if s.dtype not in (torch.int32, torch.int64):
        s = s.to(torch.int32)
    if s.device != device:
        s = s.to(device, non_blocking=True)
    s = s.contiguous()
    return s, int(s.dtype == torch.int64)


def _build_m_grouped_metadata(size_per_group: Tensor, block_m: int = BLOCK_M):
    """Tile metadata in the reference's format (gemm/BF16/m_grouped_gemm_TMA.py:297-326):
    ``(pad_start, pad_end, group_start, group_end, m_indices_pad, M_pad)``.

    The native kernel does not consume it (it rebuilds the prefix sums in LDS); it is kept
    for callers that inspect or pass it around.  The slots of ``m_indices_pad`` past the
    last padded tile are uninitialised in the reference; here they hold -1.
    """
    num_groups = size_per_group.shape[0]
    sizes = size_per_group.to(torch.int32)
    M = int(sizes.sum().item())
    padded = torch.div(sizes + block_m - 1, block_m, rounding_mode="floor") * block_m
    M_pad = padded.sum()
    repeats = (padded // block_m).to(torch.int64)
    slots = M // block_m + num_groups
    m_indices_pad = torch.full((slots,), -1, device=sizes.device, dtype=torch.int32)
    ids = torch.repeat_interleave(torch.arange(num_groups, device=sizes.device, dtype=torch.int32), repeats)
    m_indices_pad[: ids.numel()] = ids
    pad_end = padded.cumsum(0).to(torch.int32)
    pad_start = pad_end - padded
    group_end = sizes.cumsum(0)
    group_start = group_end - sizes
    return pad_start, pad_end, group_start, group_end, m_indices_pad, M_pad


def _m_grouped_gemm_launch(A: Tensor, B: Tensor, C: Tensor, size_per_group: Tensor, trans_b: bool = False,
                           numSM: int = -1, metadata=None, use_fixed_sm90_config: bool = True) -> Tensor:
    """Validate like the reference launcher (:329-374) and enqueue the native kernel.
    ``metadata`` and ``use_fixed_sm90_config`` are accepted and ignored."""
    assert A.dim() == 2
    assert B.dim() == 3
    assert C.dim() == 2
    M, K = A.shape
    if trans_b:
        num_groups, N, BK = B.shape
    else:
        num_groups, BK, N = B.shape
    assert BK == K, "K of A should be equal to K of B"
    assert C.shape == (M, N), "C should have shape [M, N]"
    assert A.stride(-1) == 1, "Please make sure A is K-major"
    assert A.dtype in _native.DTYPE_CODE, f"data type {A.dtype} not supported"
    assert B.dtype in _native.DTYPE_CODE, f"data type {B.dtype} not supported"
    assert C.dtype in _native.DTYPE_CODE, f"data type {C.dtype} not supported"
    assert A.dtype == B.dtype == C.dtype, "A, B and C must share one data type"
    assert (N * B.element_size()) % 16 == 0, "TMA required 16-byte alignment"
    assert (K * B.element_size()) % 16 == 0, "TMA required 16-byte alignment"
    assert size_per_group.dim() == 1 and size_per_group.shape[0] == num_groups, \
        "size_per_group must hold one entry per group of B"
    assert num_groups <= _native.MAX_GROUPS, f"at most {_native.MAX_GROUPS} groups are supported"
    _native.require_gpu(A, B, C)
    assert A.is_contiguous() and B.is_contiguous() and C.is_contiguous(), "A, B and C must be contiguous"
    sizes, is64 = _sizes_on_device(size_per_group, A.device)
    _native.call("tgg_m_grouped_gemm", A.data_ptr(), B.data_ptr(), C.data_ptr(), sizes.data_ptr(), is64,
                 num_groups, M, N, K, int(bool(trans_b)), _native.DTYPE_CODE[A.dtype], int(numSM),
                 _native.stream_of(A))
    return C


@torch.library.custom_op("moe::m_grouped_gemm", mutates_args=())
def m_grouped_gemm(A: Tensor, B: Tensor, size_per_group: Tensor, trans_b: bool = False, numSM: int = -1) -> Tensor:
    """``C[r] = A[r] @ B[g(r)]^T`` (``trans_b``) or ``A[r] @ B[g(r)]``; rows past ``sum(size_per_group)``
    are left uninitialised, as in the reference (:435-447)."""
    M, K = A.shape
    N = B.shape[1] if trans_b else B.shape[2]
    C = A.new_empty(M, N)
    return _m_grouped_gemm_launch(A, B, C, size_per_group, trans_b, numSM)


@m_grouped_gemm.register_fake
def _(A: Tensor, B: Tensor, size_per_group: Tensor, trans_b: bool = False, numSM: int = -1) -> Tensor:
    M, K = A.shape
    N = B.shape[1] if trans_b else B.shape[2]
    return A.new_empty(M, N)
