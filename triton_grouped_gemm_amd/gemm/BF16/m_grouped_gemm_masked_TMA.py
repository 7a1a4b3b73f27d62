"""Masked M-grouped GEMM (decode layout): only the first ``masked_m[g]`` rows of every
group are computed and written, in place, into the caller's ``out``.

Mirror of gemm/BF16/m_grouped_gemm_masked_TMA.py:164-250.  Differences that are
deliberate: the launch goes to the caller's current stream (the reference opens a fresh,
never-joined stream, :185-186), and ``trans_b=False`` (rhs ``[G, K, N]``) works.
"""
from __future__ import annotations

import torch
from torch import Tensor

from ... import _native
from .m_grouped_gemm import BLOCK_M, _sizes_on_device


def m_grouped_gemm_masked(lhs: Tensor, rhs: Tensor, out: Tensor, masked_m: Tensor, expected_m: int,
                          trans_b: bool = True) -> None:
    """lhs ``[G*m_max, K]``, rhs ``[G, N, K]``, out ``[G*m_max, N]``; ``expected_m`` is the row
    stride ``m_max`` between groups (the reference kernel uses it that way, :107-111)."""
    assert lhs.dim() == 2
    assert rhs.dim() == 3
    M, K = lhs.shape
    assert lhs.stride(-1) == 1, "Please make sure lhs is K-major"
    if trans_b:
        num_groups, N, rhsK = rhs.shape
    else:
        num_groups, rhsK, N = rhs.shape
    assert rhsK == K, "K of lhs should be equal to K of rhs"
    assert lhs.dtype in _native.DTYPE_CODE, f"data type {lhs.dtype} not supported"
    assert lhs.dtype == rhs.dtype == out.dtype, "lhs, rhs and out must share one data type"
    assert (N * rhs.element_size()) % 16 == 0, "TMA required 16-byte alignment"
    assert (K * rhs.element_size()) % 16 == 0, "TMA required 16-byte alignment"
    assert M % BLOCK_M == 0, "Only support when M is a multiple of BLOCK_M"
    assert out.dim() == 2 and tuple(out.shape) == (M, N), "out should have shape [M, N]"
    assert masked_m.dim() == 1 and masked_m.shape[0] == num_groups, "masked_m must hold one entry per group"
    assert num_groups * int(expected_m) <= M, "expected_m * num_groups must not exceed the rows of lhs"
    assert num_groups <= _native.MAX_GROUPS_OTHER, f"at most {_native.MAX_GROUPS_OTHER} groups are supported"
    _native.require_gpu(lhs, rhs, out)
    assert lhs.is_contiguous() and rhs.is_contiguous() and out.is_contiguous(), "lhs, rhs and out must be contiguous"
    mm, is64 = _sizes_on_device(masked_m, lhs.device)
    _native.call("tgg_m_grouped_gemm_masked", lhs.data_ptr(), rhs.data_ptr(), out.data_ptr(), mm.data_ptr(), is64,
                 num_groups, int(expected_m), M, N, K, int(bool(trans_b)), _native.DTYPE_CODE[lhs.dtype], -1,
                 _native.stream_of(lhs))
    return None
