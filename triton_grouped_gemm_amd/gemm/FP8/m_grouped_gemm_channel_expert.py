"""FP8 M-grouped GEMM with a per-token activation scale and a per-(expert, channel) weight scale.

Mirror of gemm/FP8/m_grouped_gemm_channel_expert.py:139-198: same operator name
(``myfp8::gmm_fp8_act_per_channel_w_per_expert``), arguments and output dtype default.
The contraction runs on the gfx950 fp8 MFMA with fp32 accumulation; both scales are
applied once to the fp32 accumulator in the epilogue.  N needs no tile divisibility here.
"""
from __future__ import annotations

import torch
from torch import Tensor

from ... import _native
from ..BF16.m_grouped_gemm import _sizes_on_device


@torch.library.custom_op("myfp8::gmm_fp8_act_per_channel_w_per_expert", mutates_args=())
def gmm_fp8_act_per_channel_w_per_expert(A: Tensor, A_scale: Tensor, B: Tensor, B_scale: Tensor,
                                         size_per_group: Tensor, dtype_out: torch.dtype = torch.float16) -> Tensor:
    """A ``[M, K]`` fp8, A_scale ``[M, 1]`` fp32, B ``[G, N, K]`` fp8, B_scale fp32 with ``G*N`` entries
    (element ``g*N + n`` scales column n of expert g)."""
    assert A.dim() == 2
    assert B.dim() == 3
    M, K = A.shape
    num_groups, N, BK = B.shape
    assert BK == K
    assert B.stride(-1) == 1, "Please make sure B is K-major"
    assert A.stride(-1) == 1, "Please make sure A is K-major"
    assert A.dtype in _native.FP8_CODE, f"data type {A.dtype} not supported"
    assert B.dtype in _native.FP8_CODE, f"data type {B.dtype} not supported"
    assert dtype_out in _native.DTYPE_CODE, f"data type {dtype_out} not supported"
    assert A_scale.numel() == M and B_scale.numel() == num_groups * N, "scale tensors have the wrong number of entries"
    assert size_per_group.dim() == 1 and size_per_group.shape[0] == num_groups
    assert num_groups <= _native.MAX_GROUPS_OTHER, f"at most {_native.MAX_GROUPS_OTHER} groups are supported"
    _native.require_gpu(A, A_scale, B, B_scale)
    assert A.is_contiguous() and B.is_contiguous(), "A and B must be contiguous"
    a_s = A_scale.to(torch.float32).contiguous()
    b_s = B_scale.to(torch.float32).contiguous()
    sizes, is64 = _sizes_on_device(size_per_group, A.device)
    C = A.new_empty(M, N, dtype=dtype_out)
    _native.call("tgg_m_grouped_gemm_fp8_channel", A.data_ptr(), a_s.data_ptr(), B.data_ptr(), b_s.data_ptr(),
                 C.data_ptr(), sizes.data_ptr(), is64, num_groups, M, N, K, _native.FP8_CODE[A.dtype],
                 _native.FP8_CODE[B.dtype], _native.DTYPE_CODE[dtype_out], -1, _native.stream_of(A))
    return C


@gmm_fp8_act_per_channel_w_per_expert.register_fake
def _(A, A_scale, B, B_scale, size_per_group, dtype_out=torch.float16):
    return A.new_empty(A.shape[0], B.shape[1], dtype=dtype_out)
