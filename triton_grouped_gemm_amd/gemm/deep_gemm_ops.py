"""Contiguous ("DeepGEMM-style") grouped GEMM entry points, served natively.

The reference's gemm/deep_gemm_ops.py:24-100 validates shapes, builds the per-row group
layout and hands the arithmetic to the external ``deep_gemm`` package.  Here the same two
functions, with the same signatures and ``ValueError`` checks, run this library's own gfx950
kernels: A (and the output) are physically padded so that every expert starts at a multiple of
``block_m`` rows; ``size_per_group`` holds the real row counts.  Rows in the padding are not
written.

``grouped_layout`` is what the reference forwards to ``deep_gemm``.  When the caller leaves it out it is
implied by ``size_per_group`` and ``block_m`` (the reference builds it from them).  When the caller passes
one, the valid rows of every expert are taken from it, on the device and without a host round trip:
the psum form ``[G]`` (``use_psum_layout=True``: end offset of every expert's valid rows, starts aligned up to
``block_m``) is differenced -- it places expert g after expert g-1 by construction; of the per-row form
``[M_padded]`` (expert id per row, -1 on padding rows) the rows of every expert are counted and their first row
is located, so the experts' regions may follow one another in any order (``make_deep_gemm_grouped_layout``
builds them ascending; a router that fills the buffer in arrival order does not).  An expert whose rows lie in
several separate regions is served as well, region by region: such a layout is recognised by one read-back of two
counters (the wrappers already wait for the device once, for the reference's check of M) and the weights of the
regions' experts are gathered into a temporary ``[regions, N, K]`` tensor for the call.  While a stream is being
captured no read-back is possible and every expert is taken to have one region.
"""
from __future__ import annotations

from typing import Optional, Tuple

import torch

from .. import _native
from .BF16.m_grouped_gemm import _sizes_on_device
from .layout import round_up_to_alignment


def _check_contiguous_layout(a: torch.Tensor, b: torch.Tensor, size_per_group: torch.Tensor, block_m: int,
                             grouped_layout: Optional[torch.Tensor], use_psum_layout: bool, what: str):
    if a.dim() != 2 or b.dim() != 3:
        raise ValueError(f"expected {what} shape [M, K] and b shape [num_groups, N, K]")
    m, k = a.shape
    g, n, bk = b.shape
    if bk != k:
        raise ValueError(f"K mismatch: a has K={k}, b has K={bk}")
    if size_per_group.dim() != 1 or size_per_group.shape[0] != g:
        raise ValueError(f"size_per_group must hold {g} entries")
    # The reference reads the padded total back to the host here (gemm/deep_gemm_ops.py:49-51), which waits for the
    # device.  While the stream is being captured into a graph no such read is possible, so the check is left out
    # there: the kernels never touch rows at or beyond M, whatever the sizes say.
    if not (size_per_group.is_cuda and torch.cuda.is_current_stream_capturing()):
        expected_m = int(round_up_to_alignment(size_per_group.to(dtype=torch.int32), block_m).sum().item())
        if m != expected_m:
            raise ValueError(f"A must include padded expert rows: expected M={expected_m}, got M={m}")
    if grouped_layout is not None:
        want = g if use_psum_layout else m
        if grouped_layout.dim() != 1 or grouped_layout.shape[0] != want:
            raise ValueError(f"grouped_layout must have {want} entries")
        if grouped_layout.dtype not in (torch.int32, torch.int64):
            raise ValueError("grouped_layout must be an int32 or int64 tensor")
    return m, n, k, g


def sizes_from_layout(grouped_layout: torch.Tensor, num_groups: int, block_m: int, use_psum_layout: bool) -> torch.Tensor:
    """Valid rows per expert as an explicit layout states them (int32 ``[G]``, on the layout's device, no sync).

    psum form (reference gemm/layout.py:100-119): ``ends[g] = start[g] + size[g]`` with
    ``start[g] = ceil(ends[g-1] / block_m) * block_m`` and ``start[0] = 0``.  Per-row form (gemm/layout.py:73-97):
    the number of rows that carry expert id g.
    """
    lay = grouped_layout.to(torch.int64)
    if use_psum_layout:
        prev = torch.cat([lay.new_zeros(1), lay[:-1]])
        starts = (prev + (block_m - 1)) // block_m * block_m
        return (lay - starts).to(torch.int32)
    # slot 0 collects the padding rows (-1) and, so that no id can index outside the table, every id that names no
    # expert of b (below -1 or >= num_groups): those rows belong to no group and are not computed
    slot = torch.where((lay >= 0) & (lay < num_groups), lay + 1, torch.zeros_like(lay))
    counts = torch.zeros(num_groups + 1, dtype=torch.int64, device=lay.device)
    counts.scatter_add_(0, slot, torch.ones_like(lay))
    return counts[1:].to(torch.int32)


def placement_from_layout(grouped_layout: torch.Tensor, num_groups: int
                          ) -> Tuple[torch.Tensor, torch.Tensor, Optional[torch.Tensor]]:
    """Per-row layout ``[M_padded]`` (expert id per row, -1 = padding) -> ``(rows, first_row, expert)``.

    Every expert's rows in one region (the usual case): rows and first_row are int32 ``[G]`` on the layout's device
    -- how many rows carry expert id g and the smallest such row index (0 for experts without rows) -- and expert
    is None.  Some expert's rows in several regions: one entry per region (maximal run of rows with the same
    non-negative id) in row order, and expert ``[regions]`` (int64) names the expert of each, for the caller to
    gather the weights by.  Telling the two cases apart takes one read-back of two counters; while the current
    stream is being captured it is left out and the first form is returned: a captured call therefore needs one
    region per expert (several regions would be served as the single span from the expert's first row on), and ids
    outside [-1, num_groups), which raise ValueError eagerly, are treated as padding there.  Reference contract:
    gemm/layout.py:73-97 builds such layouts in ascending expert order, gemm/deep_gemm_ops.py:24-100 forwards
    whatever the caller passes.
    """
    lay = grouped_layout.to(torch.int64)
    m = lay.shape[0]
    dev = lay.device
    if m and not (lay.is_cuda and torch.cuda.is_current_stream_capturing()):
        change = torch.ones(m, dtype=torch.bool, device=dev)
        change[1:] = lay[1:] != lay[:-1]
        seen = torch.zeros(num_groups + 1, dtype=torch.bool, device=dev)  # last slot: padding and ids out of range
        seen[torch.where((lay >= 0) & (lay < num_groups), lay, num_groups)] = True
        n_regions, n_experts, n_bad = torch.stack([(change & (lay >= 0)).sum(), seen[:num_groups].sum(),
                                                   ((lay >= num_groups) | (lay < -1)).sum()]).tolist()
        if n_bad:
            raise ValueError(f"grouped_layout holds ids outside [-1, {num_groups}): b has {num_groups} experts and -1 marks padding")
        if n_regions > n_experts:
            if n_regions > _native.MAX_GROUPS_OTHER:
                raise ValueError(f"grouped_layout has {n_regions} separate regions, at most {_native.MAX_GROUPS_OTHER} are supported")
            starts = torch.nonzero(change).flatten()
            lengths = torch.diff(starts, append=starts.new_tensor([m]))
            keep = lay[starts] >= 0
            return lengths[keep].to(torch.int32), starts[keep].to(torch.int32), lay[starts][keep]
    # under capture nothing was checked: ids that name no expert go to the padding slot instead of indexing outside
    slot = torch.where((lay >= 0) & (lay < num_groups), lay + 1, torch.zeros_like(lay))
    counts = torch.zeros(num_groups + 1, dtype=torch.int64, device=dev)
    counts.scatter_add_(0, slot, torch.ones_like(lay))
    first = torch.full((num_groups + 1,), m, dtype=torch.int64, device=dev)
    first.scatter_reduce_(0, slot, torch.arange(m, dtype=torch.int64, device=dev), reduce="amin")
    first = torch.where(counts > 0, first, torch.zeros_like(first))
    return counts[1:].to(torch.int32), first[1:].to(torch.int32), None


def m_grouped_bf16_nt_contiguous(a: torch.Tensor, b: torch.Tensor, size_per_group: torch.Tensor, *,
                                 out: Optional[torch.Tensor] = None, grouped_layout: Optional[torch.Tensor] = None,
                                 block_m: int = 128, use_psum_layout: bool = False) -> torch.Tensor:
    """a ``[M_padded, K]`` bf16, b ``[G, N, K]`` bf16 -> ``[M_padded, N]`` bf16
    (reference gemm/deep_gemm_ops.py:24-57)."""
    m, n, k, g = _check_contiguous_layout(a, b, size_per_group, block_m, grouped_layout, use_psum_layout, "a")
    if a.dtype != torch.bfloat16 or b.dtype != torch.bfloat16:
        raise ValueError("a and b must be bfloat16")
    if out is None:
        out = torch.empty((m, n), device=a.device, dtype=torch.bfloat16)
    _native.require_gpu(a, b, out)
    if not (a.is_contiguous() and b.is_contiguous() and out.is_contiguous()):
        raise ValueError("a, b and out must be contiguous")
    if grouped_layout is not None and not use_psum_layout:  # per-row form: experts' regions in any order
        rows, first, expert = placement_from_layout(grouped_layout.to(a.device), g)
        if expert is not None:  # an expert in several regions: one group per region, weights gathered to match
            b = b.index_select(0, expert)
        _native.call("tgg_m_grouped_gemm_placed", a.data_ptr(), b.data_ptr(), out.data_ptr(), rows.data_ptr(), 0,
                     first.data_ptr(), rows.numel(), m, n, k, _native.BF16, -1, _native.stream_of(a))
        return out
    placed = size_per_group if grouped_layout is None else sizes_from_layout(grouped_layout, g, block_m, use_psum_layout)
    sizes, is64 = _sizes_on_device(placed, a.device)
    _native.call("tgg_m_grouped_gemm_padded", a.data_ptr(), b.data_ptr(), out.data_ptr(), sizes.data_ptr(), is64, g,
                 m, n, k, int(block_m), _native.BF16, -1, _native.stream_of(a))
    return out


def m_grouped_fp8_nt_contiguous(a: Tuple[torch.Tensor, torch.Tensor], b: Tuple[torch.Tensor, torch.Tensor],
                                size_per_group: torch.Tensor, *, out: Optional[torch.Tensor] = None,
                                grouped_layout: Optional[torch.Tensor] = None,
                                recipe_a: Optional[Tuple[int, int]] = None,
                                recipe_b: Optional[Tuple[int, int]] = None, block_m: int = 128,
                                use_psum_layout: bool = False) -> torch.Tensor:
    """Block-scaled FP8 grouped GEMM (reference gemm/deep_gemm_ops.py:60-100).

    ``a = (codes [M_padded, K] e4m3fn, scales [M_padded, K/128] fp32)`` (1x128 recipe; any strides, no copy
    when stored K-block-major as ``per_token_cast_to_fp8(..., scales_mn_major=True)`` returns them),
    ``b = (codes [G, N, K] e4m3fn, scales [G, ceil(N/128), K/128] fp32)`` (128x128 recipe).
    ``out[r, n] = sum_kb (sum_{k in kb} a[r,k] b[g,n,k]) * sa[r,kb] * sb[g, n//128, kb]`` with the
    scaling applied to the fp32 accumulator once per 128-deep K block; bf16 output.
    """
    a_codes, a_scale = a
    b_codes, b_scale = b
    m, n, k, g = _check_contiguous_layout(a_codes, b_codes, size_per_group, block_m, grouped_layout,
                                          use_psum_layout, "a[0]")
    if recipe_a not in (None, (1, 128)) or recipe_b not in (None, (128, 128)):
        raise ValueError("only recipe_a=(1, 128) and recipe_b=(128, 128) are implemented")
    if a_codes.dtype != torch.float8_e4m3fn or b_codes.dtype != torch.float8_e4m3fn:
        raise ValueError("a[0] and b[0] must be float8_e4m3fn")
    if block_m % 128 != 0:
        raise ValueError(f"block_m must be a multiple of 128, got {block_m}")
    kb, nb = (k + 127) // 128, (n + 127) // 128
    if tuple(a_scale.shape) != (m, kb):
        raise ValueError(f"a[1] must have shape ({m}, {kb}), got {tuple(a_scale.shape)}")
    if tuple(b_scale.shape) != (g, nb, kb):
        raise ValueError(f"b[1] must have shape ({g}, {nb}, {kb}), got {tuple(b_scale.shape)}")
    if out is None:
        out = torch.empty((m, n), device=a_codes.device, dtype=torch.bfloat16)
    _native.require_gpu(a_codes, a_scale, b_codes, b_scale, out)
    if not (a_codes.is_contiguous() and b_codes.is_contiguous() and out.is_contiguous()):
        raise ValueError("a[0], b[0] and out must be contiguous")
    # the tuned kernel streams the activation scales one K block (= one row of a [K/128, M] array) per
    # slab: a scale tensor that is already stored that way (strides (1, M)) is used as is
    sa = a_scale.to(torch.float32)
    if sa.stride() != (1, m) and kb > 1:
        sa = sa.t().contiguous().t()
    sb = b_scale.to(torch.float32).contiguous()
    if grouped_layout is not None and not use_psum_layout:  # per-row form: experts' regions in any order
        rows, first, expert = placement_from_layout(grouped_layout.to(a_codes.device), g)
        if expert is not None:  # an expert in several regions: one group per region, weights gathered to match
            b_codes = b_codes.view(torch.uint8).index_select(0, expert)
            sb = sb.index_select(0, expert)
        _native.call("tgg_m_grouped_gemm_fp8_block_placed", a_codes.data_ptr(), sa.data_ptr(), b_codes.data_ptr(),
                     sb.data_ptr(), out.data_ptr(), rows.data_ptr(), 0, first.data_ptr(), rows.numel(), m, n, k, 1, -1,
                     _native.stream_of(a_codes))
        return out
    placed = size_per_group if grouped_layout is None else sizes_from_layout(grouped_layout, g, block_m, use_psum_layout)
    sizes, is64 = _sizes_on_device(placed, a_codes.device)
    _native.call("tgg_m_grouped_gemm_fp8_block", a_codes.data_ptr(), sa.data_ptr(), b_codes.data_ptr(),
                 sb.data_ptr(), out.data_ptr(), sizes.data_ptr(), is64, g, m, n, k, int(block_m), 1, -1,
                 _native.stream_of(a_codes))
    return out
