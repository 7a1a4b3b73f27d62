"""Grouped-GEMM row layouts: group sizes -> starts, padded sizes, per-row expert ids.

Host-side integer helpers with the interface of the reference's ``gemm/layout.py``
(:11-126).  Values *and* dtypes match it: ``sizes``/``padded_sizes`` are int32,
prefix sums come out of ``cumsum`` as int64, the two DeepGEMM-style layouts are
int32.  Unlike the reference the per-row layouts are built with vectorised
tensor ops on the tensor's own device (one size query, no Python loop over
groups), so they stay cheap at G in the hundreds.
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Sequence, Union

import torch

SizesLike = Union[torch.Tensor, Sequence[int]]


@dataclass(frozen=True)
class GroupedLayout:
    """Padded placement of every group (reference gemm/layout.py:11-23)."""

    starts: torch.Tensor
    sizes: torch.Tensor
    padded_sizes: torch.Tensor

    @property
    def total_m(self) -> torch.Tensor:
        return self.sizes.sum()

    @property
    def total_padded_m(self) -> torch.Tensor:
        return self.padded_sizes.sum()


def as_group_sizes(size_per_group: SizesLike, *, device=None, dtype: torch.dtype = torch.int32) -> torch.Tensor:
    """Normalise to a contiguous 1-D integer tensor (reference gemm/layout.py:26-45)."""
    if torch.is_tensor(size_per_group):
        sizes = size_per_group if device is None else size_per_group.to(device=device)
        sizes = sizes.to(dtype=dtype)
    else:
        sizes = torch.tensor(size_per_group, device=device, dtype=dtype)
    if sizes.dim() != 1:
        raise ValueError(f"size_per_group must be 1D, got shape {tuple(sizes.shape)}")
    if sizes.numel() == 0:
        raise ValueError("size_per_group must contain at least one group")
    if bool((sizes < 0).any().item()):
        raise ValueError("size_per_group cannot contain negative sizes")
    return sizes.contiguous()


def round_up_to_alignment(sizes: torch.Tensor, alignment: int) -> torch.Tensor:
    """ceil(sizes / alignment) * alignment, dtype preserved (reference gemm/layout.py:48-51)."""
    if alignment <= 0:
        raise ValueError(f"alignment must be positive, got {alignment}")
    return torch.div(sizes + (alignment - 1), alignment, rounding_mode="floor") * alignment


def _exclusive_prefix(values: torch.Tensor) -> torch.Tensor:
    return (values.cumsum(0) - values).contiguous()


def make_grouped_layout(size_per_group: SizesLike, block_m: int = 128) -> GroupedLayout:
    """Reference gemm/layout.py:54-58."""
    sizes = as_group_sizes(size_per_group)
    padded = round_up_to_alignment(sizes, block_m).contiguous()
    return GroupedLayout(starts=_exclusive_prefix(padded), sizes=sizes, padded_sizes=padded)


def make_group_starts(size_per_group: SizesLike, *, padded: bool = False, block_m: int = 128,
                      dtype: torch.dtype = torch.int32) -> torch.Tensor:
    """Exclusive prefix sum of the logical or padded sizes (reference gemm/layout.py:61-70)."""
    sizes = as_group_sizes(size_per_group, dtype=dtype)
    return _exclusive_prefix(round_up_to_alignment(sizes, block_m) if padded else sizes)


def make_deep_gemm_grouped_layout(size_per_group: SizesLike, *, block_m: int = 128, device=None) -> torch.Tensor:
    """One int32 per padded row: expert id on real rows, -1 on pad rows
    (reference gemm/layout.py:73-97)."""
    sizes = as_group_sizes(size_per_group, device=device, dtype=torch.int32)
    padded = round_up_to_alignment(sizes, block_m)
    total = int(padded.sum().item())
    ids = torch.arange(sizes.numel(), device=sizes.device, dtype=torch.int32)
    row_group = torch.repeat_interleave(ids, padded.to(torch.int64), output_size=total)
    starts = _exclusive_prefix(padded.to(torch.int64))
    gidx = row_group.to(torch.int64)
    offset_in_group = torch.arange(total, device=sizes.device, dtype=torch.int64) - starts[gidx]
    real = offset_in_group < sizes.to(torch.int64)[gidx]
    return torch.where(real, row_group, torch.full_like(row_group, -1)).contiguous()


def make_deep_gemm_psum_layout(size_per_group: SizesLike, *, block_m: int = 128, device=None) -> torch.Tensor:
    """End of each expert's real rows in padded-M coordinates, int32
    (reference gemm/layout.py:100-119)."""
    sizes = as_group_sizes(size_per_group, device=device, dtype=torch.int32)
    padded = round_up_to_alignment(sizes, block_m)
    return (_exclusive_prefix(padded) + sizes).to(torch.int32).contiguous()


def validate_total_m(size_per_group: SizesLike, total_m: int) -> None:
    """Reference gemm/layout.py:122-126."""
    actual = int(as_group_sizes(size_per_group, dtype=torch.int64).sum().item())
    if actual != total_m:
        raise ValueError(f"sum(size_per_group) must equal M ({total_m}), got {actual}")
