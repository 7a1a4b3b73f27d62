"""Plain-Python restatement of the reference's grouped-layout helpers (test oracle).

Follows gemm/layout.py:26-126 and the tile metadata builder
gemm/BF16/m_grouped_gemm_TMA.py:297-326.  Everything is integer arithmetic on
Python lists; dtypes of the tensors the reference returns are recorded beside
each function so the product's torch helpers can be compared on both value and
dtype.
"""
from __future__ import annotations

from typing import List, Sequence


def check_sizes(sizes: Sequence[int]) -> List[int]:
    """gemm/layout.py:39-44: 1-D, non-empty, non-negative."""
    sizes = [int(s) for s in sizes]
    if len(sizes) == 0:
        raise ValueError("size_per_group must contain at least one group")
    if any(s < 0 for s in sizes):
        raise ValueError("size_per_group cannot contain negative sizes")
    return sizes


def round_up(sizes: Sequence[int], alignment: int) -> List[int]:
    """gemm/layout.py:48-51 (floor division form)."""
    if alignment <= 0:
        raise ValueError(f"alignment must be positive, got {alignment}")
    return [((int(s) + alignment - 1) // alignment) * alignment for s in sizes]


def exclusive_prefix(values: Sequence[int]) -> List[int]:
    out, acc = [], 0
    for v in values:
        out.append(acc)
        acc += int(v)
    return out


def group_starts(sizes: Sequence[int], padded: bool = False, block_m: int = 128) -> List[int]:
    """gemm/layout.py:61-70.  dtype of the reference result: int64 (cumsum of int32)."""
    sizes = check_sizes(sizes)
    return exclusive_prefix(round_up(sizes, block_m) if padded else sizes)


def grouped_layout(sizes: Sequence[int], block_m: int = 128):
    """gemm/layout.py:54-58 -> dict(starts int64, sizes int32, padded_sizes int32, totals)."""
    sizes = check_sizes(sizes)
    padded = round_up(sizes, block_m)
    return dict(starts=exclusive_prefix(padded), sizes=sizes, padded_sizes=padded,
                total_m=sum(sizes), total_padded_m=sum(padded))


def deep_gemm_grouped_layout(sizes: Sequence[int], block_m: int = 128) -> List[int]:
    """gemm/layout.py:73-97: expert id per padded row, -1 on pad rows (int32)."""
    sizes = check_sizes(sizes)
    out: List[int] = []
    for g, (s, p) in enumerate(zip(sizes, round_up(sizes, block_m))):
        out += [g] * s + [-1] * (p - s)
    return out


def deep_gemm_psum_layout(sizes: Sequence[int], block_m: int = 128) -> List[int]:
    """gemm/layout.py:100-119: end of the real rows in padded coordinates (int32)."""
    sizes = check_sizes(sizes)
    ends, start = [], 0
    for s, p in zip(sizes, round_up(sizes, block_m)):
        ends.append(start + s)
        start += p
    return ends


def validate_total_m(sizes: Sequence[int], total_m: int) -> None:
    """gemm/layout.py:122-126."""
    actual = sum(check_sizes(sizes))
    if actual != total_m:
        raise ValueError(f"sum(size_per_group) must equal M ({total_m}), got {actual}")


def m_grouped_metadata(sizes: Sequence[int], block_m: int = 128):
    """gemm/BF16/m_grouped_gemm_TMA.py:297-326.

    Returns pad_start, pad_end, group_start, group_end, the initialised prefix of
    m_indices_pad (the reference leaves the remaining M//block_m + G - len slots
    uninitialised) and M_pad.
    """
    sizes = [int(s) for s in sizes]
    padded = round_up(sizes, block_m)
    pad_start = exclusive_prefix(padded)
    pad_end = [a + b for a, b in zip(pad_start, padded)]
    group_start = exclusive_prefix(sizes)
    group_end = [a + b for a, b in zip(group_start, sizes)]
    m_indices: List[int] = []
    for g, p in enumerate(padded):
        m_indices += [g] * (p // block_m)
    return pad_start, pad_end, group_start, group_end, m_indices, sum(padded)


def tile_rows(sizes: Sequence[int], block_m: int = 128):
    """Virtual padded tile space of the M-grouped kernels
    (gemm/BF16/m_grouped_gemm_TMA.py:138-142,161-169): for every padded M tile
    the tuple (group, first logical row, number of valid rows)."""
    pad_start, _, group_start, group_end, m_indices, _ = m_grouped_metadata(sizes, block_m)
    out = []
    for pid_m, g in enumerate(m_indices):
        row0 = group_start[g] + pid_m * block_m - pad_start[g]
        out.append((g, row0, min(block_m, group_end[g] - row0)))
    return out
