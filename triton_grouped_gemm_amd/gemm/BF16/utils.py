"""Small helpers with the reference's names (gemm/BF16/utils.py): the per-group torch loop its scripts compare
against, the tolerance check, the random group-size draw and the row normalisation of its benchmarks."""
import random
from typing import List

import torch


def gmm(a: torch.Tensor, b: torch.Tensor, batch_sizes: torch.Tensor, trans_b: bool = False) -> torch.Tensor:
    """Per-group ``torch.matmul`` loop over consecutive row blocks of ``a`` (reference :5-14); ``batch_sizes`` on
    the host."""
    pieces, start = [], 0
    for g, size in enumerate(batch_sizes.tolist()):
        rhs = b[g].t() if trans_b else b[g]
        pieces.append(a[start:start + size] @ rhs)
        start += size
    return torch.cat(pieces)


def allclose(x: torch.Tensor, y: torch.Tensor, pct: float = 2.0) -> bool:
    """True when at most ``pct`` percent of the elements differ at rtol 1e-5 (reference :16-23)."""
    close = torch.isclose(x, y, rtol=1e-5)
    return float((close.numel() - close.sum()) / close.numel() * 100) <= pct


def generate_random_list(length: int, total_sum: int) -> List[int]:
    """``length`` non-negative integers that add up to ``total_sum``: uniform draws in ``[0, 2 * mean]`` scaled to
    the total, the rounding remainder added to the last entry (reference :25-39; Python's ``random`` state)."""
    mean = total_sum // length
    draws = [random.randint(0, 2 * int(mean)) for _ in range(length)]
    scale = total_sum / max(sum(draws), 1)
    out = [int(d * scale) for d in draws]
    out[-1] += total_sum - sum(out)
    return out


def row_max_normalization(tensor: torch.Tensor) -> torch.Tensor:
    """Rows scaled to a largest magnitude of one (reference :41-44)."""
    return tensor / (tensor.abs().max(dim=-1).values + 1e-9).unsqueeze(-1)
