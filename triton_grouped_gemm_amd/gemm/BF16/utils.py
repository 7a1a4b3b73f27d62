"""Small comparison helpers with the reference's names (gemm/BF16/utils.py:16-23,41-44)."""
import torch


def row_max_normalization(tensor: torch.Tensor) -> torch.Tensor:
    return tensor / (tensor.abs().max(dim=-1).values + 1e-9).unsqueeze(-1)


def allclose(x: torch.Tensor, y: torch.Tensor, pct: float = 2.0) -> bool:
    """True when at most ``pct`` percent of the elements differ at rtol 1e-5."""
    close = torch.isclose(x, y, rtol=1e-5)
    return float((close.numel() - close.sum()) / close.numel() * 100) <= pct
