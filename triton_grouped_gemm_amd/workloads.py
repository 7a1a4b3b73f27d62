"""Seeded synthetic workloads for the grouped-GEMM path (group-size draws and operand tensors).

Group sizes follow the benchmark configurations this library is measured on: a Dirichlet(1)
probability vector over the experts, a multinomial draw of 128-row blocks (so every size is a
multiple of ``align`` and the total is exact), or an unaligned multinomial draw over rows.
"""
from __future__ import annotations

import torch


def dirichlet_multinomial_sizes(groups: int, total: int, align: int = 128, seed: int = 0) -> torch.Tensor:
    """int32 ``[groups]``, each a multiple of ``align``, summing to ``total`` exactly."""
    assert total % align == 0
    gen = torch.Generator().manual_seed(seed)
    gamma = torch._standard_gamma(torch.ones(groups, dtype=torch.float64), generator=gen)
    probs = gamma / gamma.sum()
    draws = torch.multinomial(probs, total // align, replacement=True, generator=gen)
    return (torch.bincount(draws, minlength=groups) * align).to(torch.int32)


def uniform_sizes(groups: int, total: int) -> torch.Tensor:
    assert total % groups == 0
    return torch.full((groups,), total // groups, dtype=torch.int32)


def masked_counts(groups: int, m_max: int, seed: int = 0) -> torch.Tensor:
    """Uniform integers in [0, m_max]."""
    gen = torch.Generator().manual_seed(seed)
    return torch.randint(0, m_max + 1, (groups,), generator=gen, dtype=torch.int32)


def randn_bf16(shape, scale: float, seed: int, device="cpu") -> torch.Tensor:
    """N(0, 1) * scale in bf16, drawn on ``device`` from a seeded generator."""
    gen = torch.Generator(device=device).manual_seed(seed)
    out = torch.empty(shape, device=device, dtype=torch.bfloat16)
    chunk = max(1, (1 << 26) // max(1, out[0].numel())) if out.dim() > 1 else out.numel()
    flat = out.view(out.shape[0], -1) if out.dim() > 1 else out.view(1, -1)
    if out.dim() > 1:
        for s in range(0, out.shape[0], chunk):
            e = min(out.shape[0], s + chunk)
            flat[s:e] = (torch.randn((e - s, flat.shape[1]), device=device, dtype=torch.float32, generator=gen)
                         * scale).to(torch.bfloat16)
    else:
        out.copy_((torch.randn(out.shape, device=device, dtype=torch.float32, generator=gen) * scale).to(torch.bfloat16))
    return out
