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


def reference_random_sizes(groups: int, total: int, seed: int = 0) -> list:
    """Group sizes as the reference's own benchmark draws them for ``--random-groups``
    (``_fallback_generate_random_list``, gemm/BF16/m_grouped_gemm_TMA.py:496-513): integer weights in [1, 10000)
    from a seeded CPU generator, sizes proportional to them (floor, at least 1), the remainder dealt out (or taken
    back from sizes above 1) one row at a time in index order.  Exact sum, no empty group."""
    gen = torch.Generator(device="cpu").manual_seed(seed)
    weights = torch.randint(1, 10000, (groups,), generator=gen, dtype=torch.int64)
    sizes = torch.clamp(torch.div(weights * total, weights.sum(), rounding_mode="floor"), min=1).tolist()
    diff, idx = total - sum(sizes), 0
    while diff != 0:
        j = idx % groups
        if diff > 0:
            sizes[j] += 1
            diff -= 1
        elif sizes[j] > 1:
            sizes[j] -= 1
            diff += 1
        idx += 1
    return sizes


def reference_group_sizes(groups: int, total: int, seed: int, uniform: bool, align: int = 64,
                          aligned: bool = True) -> torch.Tensor:
    """``make_group_sizes`` of the reference's benchmark main (gemm/BF16/m_grouped_gemm_TMA.py:541-562): uniform
    (its default), random in blocks of ``align`` rows (``--random-groups``, :527-538), or random with an exact sum
    and no alignment (``--unaligned-random-groups``).  int32 on the CPU."""
    if uniform:
        assert total % groups == 0, "uniform_groups requires total_m divisible by num_groups"
        sizes = [total // groups] * groups
    elif aligned:
        assert align > 0 and total % align == 0, f"total_m={total} must be divisible by align={align}"
        assert total // align >= groups, "Need at least one aligned block per group"
        sizes = [b * align for b in reference_random_sizes(groups, total // align, seed)]
    else:
        sizes = reference_random_sizes(groups, total, seed)
    return torch.tensor(sizes, dtype=torch.int32)
