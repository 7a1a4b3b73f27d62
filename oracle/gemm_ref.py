"""torch-CPU restatement of the reference's per-group matmul oracles (test oracle).

Follows gemm/BF16/utils.py:5-14 (``gmm``) == gemm/BF16/m_grouped_gemm_TMA.py:573-581
(``m_grouped_reference``), gemm/BF16/k_grouped_gemm_TMA.py:402-416
(``gmm_dw_reference``), the masked semantics of
gemm/BF16/m_grouped_gemm_masked_TMA.py:103-134, the FP8 epilogues of
gemm/FP8/m_grouped_gemm_channel_expert.py:119-136 and
gemm/FP8/k_grouped_gemm_channel_expert.py:104-140, and the block-scaled contract
of gemm/deep_gemm_ops.py:60-100 (closed form; parity unpinned by the reference).

``*_fp32`` variants accumulate and return fp32 ("exact" up to fp32 rounding);
the plain variants compute in the tensors' own dtype like the reference.
"""
from __future__ import annotations

from typing import Sequence

import torch


def _sizes(sizes) -> list:
    return [int(s) for s in (sizes.tolist() if isinstance(sizes, torch.Tensor) else sizes)]


def gmm(a: torch.Tensor, b: torch.Tensor, sizes, trans_b: bool = False) -> torch.Tensor:
    out, start = [], 0
    for g, size in enumerate(_sizes(sizes)):
        rhs = b[g].t() if trans_b else b[g]
        out.append(a[start:start + size] @ rhs)
        start += size
    return torch.cat(out).contiguous()


def gmm_fp32(a, b, sizes, trans_b=False):
    return gmm(a.float(), b.float(), sizes, trans_b)


def masked_gmm(lhs: torch.Tensor, rhs: torch.Tensor, masked_m, m_stride: int, fp32: bool = False):
    """lhs [G*m_stride, K], rhs [G, N, K] -> list of per-group [masked_m[g], N] results."""
    outs = []
    for g, mm in enumerate(_sizes(masked_m)):
        a = lhs[g * m_stride: g * m_stride + mm]
        r = rhs[g]
        outs.append((a.float() @ r.float().t()) if fp32 else (a @ r.t()))
    return outs


def gmm_dw(a: torch.Tensor, b: torch.Tensor, sizes, fp32: bool = False) -> torch.Tensor:
    """a [Ktot, M], b [Ktot, N] -> [G, M, N]; empty group -> zeros (TMA kernel behaviour,
    gemm/BF16/k_grouped_gemm_TMA.py:140-170)."""
    sizes = _sizes(sizes)
    odt = torch.float32 if fp32 else a.dtype
    out = torch.zeros(len(sizes), a.shape[1], b.shape[1], dtype=odt)
    start = 0
    for g, size in enumerate(sizes):
        if size:
            l, r = a[start:start + size], b[start:start + size]
            out[g] = (l.float().t() @ r.float()) if fp32 else (l.t() @ r)
        start += size
    return out


def fp8_channel_reference(aq_f32, a_scale, bq_f32, b_scale, sizes) -> torch.Tensor:
    """C = (Aq . Bq[g]^T) * a_scale[r] * b_scale[g*N + n] in fp32.
    aq_f32 [M,K], a_scale [M,1] or [M], bq_f32 [G,N,K], b_scale flattened [G*N]."""
    G, N, _ = bq_f32.shape
    c = gmm(aq_f32.float(), bq_f32.float(), sizes, trans_b=True)
    out, start = [], 0
    bs = b_scale.reshape(G, N).float()
    for g, size in enumerate(_sizes(sizes)):
        out.append(c[start:start + size] * a_scale.reshape(-1)[start:start + size, None].float() * bs[g][None, :])
        start += size
    return torch.cat(out)


def fp8_k_grouped_channel_reference(xq_f32, xs, yq_f32, ys, tokens_padded) -> torch.Tensor:
    """out[g] = (x[:, seg_g] . y[:, seg_g]^T) * xs[:, g] (x) ys[:, g], fp32.
    xq_f32 [M, Ktot], yq_f32 [N, Ktot], xs [M, G], ys [N, G]."""
    outs, start = [], 0
    for g, t in enumerate(_sizes(tokens_padded)):
        acc = xq_f32[:, start:start + t].float() @ yq_f32[:, start:start + t].float().t()
        outs.append(acc * xs[:, g].float()[:, None] * ys[:, g].float()[None, :])
        start += t
    return torch.stack(outs)


def fp8_block_scaled_reference(aq_f32, sa, bq_f32, sb, sizes, block_m: int = 128) -> torch.Tensor:
    """Dequantise (1x128 activation scales, 128x128 weight scales) then fp32 matmul.

    aq_f32 [M_pad, K] values of the codes, sa [M_pad, K/128]; bq_f32 [G, N, K],
    sb [G, ceil(N/128), K/128].  A is physically padded per group to ``block_m``
    (gemm/deep_gemm_ops.py:88-90); pad rows of the result are returned as zero.
    """
    M, K = aq_f32.shape
    G, N, _ = bq_f32.shape
    a = aq_f32.float() * sa.float().repeat_interleave(128, dim=1)[:, :K]
    b = bq_f32.float() * sb.float().repeat_interleave(128, dim=1)[:, :N].repeat_interleave(128, dim=2)[:, :, :K]
    out = torch.zeros(M, N, dtype=torch.float32)
    start = 0
    for g, size in enumerate(_sizes(sizes)):
        out[start:start + size] = a[start:start + size] @ b[g].t()
        start += (size + block_m - 1) // block_m * block_m
    return out


def row_max_normalization(t: torch.Tensor) -> torch.Tensor:
    """gemm/BF16/utils.py:41-44."""
    return t / (t.abs().max(dim=-1).values + 1e-9).unsqueeze(-1)


def rdiff(out: torch.Tensor, ref: torch.Tensor) -> float:
    """max|out-ref| / max(max|out|, max|ref|)  (gemm/FP8/m_grouped_gemm_channel_expert.py:349-351)."""
    out, ref = out.double(), ref.double()
    amax = max(out.abs().max().item(), ref.abs().max().item())
    return 0.0 if amax == 0 else (out - ref).abs().max().item() / amax


def cos_diff(out: torch.Tensor, ref: torch.Tensor) -> float:
    """1 - 2<x,y>/(|x|^2+|y|^2): global similarity that does not hinge on one ulp flip."""
    x, y = out.double().flatten(), ref.double().flatten()
    den = (x * x + y * y).sum().item()
    return 0.0 if den == 0 else 1.0 - 2.0 * (x * y).sum().item() / den
