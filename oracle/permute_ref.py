"""CPU restatement of the MoE permute / unpermute semantics (test infrastructure only).

Follows the torch side of the reference's own test (grouped_gemm/grouped_gemm/permute_test.py:18-72), which is what
its kernels are checked against, plus the row_id_map definition of grouped_gemm/csrc/permute.cu:40-101.
Pinned by library routines: torch.argsort(stable=True), index_select, index_copy, bincount.
"""
import torch


def permute(tokens: torch.Tensor, indices: torch.Tensor):
    """permute_test.py:18-34: rows in stable expert-major order; returns (permuted, sorted_indices)."""
    topk = indices.size(1)
    flat = indices.reshape(-1)
    order = torch.argsort(flat, stable=True)
    return tokens.index_select(0, order // topk), order


def row_id_map(indices: torch.Tensor, num_out_tokens: int = 0) -> torch.Tensor:
    """permute.cu:40-101 after a stable sort by expert id: entry [k * T + t] is the sorted position of assignment
    (t, k); assignments with expert id -1 sort first and do not count; positions >= num_out_tokens (> 0) give -1."""
    tokens, topk = indices.shape
    flat = indices.reshape(-1)
    order = torch.argsort(flat, stable=True)
    neg = int((flat < 0).sum())
    cap = num_out_tokens if num_out_tokens > 0 else tokens * topk
    out = torch.empty(tokens * topk, dtype=torch.int32)
    for pos, src in enumerate(order.tolist()):
        t, k = divmod(src, topk)
        p = pos - neg
        out[k * tokens + t] = p if 0 <= p < cap else -1
    return out


def unpermute(permuted: torch.Tensor, sorted_indices: torch.Tensor, probs: torch.Tensor = None, fp32: bool = False):
    """permute_test.py:37-72 (fp32=False: its dtype sequence; fp32=True: everything in fp32, for tolerance gates)."""
    topk = probs.size(1) if probs is not None else 1
    x = permuted.float() if fp32 else permuted
    un = torch.zeros_like(x).index_copy(0, sorted_indices, x)
    un = un.reshape(-1, topk, x.size(-1))
    if probs is not None:
        dtype = un.dtype
        un = (un * probs.unsqueeze(-1)).to(dtype)
    return un.sum(dim=1)


def tokens_per_expert(indices: torch.Tensor, num_experts: int) -> torch.Tensor:
    flat = indices.reshape(-1)
    return torch.bincount(flat[flat >= 0].long(), minlength=num_experts)
