"""Differentiable grouped GEMM: forward, activation gradient and weight gradient on the three native kernels.

Mirrors the autograd wrapper of the reference's baseline extension (grouped_gemm/grouped_gemm/ops.py:12-42):
``gmm(a, b, batch_sizes, trans_b=False, num_sm=-1)`` with

    forward   out = a[rows of g] @ b[g]      (or @ b[g].T with trans_b)        M-grouped, layout NN / NT
    d a       grad @ b[g].T                  (or grad @ b[g])                  M-grouped with trans_b flipped
    d b       a_g.T @ grad_g   ([K, N])      (or grad_g.T @ a_g, [N, K])       K-grouped over the group's rows

``batch_sizes`` may live on the host (as the reference's extension requires) or on the device; a device tensor
is used as is, with no host synchronisation.
"""
import torch

from ._native import require_gpu
from .gemm.BF16.k_grouped_gemm import k_grouped_gemm
from .gemm.BF16.m_grouped_gemm import m_grouped_gemm


def _device_sizes(batch_sizes: torch.Tensor, device: torch.device) -> torch.Tensor:
    if batch_sizes.dtype not in (torch.int32, torch.int64):
        batch_sizes = batch_sizes.to(torch.int64)
    return batch_sizes.to(device, non_blocking=True)


class GroupedGemm(torch.autograd.Function):
    """grouped_gemm/grouped_gemm/ops.py:12-38."""

    @staticmethod
    def forward(ctx, a, b, batch_sizes, trans_b, num_sm=-1):
        if not batch_sizes.is_cuda:
            # the reference asserts this on its host-side sizes; device-resident sizes are not read back
            assert torch.count_nonzero(batch_sizes) != 0, "Input batch_sizes should not be all zeros!"
        require_gpu(a, b)
        sizes = _device_sizes(batch_sizes, a.device)
        ctx.save_for_backward(a, b, sizes)
        ctx.trans_b = bool(trans_b)
        ctx.num_sm = int(num_sm)
        return m_grouped_gemm(a.contiguous(), b.contiguous(), sizes, ctx.trans_b, ctx.num_sm)

    @staticmethod
    def backward(ctx, grad):
        grad = grad.contiguous()
        a, b, sizes = ctx.saved_tensors
        trans_b = ctx.trans_b
        agrad = None
        if ctx.needs_input_grad[0]:
            agrad = m_grouped_gemm(grad, b.contiguous(), sizes, not trans_b, ctx.num_sm)
        bgrad = None
        if ctx.needs_input_grad[1]:
            lhs, rhs = (grad, a) if trans_b else (a, grad)
            bgrad = k_grouped_gemm(lhs.contiguous(), rhs.contiguous(), sizes, numSM=ctx.num_sm)
        return agrad, bgrad, None, None, None


def gmm(a, b, batch_sizes, trans_b=False, num_sm=-1):
    """grouped_gemm/grouped_gemm/ops.py:41-42."""
    return GroupedGemm.apply(a, b, batch_sizes, trans_b, num_sm)
