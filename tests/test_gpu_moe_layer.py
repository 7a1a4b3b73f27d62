"""One MoE feed-forward layer end to end through the library's operators, forward and backward: top-k routing ->
ops.permute (stable expert-major order, tokens per expert from the same sort) -> ops.gmm gate/up projection ->
SwiGLU -> ops.gmm down projection -> ops.unpermute weighted by the routing probabilities.  This is the caller's
side of the grouped GEMMs (grouped_gemm/grouped_gemm/ops.py:12-42 and :52-257 are used together this way); every
piece has its own parity test, what is checked here is that they compose: sizes from the sort feed the GEMMs, the
K-grouped kernel produces the weight gradients of both projections, and gradients flow back through both row movers.

Reference: the same layer token by token in fp32 on the CPU (torch autograd), with the forward activations rounded
to bf16 at the points where the layer stores them (after each projection, after the activation, at the output).
The backward pass of the library also stores its intermediate gradients in bf16, which the reference does not
mirror: gradients are compared in the max norm and the L2 norm at 2e-2 / 1e-2, the forward output at 1e-2 / 4e-3.
"""
import pytest
import torch
import torch.nn.functional as F

from triton_grouped_gemm_amd import ops

pytestmark = pytest.mark.gpu


def _bf16(x):
    return x.to(torch.bfloat16).float()


def _reference_layer(x, w1, w2, idx, probs, out_grad):
    """fp32 layer over bf16-valued operands; returns output and the gradients of x, w1, w2, probs."""
    x32, w1_32, w2_32 = (t.float().requires_grad_(True) for t in (x, w1, w2))
    p32 = probs.clone().requires_grad_(True)
    tokens, topk = idx.shape
    out = torch.zeros(tokens, x.shape[1])
    for k in range(topk):
        e = idx[:, k].long()
        h = _bf16(torch.einsum("th,tfh->tf", x32, w1_32[e]))
        gate, up = h.chunk(2, dim=-1)
        act = _bf16(_bf16(F.silu(gate)) * up)
        y = _bf16(torch.einsum("tf,thf->th", act, w2_32[e]))
        out = out + p32[:, k:k + 1] * y
    out = _bf16(out)
    (out * out_grad.float()).sum().backward()
    return out.detach(), x32.grad, w1_32.grad, w2_32.grad, p32.grad


def _close(got, want, max_tol, l2_tol, what):
    got, want = got.float().cpu(), want.float()
    scale = want.abs().max().clamp_min(1e-30)
    rdiff = ((got - want).abs().max() / scale).item()
    l2 = ((got - want).norm() / want.norm().clamp_min(1e-30)).item()
    assert rdiff <= max_tol and l2 <= l2_tol, f"{what}: max-norm rdiff {rdiff:.3e}, L2 {l2:.3e}"


@pytest.mark.parametrize("tokens,hidden,ffn,experts,topk", [(384, 256, 128, 8, 2), (200, 128, 256, 16, 4)])
def test_moe_ffn_layer_forward_and_backward(dev, tokens, hidden, ffn, experts, topk):
    g = torch.Generator().manual_seed(tokens + experts)
    x = (torch.randn(tokens, hidden, generator=g)).to(torch.bfloat16)
    w1 = (torch.randn(experts, 2 * ffn, hidden, generator=g) * hidden ** -0.5).to(torch.bfloat16)
    w2 = (torch.randn(experts, hidden, ffn, generator=g) * ffn ** -0.5).to(torch.bfloat16)
    logits = torch.randn(tokens, experts, generator=g)
    logits[:, 3] = -1e9  # one expert gets no tokens: empty group in both GEMMs, zero weight gradient
    probs, idx = torch.softmax(logits, -1).topk(topk, dim=-1)
    idx = idx.to(torch.int32)
    out_grad = torch.randn(tokens, hidden, generator=g).to(torch.bfloat16)
    ref_out, ref_dx, ref_dw1, ref_dw2, ref_dp = _reference_layer(x, w1, w2, idx, probs, out_grad)

    xd, w1d, w2d = (t.to(dev).requires_grad_(True) for t in (x, w1, w2))
    pd = probs.to(dev).requires_grad_(True)
    idx_d = idx.to(dev)
    permuted, row_id_map = ops.permute(xd, idx_d, num_experts=experts)
    _, tokens_per_expert = ops.permute_map(idx_d, num_experts=experts)
    assert tokens_per_expert.tolist() == torch.bincount(idx.flatten().long(), minlength=experts).tolist()
    h = ops.gmm(permuted, w1d, tokens_per_expert, trans_b=True)
    gate, up = h.chunk(2, dim=-1)
    act = F.silu(gate) * up
    y = ops.gmm(act, w2d, tokens_per_expert, trans_b=True)
    out = ops.unpermute(y, row_id_map, pd)
    out.backward(out_grad.to(dev))

    assert out.dtype == torch.bfloat16 and out.shape == (tokens, hidden)
    _close(out.detach(), ref_out, 1e-2, 4e-3, "layer output")
    _close(xd.grad, ref_dx, 2e-2, 1e-2, "grad x")
    _close(w1d.grad, ref_dw1, 2e-2, 1e-2, "grad w1")
    _close(w2d.grad, ref_dw2, 2e-2, 1e-2, "grad w2")
    _close(pd.grad, ref_dp, 2e-2, 1e-2, "grad probs")
    assert torch.count_nonzero(w1d.grad[3]) == 0 and torch.count_nonzero(w2d.grad[3]) == 0
