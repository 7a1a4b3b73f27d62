"""MoE permute / unpermute against the torch reference of the reference's own test
(grouped_gemm/grouped_gemm/permute_test.py): same generator of inputs (randperm expert choice per token,
normalised random probs), forward and backward of both ops.  Integer results (row_id_map, counts, moved rows) are
bit-exact; the weighted sums are compared in fp32 with half-ulp style bounds."""
import pytest
import torch

from oracle import permute_ref
from triton_grouped_gemm_amd import ops

pytestmark = pytest.mark.gpu


def _case(num_token, num_expert, hidden, topk, dtype, seed=0):
    g = torch.Generator().manual_seed(seed)
    x = torch.rand((num_token, hidden), generator=g).to(dtype)
    if num_token:
        indices = torch.stack([torch.randperm(num_expert, generator=g)[:topk] for _ in range(num_token)]).to(torch.int32)
    else:
        indices = torch.empty((0, topk), dtype=torch.int32)
    probs = torch.rand(num_token, topk, generator=g)
    probs = probs / probs.sum(dim=1, keepdim=True)
    return x, indices, probs


def _close(out, ref32, dtype, terms=1):
    eps = {torch.bfloat16: 2.0 ** -8, torch.float16: 2.0 ** -11, torch.float32: 2.0 ** -23}[dtype]
    err = (out.float().cpu() - ref32).abs()
    bound = ref32.abs() * eps * 1.02 + terms * 2.0 ** -22 * ref32.abs().max().clamp_min(1e-30)
    assert bool((err <= bound).all()), float((err - bound).max())


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16, torch.float32])
@pytest.mark.parametrize("num_token,num_expert,hidden,topk", [
    (4096, 8, 512, 2), (1000, 64, 264, 6), (777, 256, 4096, 8), (5, 3, 8, 1), (2048, 1024, 128, 4)])
def test_forward_backward(dev, dtype, num_token, num_expert, hidden, topk):
    x, indices, probs = _case(num_token, num_expert, hidden, topk, dtype)
    # ---- reference (CPU torch; activations in fp32 for the gradient checks)
    ref_perm, order = permute_ref.permute(x, indices)
    ref_map = permute_ref.row_id_map(indices)
    # ---- permute forward
    xd = x.to(dev).requires_grad_(True)
    perm, rmap = ops.permute(xd, indices.to(dev), num_experts=num_expert)
    assert torch.equal(rmap.cpu(), ref_map)
    assert torch.equal(perm.detach().cpu(), ref_perm)  # rows are moved, not recomputed: bit-exact
    # ---- permute backward: grad of x[t] = sum over its topk copies
    gperm = torch.rand(perm.shape, generator=torch.Generator().manual_seed(1)).to(dtype)
    perm.backward(gperm.to(dev))
    ref_gx = torch.zeros(num_token, hidden).index_add_(0, order // topk, gperm.float())
    _close(xd.grad, ref_gx, dtype, topk)
    # ---- unpermute forward with probs
    pd = probs.to(dev).requires_grad_(True)
    ud_in = perm.detach().clone().requires_grad_(True)
    un = ops.unpermute(ud_in, rmap, pd)
    p32 = probs.clone().requires_grad_(True)
    u32_in = ref_perm.float().clone().requires_grad_(True)
    ref_un = permute_ref.unpermute(u32_in, order, p32, fp32=True)
    _close(un.detach(), ref_un.detach(), dtype, topk)
    # ---- unpermute backward: activation and prob gradients
    gun = torch.rand(un.shape, generator=torch.Generator().manual_seed(2)).to(dtype)
    un.backward(gun.to(dev))
    ref_un.backward(gun.float())
    _close(ud_in.grad, u32_in.grad, dtype)
    pg, rpg = pd.grad.cpu(), p32.grad
    assert torch.allclose(pg, rpg, rtol=1e-5, atol=1e-6 * float(rpg.abs().max())), float((pg - rpg).abs().max())


def test_counts_are_the_group_sizes(dev):
    _, indices, _ = _case(3000, 40, 8, 4, torch.bfloat16, seed=3)
    for cd in (torch.int32, torch.int64):
        rmap, counts = ops.permute_map(indices.to(dev), num_experts=40, counts_dtype=cd)
        assert counts.dtype == cd
        assert torch.equal(counts.cpu().long(), permute_ref.tokens_per_expert(indices, 40))
        assert sorted(rmap.cpu().tolist()) == list(range(3000 * 4))  # a permutation of all rows


def test_dropped_assignments_and_capacity(dev):
    x, indices, _ = _case(500, 16, 64, 2, torch.bfloat16, seed=4)
    indices[::7, 1] = -1  # dropped assignments
    ref_map = permute_ref.row_id_map(indices)
    rmap, counts = ops.permute_map(indices.to(dev), num_experts=16)
    assert torch.equal(rmap.cpu(), ref_map)
    assert torch.equal(counts.cpu().long(), permute_ref.tokens_per_expert(indices, 16))
    kept = int((indices >= 0).sum())
    perm, rmap2 = ops.permute(x.to(dev), indices.to(dev), num_experts=16)
    order = torch.argsort(indices.reshape(-1), stable=True)[indices.numel() - kept:]
    assert torch.equal(perm[:kept].cpu(), x.index_select(0, order // 2))
    # capacity: only the first 300 permuted rows are kept
    ref_cap = permute_ref.row_id_map(indices, 300)
    perm_c, rmap_c = ops.permute(x.to(dev), indices.to(dev), num_out_tokens=300, num_experts=16)
    assert perm_c.shape == (300, 64) and torch.equal(rmap_c.cpu(), ref_cap)
    assert torch.equal(perm_c.cpu(), x.index_select(0, order[:300] // 2))
    # unpermute skips dropped assignments
    un = ops.unpermute(perm_c, rmap_c, torch.ones(500, 2, device=dev))
    exp = torch.zeros(500, 64)
    for k in range(2):
        rows = ref_cap[k * 500:(k + 1) * 500]
        ok = rows >= 0
        exp[ok] += perm_c.cpu().float()[rows[ok].long()]
    _close(un, exp, torch.bfloat16, 2)


def test_empty_input_passes_through(dev):
    x = torch.empty((0, 64), dtype=torch.bfloat16, device=dev)
    out, rmap = ops.permute(x, torch.empty((0, 2), dtype=torch.int32, device=dev))
    assert out.numel() == 0 and rmap is None


def test_feeds_the_grouped_gemm(dev):
    """permute -> grouped GEMM with the counts as size_per_group -> unpermute equals the dense per-token formula."""
    T, E, H, N, topk = 512, 8, 128, 64, 2
    x, indices, probs = _case(T, E, H, topk, torch.bfloat16, seed=5)
    w = (torch.randn(E, H, N, generator=torch.Generator().manual_seed(6)) * H ** -0.5).to(torch.bfloat16)
    perm, rmap = ops.permute(x.to(dev), indices.to(dev), num_experts=E)
    _, counts = ops.permute_map(indices.to(dev), num_experts=E)
    y = ops.gmm(perm, w.to(dev), counts, trans_b=False)
    out = ops.unpermute(y, rmap, probs.to(dev))
    ref = torch.zeros(T, N)
    for t in range(T):
        for k in range(topk):
            yk = (x[t].float() @ w[int(indices[t, k])].float()).to(torch.bfloat16).float()  # the GEMM's bf16 output
            ref[t] += probs[t, k] * yk
    err = (out.float().cpu() - ref).abs().max() / ref.abs().max()
    assert err <= 2.0 ** -7, float(err)
