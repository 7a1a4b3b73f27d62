"""Differentiable grouped GEMM (forward NT/NN, activation gradient, weight gradient through the K-grouped kernel)
against torch autograd on the CPU per-group loop.  Problems and structure follow the reference's own test of its
autograd wrapper (grouped_gemm/grouped_gemm/ops_test.py:30-115), with the tolerances of the other GEMM tests
instead of its "2% of values may differ" rule."""
import pytest
import torch

from oracle import gemm_ref
from tests._util import check_16bit_gemm
from triton_grouped_gemm_amd import ops

pytestmark = pytest.mark.gpu

PROBLEMS = [(1, 128, 128, 128), (8, 128, 128, 128), (16, 128, 128, 128), (1, 128, 256, 512), (8, 128, 256, 512),
            (16, 128, 256, 512)]


def _randn(shape, seed):
    g = torch.Generator().manual_seed(seed)
    return (torch.randn(shape, generator=g) * shape[-1] ** -0.5).to(torch.bfloat16)


def _reference(a, b, sizes, trans_b, w):
    """fp32 autograd through the per-group loop on the CPU (operands are the bf16 values)."""
    a32 = a.float().requires_grad_(True)
    b32 = b.float().requires_grad_(True)
    out = gemm_ref.gmm_fp32(a32, b32, sizes, trans_b)
    (out * w.float()).sum().backward()
    return out.detach(), a32.grad, b32.grad


def _run(dev, z, m, k, n, trans_b, sizes, sizes_on_device):
    a = _randn((z * m, k), 1)
    b = _randn((z, n, k) if trans_b else (z, k, n), 2)
    w = _randn((z * m, n), 3)  # upstream gradient (bf16-representable)
    ref_out, ref_da, ref_db = _reference(a, b, sizes, trans_b, w)
    ad = a.to(dev).requires_grad_(True)
    bd = b.to(dev).requires_grad_(True)
    bs = torch.tensor(sizes, dtype=torch.int64)
    out = ops.gmm(ad, bd, bs.to(dev) if sizes_on_device else bs, trans_b)
    out.backward(w.to(dev))
    assert out.dtype == torch.bfloat16 and ad.grad.shape == a.shape and bd.grad.shape == b.shape
    check_16bit_gemm(out.detach(), ref_out.to(torch.bfloat16), ref_out, "forward")
    # d a = w @ b(.T): the same kind of GEMM; d b[g] = a_g.T @ w_g (or its transpose), fp32 accumulation over the rows
    check_16bit_gemm(ad.grad, ref_da.to(torch.bfloat16), ref_da, "grad a")
    for g, s in enumerate(sizes):
        if s == 0:
            assert torch.count_nonzero(bd.grad[g]) == 0
    check_16bit_gemm(bd.grad.reshape(-1, bd.grad.shape[-1]), ref_db.reshape(-1, ref_db.shape[-1]).to(torch.bfloat16),
                     ref_db.reshape(-1, ref_db.shape[-1]), "grad b")


@pytest.mark.parametrize("trans_b", [False, True])
@pytest.mark.parametrize("z,m,k,n", PROBLEMS)
def test_fixed_sizes(dev, z, m, k, n, trans_b):
    _run(dev, z, m, k, n, trans_b, [m] * z, sizes_on_device=False)


@pytest.mark.parametrize("trans_b", [False, True])
@pytest.mark.parametrize("z,m,k,n", PROBLEMS)
def test_variable_sizes(dev, z, m, k, n, trans_b):
    g = torch.Generator().manual_seed(z * 1000 + n)
    dist = torch.rand(z, generator=g)
    sizes = (dist / dist.sum() * m * z).to(torch.long)
    sizes[-1] += m * z - sizes.sum()
    _run(dev, z, m, k, n, trans_b, sizes.tolist(), sizes_on_device=True)


def test_empty_group_and_no_weight_grad(dev):
    sizes = [100, 0, 156]
    a = _randn((256, 64), 4).to(dev).requires_grad_(True)
    b = _randn((3, 64, 72), 5).to(dev)  # no gradient wanted for b
    out = ops.gmm(a, b, torch.tensor(sizes), trans_b=False)
    out.sum().backward()
    exp = gemm_ref.gmm_fp32(torch.ones(256, 72), b.cpu().float(), sizes, True)  # ones @ b[g].T
    check_16bit_gemm(a.grad, exp.to(torch.bfloat16), exp, "grad a")
    assert b.grad is None


def test_all_zero_host_sizes_are_rejected(dev):
    a = _randn((8, 16), 6).to(dev)
    b = _randn((2, 16, 16), 7).to(dev)
    with pytest.raises(AssertionError, match="should not be all zeros"):
        ops.gmm(a, b, torch.tensor([0, 0]))
