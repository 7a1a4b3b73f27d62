"""GPU parity at the full BASELINE.json sizes (configs 2-5).

The CPU oracle cannot finish these in seconds, so each case combines
  * the oracle on sampled row blocks / groups (largest group, smallest non-empty group, a middle one),
  * size-independent properties: exact linearity under scaling by two, untouched sentinel rows,
    zero output for empty groups, and
  * a whole-output sweep against a library routine (torch's fp32 matmul on the GPU, group by group),
    to the same half-ulp bound the small cases use.
Inputs are drawn on the GPU from seeded generators (the sampled blocks are copied to the host for the oracle).
"""
import pytest
import torch

from oracle import gemm_ref
from tests._util import check_16bit_gemm
from triton_grouped_gemm_amd import workloads
from triton_grouped_gemm_amd.gemm.BF16.k_grouped_gemm_TMA import k_grouped_gemm
from triton_grouped_gemm_amd.gemm.BF16.m_grouped_gemm_masked_TMA import m_grouped_gemm_masked
from triton_grouped_gemm_amd.gemm.BF16.m_grouped_gemm_TMA import m_grouped_gemm
from triton_grouped_gemm_amd.gemm.deep_gemm_ops import m_grouped_fp8_nt_contiguous
from triton_grouped_gemm_amd.quant.fp8_cast import per_block_cast_to_fp8, per_token_cast_to_fp8

pytestmark = pytest.mark.gpu
G, M_TOTAL = 128, 655360


def _sample_groups(sizes_cpu):
    order = torch.argsort(sizes_cpu)
    nz = [int(i) for i in order if sizes_cpu[i] > 0]
    return sorted({nz[0], nz[-1], nz[len(nz) // 2]})


class _MaxNorm:
    """Whole-output max-norm rdiff against the fp32 product, max |out - ref| / max(|out|, |ref|) as the reference's
    scripts define it (gemm/BF16/utils.py), accumulated group by group; printed and attached to the test report."""

    def __init__(self):
        self.err = self.mag = 0.0

    def add(self, out, ref_fp32):
        o = out.float()
        self.err = max(self.err, float((o - ref_fp32).abs().max()))
        self.mag = max(self.mag, float(o.abs().max()), float(ref_fp32.abs().max()))

    def report(self, record_property, what):
        rd = self.err / self.mag if self.mag else 0.0
        record_property("max_norm_rdiff_vs_fp32", rd)
        print(f"\n[full size] {what}: max-norm rdiff against the fp32 product over the whole output = {rd:.3e}")
        return rd


class _StatedRdiff:
    """The stated BF16 bound, rdiff <= 1e-3 against the torch reference in the tensors' own dtype (what the
    reference's scripts compare with: torch's bf16 matmul per group on the same device, gemm/BF16/utils.py:5-14),
    on the whole output.  Asserted on the L2-relative difference, which one rounding flip cannot move; the max-norm
    form of the same comparison is printed beside it (a single flip of an element near the global maximum costs up to
    2^-8 there, whichever implementation produced either side)."""

    def __init__(self):
        self.num = self.den = 0.0
        self.err = self.mag = 0.0

    def add(self, out, ref_same_dtype):
        o, r = out.double(), ref_same_dtype.double()
        self.num += float(((o - r) ** 2).sum())
        self.den += float((r ** 2).sum())
        self.err = max(self.err, float((o - r).abs().max()))
        self.mag = max(self.mag, float(o.abs().max()), float(r.abs().max()))

    def check(self, record_property, what):
        l2 = (self.num / self.den) ** 0.5 if self.den else 0.0
        mx = self.err / self.mag if self.mag else 0.0
        record_property("l2_rdiff_vs_bf16_torch", l2)
        record_property("max_norm_rdiff_vs_bf16_torch", mx)
        print(f"[full size] {what}: against torch's bf16 matmul per group, L2 rdiff = {l2:.3e} (asserted <= 1e-3), max-norm rdiff = {mx:.3e}")
        assert l2 <= 1e-3, (what, l2)


def _half_ulp_ok(out_bf16, ref_fp32):
    err = (out_bf16.float() - ref_fp32).abs()
    bound = ref_fp32.abs() * (2.0 ** -8 * 1.05) + 2e-6 * ref_fp32.abs().max()
    return bool((err <= bound).all())


@pytest.mark.parametrize("N,K", [(1536, 2048), (2048, 768)])
@pytest.mark.parametrize("trans_b", [True, False])
def test_config2_m_grouped_full_size(dev, N, K, trans_b, record_property):
    sizes_cpu = workloads.dirichlet_multinomial_sizes(G, M_TOTAL, 128, seed=100)
    assert int(sizes_cpu.sum()) == M_TOTAL and bool((sizes_cpu % 128 == 0).all())
    sizes = sizes_cpu.to(dev)
    a = workloads.randn_bf16((M_TOTAL, K), K ** -0.5, 101, dev)
    b = workloads.randn_bf16((G, N, K) if trans_b else (G, K, N), K ** -0.5, 102, dev)
    out = m_grouped_gemm(a, b, sizes, trans_b)
    assert out.shape == (M_TOTAL, N) and out.dtype == torch.bfloat16
    starts = (sizes_cpu.cumsum(0) - sizes_cpu).tolist()
    # oracle on sampled groups (first 256 rows of each)
    for g in _sample_groups(sizes_cpu):
        s0, n = starts[g], min(int(sizes_cpu[g]), 256)
        ag, bg = a[s0:s0 + n].cpu(), b[g:g + 1].cpu()
        check_16bit_gemm(out[s0:s0 + n], gemm_ref.gmm(ag, bg, [n], trans_b), gemm_ref.gmm_fp32(ag, bg, [n], trans_b), f"g{g}")
    # every group against torch's fp32 matmul
    mn, stated = _MaxNorm(), _StatedRdiff()
    for g in range(G):
        s0, n = starts[g], int(sizes_cpu[g])
        if n == 0:
            continue
        w = b[g].float()
        ref = a[s0:s0 + n].float() @ (w.t() if trans_b else w)
        assert _half_ulp_ok(out[s0:s0 + n], ref), f"group {g}"
        mn.add(out[s0:s0 + n], ref)
        stated.add(out[s0:s0 + n], a[s0:s0 + n] @ (b[g].t() if trans_b else b[g]))
    stated.check(record_property, f"config 2 N={N} K={K} trans_b={trans_b}")
    # one bf16 rounding of the largest element costs up to 2^-8 = 3.9e-3 in this norm (half an ulp of a value just above a power of two), for any implementation
    assert mn.report(record_property, f"config 2 N={N} K={K} trans_b={trans_b}") <= 2.0 ** -8 * 1.06
    # linearity: doubling A doubles every output exactly
    out2 = m_grouped_gemm(a * 2, b, sizes, trans_b)
    assert torch.equal(out2, out * 2)


def test_config2_unaligned_sizes_full_size(dev):
    """Same shape with an unaligned multinomial draw over rows: exercises ragged boundary tiles."""
    gen = torch.Generator().manual_seed(103)
    gamma = torch._standard_gamma(torch.ones(G, dtype=torch.float64), generator=gen)
    draws = torch.multinomial(gamma / gamma.sum(), M_TOTAL, replacement=True, generator=gen)
    sizes_cpu = torch.bincount(draws, minlength=G).to(torch.int32)
    assert int(sizes_cpu.sum()) == M_TOTAL and bool((sizes_cpu % 128 != 0).any())
    N, K = 1536, 2048
    a = workloads.randn_bf16((M_TOTAL, K), K ** -0.5, 104, dev)
    b = workloads.randn_bf16((G, N, K), K ** -0.5, 105, dev)
    out = m_grouped_gemm(a, b, sizes_cpu.to(dev), True)
    starts = (sizes_cpu.cumsum(0) - sizes_cpu).tolist()
    for g in range(G):
        s0, n = starts[g], int(sizes_cpu[g])
        if n:
            assert _half_ulp_ok(out[s0:s0 + n], a[s0:s0 + n].float() @ b[g].float().t()), f"group {g}"
    for g in _sample_groups(sizes_cpu):
        s0, n = starts[g], int(sizes_cpu[g])
        lo = max(0, n - 200)  # the group's tail, where the boundary tile is
        ag, bg = a[s0 + lo:s0 + n].cpu(), b[g:g + 1].cpu()
        check_16bit_gemm(out[s0 + lo:s0 + n], gemm_ref.gmm(ag, bg, [n - lo], True), gemm_ref.gmm_fp32(ag, bg, [n - lo], True), f"g{g}")


def test_config3_masked_full_size(dev, record_property):
    m_max, N, K = 512, 4096, 1536
    mm_cpu = workloads.masked_counts(G, m_max, seed=106)
    mm_cpu[3], mm_cpu[7] = 0, m_max
    lhs = workloads.randn_bf16((G * m_max, K), K ** -0.5, 107, dev)
    valid = (torch.arange(m_max, device=dev)[None, :] < mm_cpu.to(dev)[:, None]).reshape(-1, 1)
    lhs = torch.where(valid, lhs, torch.full_like(lhs, float("nan")))  # rows beyond masked_m are garbage
    rhs = workloads.randn_bf16((G, N, K), K ** -0.5, 108, dev)
    out = torch.full((G * m_max, N), -3.0, device=dev, dtype=torch.bfloat16)
    assert m_grouped_gemm_masked(lhs, rhs, out, mm_cpu.to(dev), m_max) is None
    o3 = out.view(G, m_max, N)
    mn, stated = _MaxNorm(), _StatedRdiff()
    for g in range(G):
        mm = int(mm_cpu[g])
        assert bool((o3[g, mm:] == -3.0).all()), f"group {g}: rows beyond masked_m were written"
        if mm:
            ref = lhs.view(G, m_max, K)[g, :mm].float() @ rhs[g].float().t()
            assert _half_ulp_ok(o3[g, :mm], ref), f"group {g}"
            mn.add(o3[g, :mm], ref)
            stated.add(o3[g, :mm], lhs.view(G, m_max, K)[g, :mm] @ rhs[g].t())
    stated.check(record_property, "config 3 masked")
    assert mn.report(record_property, "config 3 masked") <= 2.0 ** -8 * 1.06
    for g in (7, int(torch.argmax(mm_cpu * (mm_cpu < m_max)))):
        mm = int(mm_cpu[g])
        ag, rg = lhs.view(G, m_max, K)[g, :mm].cpu(), rhs[g].cpu()
        check_16bit_gemm(o3[g, :mm], ag @ rg.t(), ag.float() @ rg.float().t(), f"masked g{g}")


def test_config4_k_grouped_full_size(dev, record_property):
    Md, Nd = 3072, 4096
    sizes_cpu = workloads.dirichlet_multinomial_sizes(G, M_TOTAL, 128, seed=109)
    sizes = sizes_cpu.to(dev)
    a = workloads.randn_bf16((M_TOTAL, Md), 1.0, 110, dev)
    b = workloads.randn_bf16((M_TOTAL, Nd), 1.0, 111, dev)
    out = k_grouped_gemm(a, b, sizes)
    assert out.shape == (G, Md, Nd)
    starts = (sizes_cpu.cumsum(0) - sizes_cpu).tolist()
    mn, stated = _MaxNorm(), _StatedRdiff()
    for g in range(G):
        s0, n = starts[g], int(sizes_cpu[g])
        if n == 0:
            assert torch.count_nonzero(out[g]) == 0
        else:
            ref = a[s0:s0 + n].float().t() @ b[s0:s0 + n].float()
            assert _half_ulp_ok(out[g], ref), f"group {g}"
            mn.add(out[g], ref)
            stated.add(out[g], a[s0:s0 + n].t() @ b[s0:s0 + n])
    assert mn.report(record_property, "config 4 K-grouped") <= 2.0 ** -8 * 1.06
    stated.check(record_property, "config 4 K-grouped")
    g = _sample_groups(sizes_cpu)[0]  # smallest non-empty group: the oracle finishes in seconds
    s0, n = starts[g], int(sizes_cpu[g])
    ag, bg = a[s0:s0 + n].cpu(), b[s0:s0 + n].cpu()
    check_16bit_gemm(out[g], ag.t() @ bg, ag.float().t() @ bg.float(), f"k-grouped g{g}")


def test_config5_fp8_block_scaled_full_size(dev, record_property):
    """A quantised on the GPU with the 1x128 recipe, B with the 128x128 recipe; compared with the fp32 matmul
    of the dequantised operands: rdiff <= 2e-2 (the stated FP8 target)."""
    N, K = 3072, 4096
    sizes_cpu = workloads.dirichlet_multinomial_sizes(G, M_TOTAL, 128, seed=112)
    a = workloads.randn_bf16((M_TOTAL, K), 1.0, 113, dev)
    aq, sa = per_token_cast_to_fp8(a, scales_mn_major=True)
    del a
    w = workloads.randn_bf16((G, N, K), 1.0, 114, dev)
    wq, sb = per_block_cast_to_fp8(w)
    del w
    out = m_grouped_fp8_nt_contiguous((aq, sa), (wq, sb), sizes_cpu.to(dev))
    starts = (sizes_cpu.cumsum(0) - sizes_cpu).tolist()
    worst = 0.0
    for g in range(G):
        s0, n = starts[g], int(sizes_cpu[g])
        if n == 0:
            continue
        ad = aq[s0:s0 + n].float() * sa[s0:s0 + n].repeat_interleave(128, dim=1)
        wd = wq[g].float() * sb[g].repeat_interleave(128, dim=0).repeat_interleave(128, dim=1)
        ref = ad @ wd.t()
        o = out[s0:s0 + n].float()
        worst = max(worst, ((o - ref).abs().max() / max(o.abs().max(), ref.abs().max())).item())
    record_property("max_norm_rdiff_vs_fp32", worst)
    print(f"\n[full size] config 5 FP8 block-scaled: worst per-group max-norm rdiff against the fp32 product of the dequantised operands = {worst:.3e}")
    assert worst <= 2e-2, worst
    assert worst <= 2.0 ** -7, worst  # the bf16 output rounding dominates (the MFMA's own truncation is ~2^-13)
    # CPU oracle on one sampled block
    g = _sample_groups(sizes_cpu)[1]
    s0, n = starts[g], min(int(sizes_cpu[g]), 128)
    ref = gemm_ref.fp8_block_scaled_reference(aq[s0:s0 + n].float().cpu(), sa[s0:s0 + n].cpu().contiguous(),
                                              wq[g:g + 1].float().cpu(), sb[g:g + 1].cpu(), [n])
    assert gemm_ref.rdiff(out[s0:s0 + n].float().cpu(), ref[:n]) <= 2.0 ** -7
