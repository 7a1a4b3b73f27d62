"""Operands larger than 4 GiB: byte offsets that do not fit 32 bits.

A card with 288 GB of memory is handed activation buffers of several GiB.  Every case here places a group (and a
tile inside it) across the byte offset 2^32 of at least one operand and checks the rows on both sides of it:
  * against torch's fp32 (or fp64) matmul of the same rows on the GPU, to the half-ulp bound of the small cases,
  * against the CPU oracle on a block of rows around the mark,
  * tuned kernel against generic kernel over the whole output, bit for bit (16-bit GEMMs).
The quantizer and the row movers are checked bit-exactly on rows beyond the mark.
"""
import numpy as np
import pytest
import torch

from oracle import gemm_ref, permute_ref, quant_ref
from tests._util import check_16bit_gemm, codes_np, to_np_f32
from triton_grouped_gemm_amd import _native, ops, workloads
from triton_grouped_gemm_amd.gemm.BF16.k_grouped_gemm_TMA import k_grouped_gemm
from triton_grouped_gemm_amd.gemm.BF16.m_grouped_gemm_masked_TMA import m_grouped_gemm_masked
from triton_grouped_gemm_amd.gemm.BF16.m_grouped_gemm_TMA import m_grouped_gemm
from triton_grouped_gemm_amd.gemm.deep_gemm_ops import m_grouped_fp8_nt_contiguous
from triton_grouped_gemm_amd.quant.fp8_cast import per_block_cast_to_fp8, per_token_cast_to_fp8

pytestmark = pytest.mark.gpu

# Rows of 4096 bytes (2048 bf16 / 4096 fp8 values) reach byte 2^32 at row MARK.
MARK = (1 << 32) // 4096
SIZES = [500_003, 0, 548_700, 3, 101_294]      # group 2 covers rows 500 003 .. 1 048 703: MARK lies inside a tile
SIZES_128 = [500_096, 0, 548_608, 128, 101_248]  # the same with 128-aligned groups
BLOCKS = [(0, 300), (MARK - 600, MARK + 600), (sum(SIZES) - 500, sum(SIZES))]


def _half_ulp_ok(out_bf16, ref, slack=2e-6):
    ref = ref.float()
    err = (out_bf16.float() - ref).abs()
    return bool((err <= ref.abs() * (2.0 ** -8 * 1.05) + slack * ref.abs().max()).all())


def _group_of(row, sizes):
    start = 0
    for g, n in enumerate(sizes):
        if start <= row < start + n:
            return g
        start += n
    raise AssertionError(row)


def _tuned_and_generic(fn):
    _native.set_option("force_generic", 1)
    try:
        ref = fn()
    finally:
        _native.set_option("force_generic", 0)
    return fn(), ref


@pytest.mark.parametrize("trans_b", [True, False])
def test_m_grouped_bf16_operands_and_output_beyond_4gib(dev, trans_b):
    M, N, K = sum(SIZES), 2048, 2048
    assert M * K * 2 > 1 << 32 and M * N * 2 > 1 << 32
    a = workloads.randn_bf16((M, K), K ** -0.5, 301, dev)
    b = workloads.randn_bf16((len(SIZES), N, K) if trans_b else (len(SIZES), K, N), 1.0, 302, dev)
    sizes = torch.tensor(SIZES, dtype=torch.int64, device=dev)
    out, ref = _tuned_and_generic(lambda: m_grouped_gemm(a, b, sizes, trans_b))
    assert torch.equal(out, ref)
    del ref
    for lo, hi in BLOCKS:
        for r0 in range(lo, hi, 100):  # pieces that stay inside one group
            g = _group_of(r0, SIZES)
            r1 = min(r0 + 100, hi, sum(SIZES[:g + 1]))
            w = b[g].float()
            assert _half_ulp_ok(out[r0:r1], a[r0:r1].float() @ (w.t() if trans_b else w)), (r0, r1)
    r0, r1 = MARK - 100, MARK + 100
    ag, bg = a[r0:r1].cpu(), b[2:3].cpu()
    check_16bit_gemm(out[r0:r1], gemm_ref.gmm(ag, bg, [r1 - r0], trans_b), gemm_ref.gmm_fp32(ag, bg, [r1 - r0], trans_b),
                     "rows around 4 GiB")


def test_k_grouped_bf16_operand_beyond_4gib(dev):
    M, Md, Nd = sum(SIZES), 2048, 256
    a = workloads.randn_bf16((M, Md), 1.0, 303, dev)
    b = workloads.randn_bf16((M, Nd), 1.0, 304, dev)
    assert a.numel() * 2 > 1 << 32
    sizes = torch.tensor(SIZES, dtype=torch.int32, device=dev)
    out, ref = _tuned_and_generic(lambda: k_grouped_gemm(a, b, sizes))
    assert out.shape == (len(SIZES), Md, Nd) and torch.equal(out, ref)
    assert torch.count_nonzero(out[1]) == 0
    start = 0
    for g, n in enumerate(SIZES):
        if n:
            # half a million terms per output: fp64 reference on a slice of the rows of the output; the slack
            # covers the fp32 accumulation of that many products
            ref64 = a[start:start + n, :256].double().t() @ b[start:start + n].double()
            assert _half_ulp_ok(out[g, :256], ref64, slack=2e-5), f"group {g}"
        start += n
    # the three-token group, wholly beyond the mark, pins which rows went where
    s3 = sum(SIZES[:3])
    assert s3 > MARK
    exact = a[s3:s3 + 3].float().t() @ b[s3:s3 + 3].float()
    assert _half_ulp_ok(out[3], exact)


def test_masked_bf16_operand_beyond_4gib(dev):
    G, m_max, N, K = 80, 7168, 256, 4096
    assert G * m_max * K * 2 > 1 << 32
    mark_group = (1 << 32) // (m_max * K * 2)  # the expert whose block contains byte 2^32
    gen = torch.Generator().manual_seed(305)
    mm_cpu = torch.randint(0, m_max + 1, (G,), generator=gen, dtype=torch.int32)
    mm_cpu[mark_group], mm_cpu[G - 1], mm_cpu[5] = m_max, m_max - 3, 0
    lhs = workloads.randn_bf16((G * m_max, K), K ** -0.5, 306, dev)
    rhs = workloads.randn_bf16((G, N, K), 1.0, 307, dev)
    mm = mm_cpu.to(dev)

    def run():
        o = torch.full((G * m_max, N), -3.0, device=dev, dtype=torch.bfloat16)
        assert m_grouped_gemm_masked(lhs, rhs, o, mm, m_max) is None
        return o

    out, ref = _tuned_and_generic(run)
    assert torch.equal(out, ref)
    o3, l3 = out.view(G, m_max, N), lhs.view(G, m_max, K)
    for g in range(G):
        n = int(mm_cpu[g])
        assert bool((o3[g, n:] == -3.0).all()), f"group {g}: rows beyond masked_m were written"
        if n:
            assert _half_ulp_ok(o3[g, :n], l3[g, :n].float() @ rhs[g].float().t()), f"group {g}"
    r0 = (1 << 32) // (K * 2) - mark_group * m_max  # the row of that expert at byte 2^32
    assert 64 <= r0 <= m_max - 64
    ag, rg = l3[mark_group, r0 - 64:r0 + 64].cpu(), rhs[mark_group].cpu()
    check_16bit_gemm(o3[mark_group, r0 - 64:r0 + 64], ag @ rg.t(), ag.float() @ rg.float().t(), "rows around 4 GiB")


def test_fp8_cast_and_block_scaled_gemm_beyond_4gib(dev):
    M, N, K = sum(SIZES_128), 256, 4096
    a = workloads.randn_bf16((M, K), 1.0, 308, dev)  # 8192-byte rows: 2^32 at row MARK / 2
    aq, sa = per_token_cast_to_fp8(a, scales_mn_major=True)  # 4096-byte rows: 2^32 at row MARK
    assert aq.numel() > 1 << 32
    # the quantizer, bit-exact on rows around both marks and at the end
    for r0, r1 in [(MARK // 2 - 40, MARK // 2 + 40), (MARK - 40, MARK + 40), (M - 40, M)]:
        rc, rs = quant_ref.per_token_cast_to_fp8(to_np_f32(a[r0:r1]), "e4m3fn")
        assert np.array_equal(codes_np(aq[r0:r1]), rc), (r0, r1)
        assert np.array_equal(sa[r0:r1].cpu().contiguous().numpy().view(np.uint32), rs.view(np.uint32)), (r0, r1)
    del a
    w = workloads.randn_bf16((len(SIZES_128), N, K), 1.0, 309, dev)
    wq, sb = per_block_cast_to_fp8(w)
    del w
    out = m_grouped_fp8_nt_contiguous((aq, sa), (wq, sb), torch.tensor(SIZES_128, dtype=torch.int32, device=dev))
    for lo, hi in [(0, 256), (MARK - 512, MARK + 512), (M - 256, M)]:
        for r0 in range(lo, hi, 128):
            g = _group_of(r0, SIZES_128)
            r1 = min(r0 + 128, hi, sum(SIZES_128[:g + 1]))
            ad = aq[r0:r1].float() * sa[r0:r1].repeat_interleave(128, dim=1)
            wd = wq[g].float() * sb[g].repeat_interleave(128, dim=0).repeat_interleave(128, dim=1)
            ref = ad @ wd.t()
            o = out[r0:r1].float()
            assert ((o - ref).abs().max() / max(o.abs().max(), ref.abs().max())).item() <= 2.0 ** -7, (r0, r1)
    r0, r1 = MARK - 64, MARK + 64
    ref = gemm_ref.fp8_block_scaled_reference(aq[r0:r1].float().cpu(), sa[r0:r1].cpu().contiguous(),
                                              wq[2:3].float().cpu(), sb[2:3].cpu(), [r1 - r0])
    assert gemm_ref.rdiff(out[r0:r1].float().cpu(), ref[:r1 - r0]) <= 2.0 ** -7


def test_permute_unpermute_beyond_4gib(dev):
    T, H, topk, E = 150_000, 4096, 4, 64
    assert T * topk * H * 2 > 1 << 32
    gen = torch.Generator(device=dev).manual_seed(310)
    x = torch.rand((T, H), device=dev, generator=gen).to(torch.bfloat16)
    scores = torch.rand((T, E), device=dev, generator=gen)
    indices = scores.topk(topk, dim=1).indices.to(torch.int32)  # distinct experts per token
    perm, rmap = ops.permute(x, indices, num_experts=E)
    assert torch.equal(rmap.cpu(), permute_ref.row_id_map(indices.cpu()))
    order = torch.argsort(indices.flatten().to(torch.int64), stable=True)
    assert perm.shape == (T * topk, H)
    for r0 in range(0, T * topk, 100_000):  # rows are moved, not recomputed: bit-exact
        src = torch.div(order[r0:r0 + 100_000], topk, rounding_mode="floor")
        assert torch.equal(perm[r0:r0 + 100_000], x[src]), r0
    un = ops.unpermute(perm, rmap)  # without probs every assignment is its own token (the reference's topK = 1 case)
    assert un.shape == (T * topk, H)
    for k in range(topk):
        assert torch.equal(un[k * T:(k + 1) * T], x), k
    del un
    quarter = torch.full((T, topk), 0.25, device=dev)
    assert torch.equal(ops.unpermute(perm, rmap, quarter), x)  # four exact quarters of one bf16 value sum exactly


def test_fp8_channel_operands_beyond_4gib(dev):
    """Per-channel FP8, M-grouped (A of 4.7 GB) and K-grouped (x of 4.7 GB, tokens along K): rows on both sides of
    byte 2^32 against torch's fp32 matmul; the bound allows for the matrix instruction's product truncation."""
    from triton_grouped_gemm_amd.gemm.FP8.k_grouped_gemm_channel_expert import matmul as k_grouped_fp8
    from triton_grouped_gemm_amd.gemm.FP8.m_grouped_gemm_channel_expert import gmm_fp8_act_per_channel_w_per_expert

    def close(out, ref, mag):
        err = (out.float() - ref).abs()
        return bool((err <= ref.abs() * (2.0 ** -8 * 1.05) + 2.0 ** -12 * mag + 1e-30).all())

    gen = torch.Generator(device=dev).manual_seed(311)
    M, N, K = sum(SIZES), 256, 4096
    a = workloads.randn_bf16((M, K), 1.0, 312, dev).to(torch.float8_e4m3fn)
    assert a.numel() > 1 << 32
    w = workloads.randn_bf16((len(SIZES), N, K), 1.0, 313, dev).to(torch.float8_e4m3fn)
    sa = torch.rand(M, 1, device=dev, generator=gen) + 0.5
    sb = torch.rand(len(SIZES) * N, device=dev, generator=gen) + 0.5
    out = gmm_fp8_act_per_channel_w_per_expert(a, sa, w, sb, torch.tensor(SIZES, dtype=torch.int32, device=dev), torch.bfloat16)
    for lo, hi in BLOCKS:
        for r0 in range(lo, hi, 100):
            g = _group_of(r0, SIZES)
            r1 = min(r0 + 100, hi, sum(SIZES[:g + 1]))
            scale = sa[r0:r1] * sb[g * N:(g + 1) * N][None, :]
            ref = (a[r0:r1].float() @ w[g].float().t()) * scale
            mag = (a[r0:r1].float().abs() @ w[g].float().abs().t()) * scale
            assert close(out[r0:r1], ref, mag), (r0, r1)
    del a, w, out
    # K-grouped: x [Md, Ktot], y [Nd, Ktot]; row r of x starts at byte r * Ktot, so rows from 2^32 / Ktot on lie beyond
    tokens = [128 * n for n in (3000, 0, 9000, 1, 5187)]
    Ktot, Md, Nd, G = sum(tokens), 2048, 256, len(tokens)
    assert Md * Ktot > 1 << 32
    x = workloads.randn_bf16((Md, Ktot), 1.0, 314, dev).to(torch.float8_e4m3fn)
    y = workloads.randn_bf16((Nd, Ktot), 1.0, 315, dev).to(torch.float8_e4m3fn)
    xs = torch.rand(Md, G, device=dev, generator=gen) + 0.5
    ys = torch.rand(Nd, G, device=dev, generator=gen) + 0.5
    out = k_grouped_fp8(x, xs, y, ys, torch.tensor(tokens, dtype=torch.int32, device=dev), Md, Nd, Ktot, G)
    assert out.shape == (G, Md, Nd) and torch.count_nonzero(out[1]) == 0
    row_mark = (1 << 32) // Ktot
    rows = torch.cat([torch.arange(0, 64), torch.arange(row_mark - 64, row_mark + 64), torch.arange(Md - 64, Md)]).to(dev)
    start = 0
    for g, n in enumerate(tokens):
        if n:
            xg, yg = x[rows, start:start + n].float(), y[:, start:start + n].float()
            scale = xs[rows, g][:, None] * ys[:, g][None, :]
            assert close(out[g][rows], (xg @ yg.t()) * scale, (xg.abs() @ yg.abs().t()) * scale), f"group {g}"
        start += n
