"""GEMM with fused 1x128 FP8 quantisation of the output: bit-identical to the two separate kernels (each of which is
checked against the oracle elsewhere), and, on integer-valued inputs where the GEMM is exact, to the oracle chain
per-group matmul -> round to bf16 -> per_token_cast_to_fp8."""
import numpy as np
import pytest
import torch

from oracle import gemm_ref, quant_ref
from tests._util import to_np_f32
from triton_grouped_gemm_amd.gemm.BF16.m_grouped_gemm import m_grouped_gemm
from triton_grouped_gemm_amd.gemm.deep_gemm_ops import m_grouped_fp8_nt_contiguous
from triton_grouped_gemm_amd.gemm.fused import m_grouped_gemm_fp8_out
from triton_grouped_gemm_amd.quant.fp8_cast import per_block_cast_to_fp8, per_token_cast_to_fp8

pytestmark = pytest.mark.gpu
FMT = {torch.float8_e4m3fn: "e4m3fn", torch.float8_e5m2: "e5m2"}


def _randn(shape, seed, scale=1.0):
    g = torch.Generator().manual_seed(seed)
    return (torch.randn(shape, generator=g) * scale).to(torch.bfloat16)


def _valid_rows(sizes):
    return sum(sizes)


@pytest.mark.parametrize("dtype", [torch.float8_e4m3fn, torch.float8_e5m2])
@pytest.mark.parametrize("mn_major", [False, True])
@pytest.mark.parametrize("trans_b", [True, False])
@pytest.mark.parametrize("sizes,N,K", [
    ([128, 0, 300, 77], 256, 192),
    ([1, 255, 256, 257], 384, 72),
    ([700], 128, 64),
    ([5120, 3333], 1536, 512),
])
def test_same_bits_as_two_kernels(dev, dtype, mn_major, trans_b, sizes, N, K):
    M, G = sum(sizes), len(sizes)
    a = _randn((M, K), 1, K ** -0.5).to(dev)
    b = _randn((G, N, K) if trans_b else (G, K, N), 2).to(dev)
    s = torch.tensor(sizes, dtype=torch.int32, device=dev)
    codes, scales = m_grouped_gemm_fp8_out(a, b, s, trans_b, dtype, mn_major)
    rc, rs = per_token_cast_to_fp8(m_grouped_gemm(a, b, s, trans_b), dtype, mn_major)
    assert codes.dtype == dtype and codes.shape == (M, N) and scales.shape == (M, N // 128)
    assert scales.stride() == rs.stride()
    assert torch.equal(codes.view(torch.uint8), rc.view(torch.uint8))
    assert torch.equal(scales, rs)


def test_exact_against_the_oracle_chain(dev):
    g = torch.Generator().manual_seed(3)
    sizes, N, K = [100, 0, 412], 256, 128
    M = sum(sizes)
    a = torch.randint(-3, 4, (M, K), generator=g).to(torch.bfloat16)
    b = torch.randint(-3, 4, (3, N, K), generator=g).to(torch.bfloat16)
    codes, scales = m_grouped_gemm_fp8_out(a.to(dev), b.to(dev), torch.tensor(sizes, device=dev), True)
    ref = gemm_ref.gmm_fp32(a, b, sizes, True)          # integers up to 9 * 128: exact in fp32
    ref16 = ref.to(torch.bfloat16)
    rc, rs = quant_ref.per_token_cast_to_fp8(to_np_f32(ref16), "e4m3fn")
    assert np.array_equal(codes.view(torch.uint8).cpu().numpy(), rc)
    assert np.array_equal(scales.cpu().numpy().view(np.uint32), rs.view(np.uint32))


def test_rows_past_the_groups_are_untouched_and_feeds_the_second_gemm(dev):
    sizes = [256, 128]  # 128-aligned: the output is directly a valid A operand of the block-scaled GEMM
    M, N, K, N2 = 384, 256, 128, 128
    a = _randn((M, K), 4, K ** -0.5).to(dev)
    w1 = _randn((2, N, K), 5).to(dev)
    w2 = _randn((2, N2, N), 6, N ** -0.5).to(dev)
    s = torch.tensor(sizes, dtype=torch.int32, device=dev)
    codes, scales = m_grouped_gemm_fp8_out(a, w1, s, True, scales_mn_major=True)
    out = m_grouped_fp8_nt_contiguous((codes, scales), per_block_cast_to_fp8(w2), s)
    h = m_grouped_gemm(a, w1, s, True)
    ref = m_grouped_fp8_nt_contiguous(per_token_cast_to_fp8(h, scales_mn_major=True), per_block_cast_to_fp8(w2), s)
    assert torch.equal(out, ref)
    # fewer valid rows than M: the tail keeps what was there
    codes2 = torch.full((M, N), 0x55, dtype=torch.uint8, device=dev).view(torch.float8_e4m3fn)
    short = torch.tensor([100, 50], dtype=torch.int32, device=dev)
    c3, s3 = m_grouped_gemm_fp8_out(a, w1, short, True)
    r3c, r3s = per_token_cast_to_fp8(m_grouped_gemm(a, w1, short, True))
    assert torch.equal(c3.view(torch.uint8)[:150], r3c.view(torch.uint8)[:150]) and torch.equal(s3[:150], r3s[:150])
    del codes2


def test_more_groups_than_the_fused_kernel_takes(dev):
    G = 600
    sizes = [2] * G
    a = _randn((2 * G, 64), 7).to(dev)
    b = _randn((G, 128, 64), 8).to(dev)
    s = torch.tensor(sizes, dtype=torch.int32, device=dev)
    codes, scales = m_grouped_gemm_fp8_out(a, b, s, True)
    rc, rs = per_token_cast_to_fp8(m_grouped_gemm(a, b, s, True))
    assert torch.equal(codes.view(torch.uint8), rc.view(torch.uint8)) and torch.equal(scales, rs)
