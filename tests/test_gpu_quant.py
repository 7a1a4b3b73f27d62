"""GPU parity: FP8 quantizers through the C ABI, bit-exact against the numpy oracle."""
import ctypes

import numpy as np
import pytest
import torch

from oracle import fp8_soft, quant_ref
from tests._util import codes_np, to_np_f32
from triton_grouped_gemm_amd import _native
from triton_grouped_gemm_amd.quant.fp8_cast import per_block_cast_to_fp8, per_token_cast_to_fp8
from triton_grouped_gemm_amd.quant.trans_per_block_quant_expand_128x import trans_per_block_quant_expand_128x

pytestmark = pytest.mark.gpu
FMT = {torch.float8_e4m3fn: "e4m3fn", torch.float8_e5m2: "e5m2"}


def _randn(shape, seed, scale=1.0):
    g = torch.Generator().manual_seed(seed)
    return (torch.randn(shape, generator=g) * scale).to(torch.bfloat16)


@pytest.mark.parametrize("fmt,code", [("e4m3fn", _native.E4M3), ("e5m2", _native.E5M2)])
def test_hardware_fp8_conversion_equals_software_rne(dev, fmt, code):
    """Every bf16 bit pattern and a spread of fp32 values inside the clamp range: the hardware
    conversion used by the quantizers equals the software round-to-nearest-even encoder."""
    fmax = 448.0 if fmt == "e4m3fn" else 57344.0
    rng = np.random.default_rng(0)
    x = np.concatenate([fp8_soft.bf16_bits_to_f32(np.arange(65536, dtype=np.uint16)),
                        (rng.standard_normal(400000) * np.exp(rng.uniform(-25, 11, 400000))).astype(np.float32)])
    x = np.clip(np.nan_to_num(x, nan=0.0), -fmax, fmax).astype(np.float32)
    xin = torch.from_numpy(x).to(dev)
    out = torch.empty(x.shape[0], dtype=torch.uint8, device=dev)
    _native.call("tgg_cvt_f32_to_fp8", xin.data_ptr(), out.data_ptr(), x.shape[0], code, _native.stream_of(xin))
    enc = fp8_soft.encode_e4m3fn if fmt == "e4m3fn" else fp8_soft.encode_e5m2
    assert np.array_equal(out.cpu().numpy(), enc(x))


@pytest.mark.parametrize("dtype", [torch.float8_e4m3fn, torch.float8_e5m2])
@pytest.mark.parametrize("sizes,N", [
    ([128, 256], 128),
    ([5, 0, 130, 128, 1], 256),
    ([0, 0, 0], 128),
    ([300] * 7 + [77], 384),
    ([3, 0, 17] * 100, 128),  # 300 groups: the large group table
])
def test_trans_quant_bit_exact(dev, dtype, sizes, N):
    M = sum(sizes)
    x = _randn((max(M, 1), N), 80, 2.0)[:M]
    codes, scales, padded = trans_per_block_quant_expand_128x(x.to(dev), torch.tensor(sizes, dtype=torch.int32, device=dev),
                                                               dtype=dtype)
    rc, rs, rp = quant_ref.trans_per_block_quant_expand_128x(to_np_f32(x), sizes, FMT[dtype])
    assert codes.dtype == dtype and tuple(codes.shape) == rc.shape and tuple(scales.shape) == rs.shape
    assert padded.tolist() == rp.tolist()
    assert np.array_equal(scales.cpu().numpy().view(np.uint32), rs.view(np.uint32))
    assert np.array_equal(codes_np(codes), rc)


def _check_trans_quant(dev, x, sizes, dtype=torch.float8_e4m3fn, size_dtype=torch.int32):
    codes, scales, padded = trans_per_block_quant_expand_128x(
        x.to(dev), torch.tensor(sizes, dtype=size_dtype, device=dev), dtype=dtype)
    rc, rs, rp = quant_ref.trans_per_block_quant_expand_128x(to_np_f32(x), sizes, FMT[dtype])
    assert tuple(codes.shape) == rc.shape and tuple(scales.shape) == rs.shape
    assert padded.tolist() == rp.tolist()
    assert np.array_equal(scales.cpu().numpy().view(np.uint32), rs.view(np.uint32))
    assert np.array_equal(codes_np(codes), rc)


@pytest.mark.parametrize("N", [1152, 2048, 4096, 7168])
def test_trans_quant_bit_exact_wide(dev, N):
    """More than eight 128-column blocks per row (the GEMM tile order cuts such widths into column chunks; the
    quantizer must not follow it), ragged groups of three and more row blocks, an empty group."""
    sizes = [300, 0, 417, 128, 385, 1]
    x = _randn((sum(sizes), N), 90 + N % 7, 1.5)
    _check_trans_quant(dev, x, sizes)


def test_trans_quant_bit_exact_wide_many_groups(dev):
    """G > 256 (the large group table) at N = 2048, int64 sizes, e5m2."""
    sizes = [(i * 53) % 290 for i in range(300)]
    x = _randn((sum(sizes), 2048), 91)
    _check_trans_quant(dev, x, sizes, torch.float8_e5m2, torch.int64)


@pytest.mark.parametrize("n_chunk", [1, 2])
def test_trans_quant_ignores_gemm_tile_order_option(dev, n_chunk):
    """The column-chunk option of the GEMM tile order must not reach the quantizer."""
    sizes = [300, 0, 130, 128]
    x = _randn((sum(sizes), 512), 92)
    _native.set_option("n_chunk", n_chunk)
    try:
        _check_trans_quant(dev, x, sizes)
    finally:
        _native.set_option("n_chunk", 0)


def test_trans_quant_reference_self_test_shape(dev):
    """The shape of the reference's own self-test: 65536 x 7168 bf16, 32 groups of 2048 rows
    (quant/trans_per_block_quant_expand_128x.py:276-277), every block against the oracle."""
    sizes = [2048] * 32
    x = _randn((65536, 7168), 93)
    _check_trans_quant(dev, x, sizes)


def test_trans_quant_special_values(dev):
    """All-zero blocks (scale clamps to 1e-12, codes 0), huge and tiny magnitudes, exact ties."""
    sizes = [128, 128, 128]
    x = torch.zeros(384, 128, dtype=torch.bfloat16)
    x[128:256] = _randn((128, 128), 81, 1e30)
    x[256:] = _randn((128, 128), 82, 1e-30)
    x[256, 0] = 448.0 * 2.0 ** -100
    codes, scales, _ = trans_per_block_quant_expand_128x(x.to(dev), torch.tensor(sizes, dtype=torch.int64, device=dev))
    rc, rs, _ = quant_ref.trans_per_block_quant_expand_128x(to_np_f32(x), sizes)
    assert np.array_equal(scales.cpu().numpy().view(np.uint32), rs.view(np.uint32))
    assert np.array_equal(codes_np(codes), rc)
    assert scales[0, 0].item() == np.float32(1e-12)


def test_trans_quant_roundtrip_at_larger_size(dev):
    """Size-independent properties on a larger draw: dequantised codes within half an e4m3 step of the
    input, |codes| <= 448 with every non-empty block reaching it, tail zero."""
    G, N = 16, 1024
    sizes = [(i * 37) % 500 + 1 for i in range(G)]
    M = sum(sizes)
    x = _randn((M, N), 83)
    codes, scales, padded = trans_per_block_quant_expand_128x(x.to(dev), torch.tensor(sizes, dtype=torch.int32, device=dev))
    deq = codes.float() * scales.repeat_interleave(128, 0).repeat_interleave(128, 1)
    src = dst = 0
    for s, p in zip(sizes, padded.tolist()):
        blk = deq[:, dst:dst + s].t().cpu()
        ref = x[src:src + s].float()
        sc = scales[:, dst // 128:(dst + p) // 128].repeat_interleave(128, 0).repeat_interleave(128, 1)[:, :s].t().cpu()
        assert bool(((blk - ref).abs() <= sc * 16.0 * 1.0001 + 1e-12).all())  # half of the largest e4m3 step (32) times scale
        assert not codes[:, dst + s:dst + p].view(torch.uint8).any()
        src += s
        dst += p
    assert not codes[:, dst:].view(torch.uint8).any() and not scales[:, dst // 128:].any()
    assert (codes.view(torch.uint8) & 0x7F).max().item() == 0x7E


@pytest.mark.parametrize("rows,K", [(300, 512), (17, 128), (4096, 1024), (33, 384)])
@pytest.mark.parametrize("dtype", [torch.float8_e4m3fn, torch.float8_e5m2])
def test_per_token_cast_bit_exact(dev, dtype, rows, K):
    x = _randn((rows, K), 84, 3.0)
    x[7] = 0  # hits the 1e-4 clamp
    x[8, :128] *= 1e-6
    codes, scales = per_token_cast_to_fp8(x.to(dev), dtype)
    rc, rs = quant_ref.per_token_cast_to_fp8(to_np_f32(x), FMT[dtype])
    assert np.array_equal(scales.cpu().numpy().view(np.uint32), rs.view(np.uint32))
    assert np.array_equal(codes_np(codes), rc)
    codes2, scales2 = per_token_cast_to_fp8(x.to(dev), dtype, scales_mn_major=True)
    assert scales2.shape == scales.shape and (K == 128 or scales2.stride() == (1, rows))
    assert torch.equal(scales2, scales) and torch.equal(codes2.view(torch.uint8), codes.view(torch.uint8))


@pytest.mark.parametrize("shape", [(256, 384), (130, 200), (3, 136, 264), (2, 128, 128)])
def test_per_block_cast_bit_exact(dev, shape):
    x = _randn(shape, 85, 0.7)
    codes, scales = per_block_cast_to_fp8(x.to(dev))
    xs = to_np_f32(x).reshape((-1,) + shape[-2:])
    for b in range(xs.shape[0]):
        rc, rs = quant_ref.per_block_cast_to_fp8(xs[b])
        cb = codes_np(codes).reshape((-1,) + shape[-2:])[b]
        sb = scales.cpu().numpy().reshape((xs.shape[0],) + rs.shape)[b]
        assert np.array_equal(sb.view(np.uint32), rs.view(np.uint32))
        assert np.array_equal(cb, rc)
