"""The reference's own GPU scripts, as tests: same problems, same comparison, same tolerances.

The reference ships `__main__` scripts rather than collected tests (tests/test_BF16/test_m_grouped_gemm_TMA.py:37-103,
test_m_grouped_gemm_masked_TMA.py:35-107, test_k_grouped_gemm_TMA.py:42-106, tests/test_FP8/*.py).  Each draws 128
group sizes with `generate_random_list`, runs the four (n, k) shapes (1536, 2048), (2048, 768), (3072, 4096),
(4096, 1536), normalises every output row to a largest magnitude of one and calls `torch.testing.assert_close`
against the per-group torch loop.  Here the same steps run through this library's entry points (the profiler
parts of the scripts are left out; the random draw is seeded).  The FP8 scripts only print their rdiff; here it is
also asserted against the fp32 product of the dequantised operands.
"""
import random

import pytest
import torch

from triton_grouped_gemm_amd.gemm.BF16.k_grouped_gemm_TMA import k_grouped_gemm
from triton_grouped_gemm_amd.gemm.BF16.m_grouped_gemm_masked_TMA import m_grouped_gemm_masked
from triton_grouped_gemm_amd.gemm.BF16.m_grouped_gemm_TMA import m_grouped_gemm
from triton_grouped_gemm_amd.gemm.BF16.utils import generate_random_list, gmm, row_max_normalization
from triton_grouped_gemm_amd.gemm.FP8.k_grouped_gemm_channel_expert import matmul as k_grouped_fp8
from triton_grouped_gemm_amd.gemm.FP8.m_grouped_gemm_channel_expert import gmm_fp8_act_per_channel_w_per_expert

pytestmark = pytest.mark.gpu
GROUPS = 128
SHAPES = [(768 * 2, 2048), (2048, 768), (1536 * 2, 4096), (4096, 1536)]


def _randn(shape, seed, dev):
    g = torch.Generator(device=dev).manual_seed(seed)
    out = torch.empty(shape, dtype=torch.bfloat16, device=dev)
    rows = max(1, (1 << 26) // max(1, out[0].numel()))
    for s in range(0, shape[0], rows):  # in pieces: the fp32 draw of a whole operand would not fit beside it
        e = min(shape[0], s + rows)
        out[s:e] = torch.randn((e - s,) + tuple(shape[1:]), generator=g, device=dev, dtype=torch.float32).to(torch.bfloat16)
    return out


@pytest.mark.parametrize("trans_b", [True, False])
@pytest.mark.parametrize("n,k", SHAPES)
def test_m_grouped_gemm_script(dev, n, k, trans_b):
    """tests/test_BF16/test_m_grouped_gemm_TMA.py:37-86: rtol = atol = 1e-2 on row-normalised outputs."""
    random.seed(1234)
    batch_sizes = torch.tensor(generate_random_list(GROUPS, GROUPS * 5120), dtype=torch.int64, device=dev)
    M = int(batch_sizes.sum())
    a = _randn((M, k), 1, dev)
    b = _randn((GROUPS, n, k) if trans_b else (GROUPS, k, n), 2, dev)
    out_ref = gmm(a, b, batch_sizes.cpu(), trans_b)
    out = m_grouped_gemm(a, b, batch_sizes, trans_b)
    torch.testing.assert_close(row_max_normalization(out), row_max_normalization(out_ref), rtol=1e-2, atol=1e-2)


@pytest.mark.parametrize("trans_b", [True, False])
@pytest.mark.parametrize("n,k", SHAPES)
def test_m_grouped_gemm_masked_script(dev, n, k, trans_b):
    """tests/test_BF16/test_m_grouped_gemm_masked_TMA.py:35-92: expected_m = 4096, every fifth group empty, counts
    clipped to expected_m; per group, valid rows only, rtol = 1e-3, atol = 5e-3 on row-normalised outputs.  (The
    script sets trans_b = False, which the reference's masked kernel does not take; here both layouts run.)"""
    random.seed(4321)
    expected_m = 4096
    batch_sizes = torch.full((GROUPS,), expected_m, dtype=torch.int32, device=dev)
    masked_m = torch.tensor(generate_random_list(GROUPS, GROUPS * 1024), dtype=torch.int64, device=dev).abs()
    masked_m[0:127:5] = 0
    masked_m = torch.where(masked_m > batch_sizes, batch_sizes.to(torch.int64), masked_m)
    M = GROUPS * expected_m
    a = _randn((M, k), 3, dev)
    b = _randn((GROUPS, n, k) if trans_b else (GROUPS, k, n), 4, dev)
    out = torch.full((M, n), float("nan"), dtype=torch.bfloat16, device=dev)
    m_grouped_gemm_masked(a, b, out, masked_m, expected_m, trans_b)
    starts = (batch_sizes.cumsum(0) - batch_sizes).tolist()
    counts = masked_m.tolist()
    for g in range(GROUPS):
        s, c = starts[g], counts[g]
        if c == 0:
            continue
        ref = a[s:s + c] @ (b[g].t() if trans_b else b[g])
        torch.testing.assert_close(row_max_normalization(out[s:s + c]), row_max_normalization(ref), rtol=1e-3, atol=5e-3)
        assert bool(torch.isnan(out[s + c:s + expected_m].float()).all()), f"group {g}: rows beyond masked_m were written"


@pytest.mark.parametrize("m,n", SHAPES)
def test_k_grouped_gemm_script(dev, m, n):
    """tests/test_BF16/test_k_grouped_gemm_TMA.py:42-87: C[g] = A_g^T B_g over the group's tokens; rtol = 1e-3,
    atol = 1e-2 on row-normalised outputs."""
    random.seed(5678)
    batch_sizes = torch.tensor(generate_random_list(GROUPS, GROUPS * 5120), dtype=torch.int64, device=dev).abs()
    K = int(batch_sizes.sum())
    a = _randn((K, m), 5, dev)
    b = _randn((K, n), 6, dev)
    out = k_grouped_gemm(a, b, batch_sizes)
    start = 0
    for g, size in enumerate(batch_sizes.tolist()):
        ref = a[start:start + size].t() @ b[start:start + size]
        torch.testing.assert_close(row_max_normalization(out[g]), row_max_normalization(ref), rtol=1e-3, atol=1e-2)
        start += size


def _per_row_cast(x, dtype):
    """The script's per_channel_cast_to_fp8 (tests/test_FP8/test_m_grouped_gemm_channel_expert.py:36-47): one scale per
    row over the whole of it."""
    fmax = torch.finfo(dtype).max
    amax = x.abs().float().amax(dim=1, keepdim=True).clamp(1e-4)
    return (x * (fmax / amax)).to(dtype), amax / fmax


def _per_expert_cast(w, dtype):
    """One scale per expert over its whole matrix (the script's per_expert_cast_to_fp8)."""
    fmax = torch.finfo(dtype).max
    amax = w.abs().float().amax(dim=(1, 2), keepdim=True).clamp(1e-4)
    return (w * (fmax / amax)).to(dtype), (amax / fmax).view(-1)


def test_fp8_m_grouped_channel_expert_script(dev):
    """tests/test_FP8/test_m_grouped_gemm_channel_expert.py:100-164: 32 experts with token counts
    [509, 3587, 125, 3971] x 8, N = 6144, K = 5120, activations e5m2, weights e4m3fn, bf16 out.  The script prints
    max|out - ref| / max(|out|, |ref|) against the unquantised product; that figure is printed here too, and the
    kernel itself is held to 2e-2 against the fp32 product of the dequantised operands."""
    bias = 3
    tokens = [512 - bias, 2 * 2048 - 512 + bias, 128 - bias, 2 * 2048 - 128 + bias] * 8
    M, N, K, G = sum(tokens), 6144, 5120, len(tokens)
    x = _randn((M, K), 7, dev)
    w = _randn((G, N, K), 8, dev)
    xq, xs = _per_row_cast(x, torch.float8_e5m2)
    wq, ws = _per_expert_cast(w, torch.float8_e4m3fn)
    sizes = torch.tensor(tokens, dtype=torch.int32, device=dev)
    out = gmm_fp8_act_per_channel_w_per_expert(xq, xs, wq, ws.view(-1, 1).repeat(1, N).reshape(-1), sizes, dtype_out=torch.bfloat16)
    worst_q = worst_u = 0.0
    start = 0
    for g, t in enumerate(tokens):
        o = out[start:start + t].float()
        ref_q = (xq[start:start + t].float() * xs[start:start + t]) @ (wq[g].float() * ws[g]).t()
        ref_u = x[start:start + t].float() @ w[g].float().t()
        worst_q = max(worst_q, float((o - ref_q).abs().max() / max(o.abs().max(), ref_q.abs().max())))
        worst_u = max(worst_u, float((o - ref_u).abs().max() / max(o.abs().max(), ref_u.abs().max())))
        start += t
    print(f"\nmax relative difference of the layer: {worst_u:.3e} against the unquantised product (what the script prints), "
          f"{worst_q:.3e} against the product of the dequantised operands")
    assert worst_q <= 2e-2, worst_q


def test_fp8_k_grouped_channel_expert_script(dev):
    """tests/test_FP8/test_k_grouped_gemm_channel_expert.py: weight gradient per expert over its tokens, per-channel
    scales on both operands for every expert (token counts padded to 128 as the script does); 2e-2 against the fp32
    product of the dequantised operands."""
    tokens = [512, 2 * 2048 - 512, 128, 2 * 2048 - 128] * 8
    G, Md, Nd, Kt = len(tokens), 2048, 1536, sum(tokens)
    x = _randn((Md, Kt), 9, dev)
    y = _randn((Nd, Kt), 10, dev)
    xq = torch.empty((Md, Kt), dtype=torch.float8_e4m3fn, device=dev)
    yq = torch.empty((Nd, Kt), dtype=torch.float8_e4m3fn, device=dev)
    xs = torch.empty((Md, G), dtype=torch.float32, device=dev)
    ys = torch.empty((Nd, G), dtype=torch.float32, device=dev)
    start = 0
    for g, t in enumerate(tokens):  # one scale per (row, expert) over the expert's tokens
        q, s = _per_row_cast(x[:, start:start + t], torch.float8_e4m3fn)
        xq[:, start:start + t], xs[:, g] = q, s.view(-1)
        q, s = _per_row_cast(y[:, start:start + t], torch.float8_e4m3fn)
        yq[:, start:start + t], ys[:, g] = q, s.view(-1)
        start += t
    out = k_grouped_fp8(xq, xs, yq, ys, torch.tensor(tokens, dtype=torch.int32, device=dev), Md, Nd, Kt, G)
    worst, start = 0.0, 0
    for g, t in enumerate(tokens):
        ref = (xq[:, start:start + t].float() * xs[:, g:g + 1]) @ (yq[:, start:start + t].float() * ys[:, g:g + 1]).t()
        o = out[g].float()
        worst = max(worst, float((o - ref).abs().max() / max(o.abs().max(), ref.abs().max())))
        start += t
    print(f"\nK-grouped FP8: worst per-expert rdiff {worst:.3e}")
    assert worst <= 2e-2, worst
