"""The GPU baselines that bench.py times beside the library (one vendor GEMM per expert through torch, the
baseline the reference's own tables use: gemm/BF16/m_grouped_gemm_TMA.py:573-581 loops torch matmuls per group)
must do the same work as the library call they are compared with: same operands, same output up to the 16-bit
rounding of the result."""
import pytest
import torch

import bench
from tests._util import l2_rdiff

pytestmark = pytest.mark.gpu

SMALL = dict(groups=16, m_total=16 * 1024)


def _run(name, dev, **kw):
    fn, flops, nbytes, tag, cfg, _ = bench.build_workload(name, dev, **SMALL, **kw)
    out = fn()
    bench.build_workload.vendor_loop()
    torch.cuda.synchronize()
    return out, bench.build_workload.vendor_out, cfg


@pytest.mark.parametrize("name", ["bf16_m_grouped_gateup_nt", "bf16_m_grouped_gateup_nn", "bf16_m_grouped_down_nt"])
@pytest.mark.parametrize("uniform", [False, True])
def test_vendor_loop_matches_library_bf16(dev, name, uniform):
    out, ven, cfg = _run(name, dev, uniform=uniform)
    assert ("uniform" in cfg["group_sizes"]) == uniform
    # both are fp32-accumulated products rounded once to bf16; they may differ by accumulation order only
    assert l2_rdiff(out, ven) <= 1e-3
    assert float((out.float() - ven.float()).abs().max()) <= 2.0 ** -7 * float(ven.float().abs().max())


def test_vendor_loop_matches_library_k_grouped(dev):
    out, ven, _ = _run("bf16_k_grouped_wgrad", dev)
    assert l2_rdiff(out, ven) <= 1e-3


def test_vendor_loop_fp8_block_same_codes_unit_scales(dev):
    """The FP8 vendor loop multiplies the same e4m3 codes but knows no block scales: with every scale set to one the
    two must agree (each 128-deep slab is exact in fp32 here: the codes' products are small integers times 2^-k)."""
    fn, *_ = bench.build_workload("fp8_block_m_grouped", dev, **SMALL)
    ops = bench.build_workload.operands
    ops["aq"][1].fill_(1.0)
    ops["wq"][1].fill_(1.0)
    out = fn()
    try:
        bench.build_workload.vendor_loop()
    except Exception as exc:  # this torch / hipBLASLt build may not offer the call: bench.py then reports the error
        pytest.skip(f"torch._scaled_mm unavailable here: {exc}")
    torch.cuda.synchronize()
    ven = bench.build_workload.vendor_out
    assert l2_rdiff(out, ven) <= 2e-3
    assert float((out.float() - ven.float()).abs().max()) <= 2e-2 * float(ven.float().abs().max())


def test_vendor_loop_fp8_channel(dev):
    fn, *_ = bench.build_workload("fp8_channel_m_grouped", dev, **SMALL)
    out = fn()
    try:
        bench.build_workload.vendor_loop()
    except Exception as exc:
        pytest.skip(f"row-wise torch._scaled_mm unavailable here: {exc}")
    torch.cuda.synchronize()
    ven = bench.build_workload.vendor_out
    assert l2_rdiff(out, ven) <= 2e-3
    assert float((out.float() - ven.float()).abs().max()) <= 2e-2 * float(ven.float().abs().max())
