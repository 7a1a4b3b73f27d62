"""Committed fixtures (tests/golden): the reference's own layout known answers, and small seeded cases whose
expected outputs were written by tests/golden/make_fixtures.py from the CPU oracle.  The CPU tests check that the
oracle still reproduces the stored bits; the GPU tests check the kernels against the same stored data."""
import json
import os

import numpy as np
import pytest
import torch

from oracle import gemm_ref, quant_ref
from tests._util import check_16bit_gemm
from triton_grouped_gemm_amd.gemm import layout as L

HERE = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")


def _load():
    return np.load(os.path.join(HERE, "small_cases.npz"), allow_pickle=False)


def _bf16(bits: np.ndarray) -> torch.Tensor:
    return torch.from_numpy(bits.view(np.int16).copy()).view(torch.bfloat16)


def test_layout_known_answers_of_the_reference():
    k = json.load(open(os.path.join(HERE, "layout_known_answers.json")))
    c = k["round_up_to_alignment"]
    assert L.round_up_to_alignment(torch.tensor(c["sizes"], dtype=torch.int32), c["alignment"]).tolist() == c["expected"]
    c = k["make_group_starts"]
    s = torch.tensor(c["sizes"], dtype=torch.int32)
    assert L.make_group_starts(s, padded=False, block_m=c["block_m"]).tolist() == c["logical"]
    assert L.make_group_starts(s, padded=True, block_m=c["block_m"]).tolist() == c["padded"]
    c = k["make_grouped_layout"]
    lay = L.make_grouped_layout(c["sizes"], block_m=c["block_m"])
    assert lay.padded_sizes.tolist() == c["padded_sizes"] and lay.starts.tolist() == c["starts"]
    assert int(lay.total_m) == c["total_m"] and int(lay.total_padded_m) == c["total_padded_m"]
    c = k["make_deep_gemm_grouped_layout"]
    assert L.make_deep_gemm_grouped_layout(c["sizes"], block_m=c["block_m"]).tolist() == c["expected"]
    c = k["make_deep_gemm_psum_layout"]
    assert L.make_deep_gemm_psum_layout(c["sizes"], block_m=c["block_m"]).tolist() == c["expected"]
    c = k["validate_total_m"]
    L.validate_total_m(c["sizes"], c["ok"])
    with pytest.raises(ValueError):
        L.validate_total_m(c["sizes"], c["bad"])


def test_oracle_reproduces_the_stored_vectors():
    d = _load()
    out = gemm_ref.gmm_fp32(_bf16(d["mg_a"]), _bf16(d["mg_b"]), d["mg_sizes"].tolist(), True).numpy()
    assert np.array_equal(out, d["mg_out_fp32"])
    kout = gemm_ref.gmm_dw(_bf16(d["kg_a"]), _bf16(d["kg_b"]), d["kg_sizes"].tolist(), fp32=True).numpy()
    assert np.array_equal(kout, d["kg_out_fp32"])
    codes, scales, padded = quant_ref.trans_per_block_quant_expand_128x(_bf16(d["tq_x"]).float().numpy(),
                                                                       d["tq_sizes"].tolist(), "e4m3fn")
    assert np.array_equal(codes, d["tq_codes"]) and np.array_equal(scales.view(np.uint32), d["tq_scales"].view(np.uint32))
    assert list(padded) == d["tq_padded"].tolist()
    c2, s2 = quant_ref.per_token_cast_to_fp8(_bf16(d["pt_x"]).float().numpy(), "e4m3fn")
    assert np.array_equal(c2, d["pt_codes"]) and np.array_equal(s2.view(np.uint32), d["pt_scales"].view(np.uint32))


@pytest.mark.gpu
def test_kernels_against_the_stored_vectors(dev):
    from triton_grouped_gemm_amd.gemm.BF16.k_grouped_gemm_TMA import k_grouped_gemm
    from triton_grouped_gemm_amd.gemm.BF16.m_grouped_gemm_TMA import m_grouped_gemm
    from triton_grouped_gemm_amd.quant.fp8_cast import per_token_cast_to_fp8
    from triton_grouped_gemm_amd.quant.trans_per_block_quant_expand_128x import trans_per_block_quant_expand_128x
    d = _load()
    ref = torch.from_numpy(d["mg_out_fp32"])
    out = m_grouped_gemm(_bf16(d["mg_a"]).to(dev), _bf16(d["mg_b"]).to(dev), torch.from_numpy(d["mg_sizes"]).to(dev), True)
    check_16bit_gemm(out, ref.to(torch.bfloat16), ref, "golden m-grouped")
    kref = torch.from_numpy(d["kg_out_fp32"])
    kout = k_grouped_gemm(_bf16(d["kg_a"]).to(dev), _bf16(d["kg_b"]).to(dev), torch.from_numpy(d["kg_sizes"]).to(dev))
    assert torch.count_nonzero(kout[1]) == 0
    for g in (0, 2):
        check_16bit_gemm(kout[g], kref[g].to(torch.bfloat16), kref[g], f"golden k-grouped {g}")
    codes, scales, padded = trans_per_block_quant_expand_128x(_bf16(d["tq_x"]).to(dev), torch.from_numpy(d["tq_sizes"]).to(dev))
    assert np.array_equal(codes.view(torch.uint8).cpu().numpy(), d["tq_codes"])
    assert np.array_equal(scales.cpu().numpy().view(np.uint32), d["tq_scales"].view(np.uint32))
    assert padded.tolist() == d["tq_padded"].tolist()
    c2, s2 = per_token_cast_to_fp8(_bf16(d["pt_x"]).to(dev))
    assert np.array_equal(c2.view(torch.uint8).cpu().numpy(), d["pt_codes"])
    assert np.array_equal(s2.cpu().numpy().view(np.uint32), d["pt_scales"].view(np.uint32))
