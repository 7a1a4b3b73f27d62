"""Writes tests/golden/small_cases.npz: seeded small inputs and the outputs the CPU oracle gives for them.

The reference holds no numeric fixtures for the GEMMs or the quantizer (its scripts compare against torch on the
fly), so these vectors come from this repository's oracle, whose functions are pinned in tests/test_oracle_pins.py.
They freeze the oracle's answers: a later change to the oracle or to torch's CPU arithmetic that moves a bit shows up
as a fixture mismatch, and the GPU kernels are checked against the same stored bits.

Run from the repository root:  python tests/golden/make_fixtures.py
"""
import os
import sys

import numpy as np
import torch

sys.path.insert(0, os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__)))))
from oracle import gemm_ref, quant_ref  # noqa: E402


def bits16(t: torch.Tensor) -> np.ndarray:
    return t.contiguous().view(torch.int16).numpy().view(np.uint16)


def main() -> None:
    g = torch.Generator().manual_seed(20260101)
    out = {}
    # M-grouped GEMM, NT, bf16: G=3, rows [40, 0, 56], K=64, N=128
    sizes = [40, 0, 56]
    a = (torch.randn(96, 64, generator=g) / 8).to(torch.bfloat16)
    b = (torch.randn(3, 128, 64, generator=g) / 8).to(torch.bfloat16)
    out["mg_sizes"] = np.array(sizes, dtype=np.int32)
    out["mg_a"], out["mg_b"] = bits16(a), bits16(b)
    out["mg_out_fp32"] = gemm_ref.gmm_fp32(a, b, sizes, True).numpy()
    # K-grouped GEMM: G=3, tokens [24, 0, 40], M_dim=64, N_dim=72
    ksizes = [24, 0, 40]
    ka = torch.randn(64, 64, generator=g).to(torch.bfloat16)
    kb = torch.randn(64, 72, generator=g).to(torch.bfloat16)
    out["kg_sizes"] = np.array(ksizes, dtype=np.int32)
    out["kg_a"], out["kg_b"] = bits16(ka), bits16(kb)
    out["kg_out_fp32"] = gemm_ref.gmm_dw(ka, kb, ksizes, fp32=True).numpy()
    # transposing 128x128 quantizer: rows [100, 0, 130], N=128, e4m3fn
    qsizes = [100, 0, 130]
    x = (torch.randn(230, 128, generator=g) * 2).to(torch.bfloat16)
    codes, scales, padded = quant_ref.trans_per_block_quant_expand_128x(x.float().numpy(), qsizes, "e4m3fn")
    out["tq_sizes"] = np.array(qsizes, dtype=np.int32)
    out["tq_x"] = bits16(x)
    out["tq_codes"], out["tq_scales"], out["tq_padded"] = codes, scales, np.asarray(padded, dtype=np.int64)
    # 1x128 activation recipe: 50 x 256, e4m3fn
    y = (torch.randn(50, 256, generator=g) * 3).to(torch.bfloat16)
    c2, s2 = quant_ref.per_token_cast_to_fp8(y.float().numpy(), "e4m3fn")
    out["pt_x"], out["pt_codes"], out["pt_scales"] = bits16(y), c2, s2
    path = os.path.join(os.path.dirname(os.path.abspath(__file__)), "small_cases.npz")
    np.savez_compressed(path, **out)
    print(path, os.path.getsize(path), "bytes")


if __name__ == "__main__":
    main()
