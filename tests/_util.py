"""Shared helpers for the GPU parity tests."""
import numpy as np
import torch

from oracle import gemm_ref


def bf16_ulp_distance(a: torch.Tensor, b: torch.Tensor) -> int:
    """Largest distance in units of bf16/fp16 code steps (monotone integer mapping of the codes)."""
    def key(t):
        i = t.contiguous().view(torch.int16).to(torch.int32)
        return torch.where(i < 0, -(i & 0x7FFF), i)
    return int((key(a) - key(b)).abs().max().item()) if a.numel() else 0


def l2_rdiff(out: torch.Tensor, ref: torch.Tensor) -> float:
    o, r = out.double(), ref.double()
    den = r.norm().item()
    return 0.0 if den == 0 else (o - r).norm().item() / den


def check_16bit_gemm(out: torch.Tensor, ref_same_dtype: torch.Tensor, ref_fp32: torch.Tensor, what: str = ""):
    """Gate for bf16/fp16-output GEMMs against the reference's torch oracle.

    Stated target: rdiff <= 1e-3 against the torch reference.  What is asserted:
      * every element within half an output ulp (+2%, + 1e-6 of the largest magnitude for
        fp32 accumulation-order noise on cancelling sums) of the fp32-accumulated oracle, i.e.
        the result is the correctly rounded product up to accumulation order;
      * against the oracle computed in the tensors' own dtype (what the reference's scripts
        compare with): L2-relative difference <= 1e-3 and cosine difference <= 1e-6;
      * max-norm rdiff against that same-dtype oracle <= 2^-7.  It is returned for reporting:
        a single rounding flip on a large element costs 2^-8..2^-7 (4e-3..8e-3) in that norm for
        any implementation (the same-dtype CPU oracle itself sits that far from the rounded fp32
        oracle), so 1e-3 in max-norm is only asserted where the case is small enough to be flip-free.
    """
    out_c, ref_c = out.cpu(), ref_same_dtype.cpu()
    assert out_c.shape == ref_c.shape, what
    assert torch.isfinite(out_c.float()).all(), what + ": non-finite output"
    eps = 2.0 ** -8 if out.dtype == torch.bfloat16 else 2.0 ** -11
    err = (out_c.float() - ref_fp32).abs()
    bound = ref_fp32.abs() * eps * 1.02 + 1e-6 * ref_fp32.abs().max()
    assert bool((err <= bound).all()), f"{what}: element off by more than half an ulp of the exact result"
    l2 = l2_rdiff(out_c, ref_c)
    assert l2 <= 1e-3, f"{what}: L2 rdiff {l2}"
    assert gemm_ref.cos_diff(out_c, ref_c) <= 1e-6, what
    rd = gemm_ref.rdiff(out_c, ref_c)
    assert rd <= 2.0 ** -7, f"{what}: max-norm rdiff {rd}"
    return rd


def to_np_f32(t: torch.Tensor) -> np.ndarray:
    return t.detach().cpu().float().numpy()


def codes_np(t: torch.Tensor) -> np.ndarray:
    return t.detach().cpu().contiguous().view(torch.uint8).numpy()
