"""Import path kept for callers of the reference's gemm/BF16/k_grouped_gemm_TMA.py."""
from .k_grouped_gemm import _check_k_grouped_gemm_inputs, _dtype_code, k_grouped_gemm  # noqa: F401
