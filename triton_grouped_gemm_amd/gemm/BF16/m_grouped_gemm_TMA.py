"""Import path kept for callers of the reference's gemm/BF16/m_grouped_gemm_TMA.py.
There is a single native implementation; see ``m_grouped_gemm``."""
from .m_grouped_gemm import (BLOCK_M, _build_m_grouped_metadata, _m_grouped_gemm_launch,  # noqa: F401
                             m_grouped_gemm)
