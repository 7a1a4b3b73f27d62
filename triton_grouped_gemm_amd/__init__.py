"""MI355X-native grouped GEMM: hand-written gfx950 HIP kernels behind the Python API of
DeepLink-org/Triton_Grouped_GEMM's hot path.

``triton_grouped_gemm_amd.gemm`` and ``triton_grouped_gemm_amd.quant`` have the module layout
of the reference's top-level ``gemm`` and ``quant`` packages; ``install_aliases()`` registers
them under those names so unmodified callers (``from gemm.BF16.m_grouped_gemm_TMA import
m_grouped_gemm``) resolve to this library.
"""
import importlib
import sys

__version__ = "0.1.0"

_ALIASED = [
    "gemm", "gemm.layout", "gemm.deep_gemm_ops", "gemm.BF16", "gemm.BF16.m_grouped_gemm",
    "gemm.BF16.m_grouped_gemm_TMA", "gemm.BF16.m_grouped_gemm_masked_TMA", "gemm.BF16.k_grouped_gemm",
    "gemm.BF16.k_grouped_gemm_TMA", "gemm.BF16.utils", "gemm.FP8", "gemm.FP8.m_grouped_gemm_channel_expert",
    "gemm.FP8.k_grouped_gemm_channel_expert", "quant", "quant.trans_per_block_quant_expand_128x",
    "quant.fp8_cast",
]


def install_aliases() -> None:
    """Make ``import gemm...`` / ``import quant...`` resolve to this package's modules."""
    for name in _ALIASED:
        sys.modules.setdefault(name, importlib.import_module(__name__ + "." + name))
