"""CPU: the C-ABI library loads and exports what include/tgg_amd.h declares; host-side
validation raises the reference's errors before anything touches a GPU."""
import ctypes
import re
from pathlib import Path

import pytest
import torch

import triton_grouped_gemm_amd as tgg
from triton_grouped_gemm_amd import _native

ROOT = Path(__file__).resolve().parents[1]


def _declared_symbols():
    text = (ROOT / "include" / "tgg_amd.h").read_text()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(tgg_[a-z0-9_]+)\s*\(", text)))


def test_library_exports_every_declared_symbol():
    lib = _native.load()
    names = _declared_symbols()
    assert len(names) >= 14
    for name in names:
        assert hasattr(lib, name), name
    assert set(_native.SIGNATURES) | {"tgg_last_error"} == set(names)
    assert lib.tgg_version() >= 100


def test_c_abi_rejects_bad_arguments_without_a_gpu():
    lib = _native.load()
    rc = lib.tgg_m_grouped_gemm(None, None, None, None, 0, 4, 128, 128, 128, 1, 0, -1, None)
    assert rc == 1 and "null" in _native.last_error()
    buf = ctypes.create_string_buffer(4096)
    p = ctypes.addressof(buf)
    p += (-p) % 16
    assert lib.tgg_m_grouped_gemm(p, p, p, p, 0, 0, 128, 128, 128, 1, 0, -1, None) == 1
    assert "G=0" in _native.last_error()
    assert lib.tgg_m_grouped_gemm(p, p, p, p, 0, 4, 128, 128, 100, 1, 0, -1, None) == 1
    assert "multiples of 8" in _native.last_error()
    assert lib.tgg_m_grouped_gemm(p, p, p, p, 0, 4, 128, 128, 128, 1, 7, -1, None) == 1
    assert "not supported" in _native.last_error()
    assert lib.tgg_m_grouped_gemm(p + 4, p, p, p, 0, 4, 128, 128, 128, 1, 0, -1, None) == 1
    assert "aligned" in _native.last_error()
    assert lib.tgg_trans_per_block_quant_expand_128x(p, p, p, p, 0, 2, 256, 100, 512, 2, None) == 1
    assert lib.tgg_per_token_cast_to_fp8(p, p, p, 4, 100, 2, 0, None) == 1
    assert lib.tgg_set_option(b"nope", 1) == 1
    assert lib.tgg_set_option(b"force_generic", 0) == 0


def test_group_count_limits_per_entry_point():
    """More than 512 groups are taken by the plain 16-bit M-grouped and K-grouped entry points only (up to 1024: the
    shape-agnostic kernel serves them and is exercised there on the GPU); every other GEMM entry point rejects
    them before anything is launched."""
    lib = _native.load()
    buf = ctypes.create_string_buffer(4096)
    p = ctypes.addressof(buf)
    p += (-p) % 16
    calls = [
        lambda g: lib.tgg_m_grouped_gemm_padded(p, p, p, p, 0, g, 1024, 128, 128, 128, 0, -1, None),
        lambda g: lib.tgg_m_grouped_gemm_placed(p, p, p, p, 0, p, g, 1024, 128, 128, 0, -1, None),
        lambda g: lib.tgg_m_grouped_gemm_masked(p, p, p, p, 0, g, 128, 1024, 128, 128, 1, 0, -1, None),
        lambda g: lib.tgg_m_grouped_gemm_fp8_out(p, p, p, p, p, 0, g, 1024, 128, 128, 1, 0, 2, 0, -1, None),
        lambda g: lib.tgg_m_grouped_gemm_fp8_channel(p, p, p, p, p, p, 0, g, 1024, 128, 128, 2, 2, 0, -1, None),
        lambda g: lib.tgg_k_grouped_gemm_fp8_channel(p, p, p, p, p, p, g, 128, 128, 1024, 2, 2, -1, None),
        lambda g: lib.tgg_m_grouped_gemm_fp8_block(p, p, p, p, p, p, 0, g, 1024, 128, 128, 128, 1, -1, None),
        lambda g: lib.tgg_m_grouped_gemm_fp8_block_placed(p, p, p, p, p, p, 0, p, g, 1024, 128, 128, 1, -1, None),
    ]
    for call in calls:
        assert call(_native.MAX_GROUPS_OTHER + 1) == 1
        assert f"G=513 outside [1, {_native.MAX_GROUPS_OTHER}]" in _native.last_error()
    assert lib.tgg_m_grouped_gemm(p, p, p, p, 0, _native.MAX_GROUPS + 1, 128, 128, 128, 1, 0, -1, None) == 1
    assert "G=1025 outside [1, 1024]" in _native.last_error()
    assert lib.tgg_k_grouped_gemm(p, p, p, p, p, _native.MAX_GROUPS + 1, 128, 128, 1024, 0, -1, None) == 1
    assert "G=1025 outside [1, 1024]" in _native.last_error()


def test_reference_import_paths_resolve():
    tgg.install_aliases()
    from gemm.BF16.m_grouped_gemm_TMA import m_grouped_gemm, _build_m_grouped_metadata, _m_grouped_gemm_launch  # noqa
    from gemm.BF16.m_grouped_gemm import m_grouped_gemm as mg2
    from gemm.BF16.m_grouped_gemm_masked_TMA import m_grouped_gemm_masked  # noqa
    from gemm.BF16.k_grouped_gemm_TMA import k_grouped_gemm  # noqa
    from gemm.BF16.k_grouped_gemm import k_grouped_gemm as kg2  # noqa
    from gemm.FP8.m_grouped_gemm_channel_expert import gmm_fp8_act_per_channel_w_per_expert  # noqa
    from gemm.FP8.k_grouped_gemm_channel_expert import matmul  # noqa
    from gemm.deep_gemm_ops import m_grouped_bf16_nt_contiguous, m_grouped_fp8_nt_contiguous  # noqa
    from gemm.layout import make_grouped_layout  # noqa
    from quant.trans_per_block_quant_expand_128x import trans_per_block_quant_expand_128x, trans_quant  # noqa
    assert m_grouped_gemm is mg2
    assert torch.ops.moe.m_grouped_gemm is not None


def test_fake_kernel_shapes():
    from torch._subclasses.fake_tensor import FakeTensorMode
    with FakeTensorMode():
        a = torch.empty(256, 64, dtype=torch.bfloat16)
        bt = torch.empty(2, 96, 64, dtype=torch.bfloat16)
        bn = torch.empty(2, 64, 96, dtype=torch.bfloat16)
        s = torch.empty(2, dtype=torch.int32)
        assert torch.ops.moe.m_grouped_gemm(a, bt, s, True).shape == (256, 96)
        out = torch.ops.moe.m_grouped_gemm(a, bn, s, False)
        assert out.shape == (256, 96) and out.dtype == torch.bfloat16


def test_m_grouped_validation_messages():
    from triton_grouped_gemm_amd.gemm.BF16.m_grouped_gemm import _m_grouped_gemm_launch
    a = torch.zeros(128, 64, dtype=torch.bfloat16)
    b = torch.zeros(2, 96, 64, dtype=torch.bfloat16)
    c = torch.zeros(128, 96, dtype=torch.bfloat16)
    s = torch.tensor([64, 64], dtype=torch.int32)
    with pytest.raises(AssertionError, match="K of A should be equal to K of B"):
        _m_grouped_gemm_launch(a, torch.zeros(2, 96, 32, dtype=torch.bfloat16), c, s, True)
    with pytest.raises(AssertionError, match=r"C should have shape \[M, N\]"):
        _m_grouped_gemm_launch(a, b, torch.zeros(128, 64, dtype=torch.bfloat16), s, True)
    with pytest.raises(AssertionError, match="K-major"):
        _m_grouped_gemm_launch(torch.zeros(64, 128, dtype=torch.bfloat16).t(), b, c, s, True)
    with pytest.raises(AssertionError, match="not supported"):
        _m_grouped_gemm_launch(a.float(), b, c, s, True)
    with pytest.raises(AssertionError, match="16-byte alignment"):
        _m_grouped_gemm_launch(torch.zeros(128, 60, dtype=torch.bfloat16), torch.zeros(2, 96, 60, dtype=torch.bfloat16), c, s, True)
    with pytest.raises(AssertionError, match="no CPU path"):
        _m_grouped_gemm_launch(a, b, c, s, True)


def test_masked_and_k_grouped_validation_messages():
    from triton_grouped_gemm_amd.gemm.BF16.m_grouped_gemm_masked_TMA import m_grouped_gemm_masked
    from triton_grouped_gemm_amd.gemm.BF16.k_grouped_gemm import k_grouped_gemm
    lhs = torch.zeros(2 * 128, 64, dtype=torch.bfloat16)
    rhs = torch.zeros(2, 96, 64, dtype=torch.bfloat16)
    out = torch.zeros(2 * 128, 96, dtype=torch.bfloat16)
    mm = torch.tensor([3, 4], dtype=torch.int32)
    with pytest.raises(AssertionError):
        m_grouped_gemm_masked(lhs.view(2, 128, 64), rhs, out, mm, 128)
    with pytest.raises(AssertionError, match="multiple of BLOCK_M"):
        m_grouped_gemm_masked(lhs[:200], rhs, out[:200], mm, 100)
    with pytest.raises(AssertionError, match="K of lhs"):
        m_grouped_gemm_masked(lhs, torch.zeros(2, 96, 32, dtype=torch.bfloat16), out, mm, 128)
    a = torch.zeros(256, 64, dtype=torch.bfloat16)
    b = torch.zeros(256, 96, dtype=torch.bfloat16)
    with pytest.raises(AssertionError, match="trans_b=True path has been removed"):
        k_grouped_gemm(a, b, mm, trans_b=True)
    with pytest.raises(AssertionError, match="must be CUDA tensors"):
        k_grouped_gemm(a, b, mm)


def test_contiguous_entry_validation():
    from triton_grouped_gemm_amd.gemm.deep_gemm_ops import m_grouped_bf16_nt_contiguous, m_grouped_fp8_nt_contiguous
    a = torch.zeros(256, 128, dtype=torch.bfloat16)
    b = torch.zeros(2, 64, 128, dtype=torch.bfloat16)
    s = torch.tensor([100, 128], dtype=torch.int32)
    with pytest.raises(ValueError, match="K mismatch"):
        m_grouped_bf16_nt_contiguous(a, torch.zeros(2, 64, 64, dtype=torch.bfloat16), s)
    with pytest.raises(ValueError, match="A must include padded expert rows: expected M=256, got M=128"):
        m_grouped_bf16_nt_contiguous(a[:128], b, s)
    with pytest.raises(ValueError, match="expected a shape"):
        m_grouped_bf16_nt_contiguous(a.view(2, 128, 128), b, s)
    aq = torch.zeros(256, 128, dtype=torch.float8_e4m3fn)
    bq = torch.zeros(2, 64, 128, dtype=torch.float8_e4m3fn)
    with pytest.raises(ValueError, match=r"a\[1\] must have shape"):
        m_grouped_fp8_nt_contiguous((aq, torch.zeros(256, 2)), (bq, torch.zeros(2, 1, 1)), s)
    with pytest.raises(ValueError, match="recipe"):
        m_grouped_fp8_nt_contiguous((aq, torch.zeros(256, 1)), (bq, torch.zeros(2, 1, 1)), s, recipe_a=(1, 64))


def test_missing_library_fails_loudly(monkeypatch, tmp_path):
    monkeypatch.setattr(_native, "_lib", None)
    monkeypatch.setattr(_native, "LIB_PATH", tmp_path / "libtgg_amd.so")
    with pytest.raises(RuntimeError, match="no non-HIP fallback"):
        _native.load()
