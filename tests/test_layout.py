"""CPU: the product's gemm.layout helpers against the reference's known answers
(tests/test_layout_backend.py:22-52), the plain-Python oracle, and the dtype rules."""
import pytest
import torch
from hypothesis import given, settings, strategies as st

from oracle import layout_ref
from triton_grouped_gemm_amd.gemm import layout as L


def test_round_up_to_alignment():
    sizes = torch.tensor([0, 1, 127, 128, 129], dtype=torch.int32)
    assert L.round_up_to_alignment(sizes, 128).tolist() == [0, 128, 128, 128, 256]
    with pytest.raises(ValueError, match="alignment must be positive"):
        L.round_up_to_alignment(sizes, 0)


def test_make_group_starts_logical_and_padded():
    sizes = torch.tensor([3, 5, 0, 7], dtype=torch.int32)
    assert L.make_group_starts(sizes, padded=False, block_m=4).tolist() == [0, 3, 8, 8]
    assert L.make_group_starts(sizes, padded=True, block_m=4).tolist() == [0, 4, 12, 12]


def test_make_grouped_layout_summary_and_dtypes():
    lay = L.make_grouped_layout([3, 5, 0, 7], block_m=4)
    assert lay.sizes.tolist() == [3, 5, 0, 7]
    assert lay.padded_sizes.tolist() == [4, 8, 0, 8]
    assert lay.starts.tolist() == [0, 4, 12, 12]
    assert int(lay.total_m.item()) == 15 and int(lay.total_padded_m.item()) == 20
    # cumsum of int32 is int64 in torch; the reference's starts therefore are int64
    assert lay.sizes.dtype == torch.int32 and lay.padded_sizes.dtype == torch.int32
    assert lay.starts.dtype == torch.int64 and lay.total_m.dtype == torch.int64
    assert L.make_group_starts([1, 2]).dtype == torch.int64


def test_deep_gemm_layouts():
    assert L.make_deep_gemm_grouped_layout([3, 5], block_m=4).tolist() == [0, 0, 0, -1, 1, 1, 1, 1, 1, -1, -1, -1]
    assert L.make_deep_gemm_psum_layout([3, 5], block_m=4).tolist() == [3, 9]
    assert L.make_deep_gemm_grouped_layout([3, 5], block_m=4).dtype == torch.int32
    assert L.make_deep_gemm_psum_layout([3, 5], block_m=4).dtype == torch.int32
    assert L.make_deep_gemm_grouped_layout([0, 0]).numel() == 0


def test_validate_total_m_and_size_checks():
    L.validate_total_m([2, 3, 4], 9)
    with pytest.raises(ValueError, match=r"sum\(size_per_group\)"):
        L.validate_total_m([2, 3, 4], 10)
    with pytest.raises(ValueError, match="1D"):
        L.as_group_sizes(torch.zeros(2, 2, dtype=torch.int32))
    with pytest.raises(ValueError, match="at least one group"):
        L.as_group_sizes([])
    with pytest.raises(ValueError, match="negative"):
        L.as_group_sizes([1, -1])
    assert L.as_group_sizes(torch.tensor([1, 2], dtype=torch.int64)).dtype == torch.int32


@settings(max_examples=60, deadline=None)
@given(st.lists(st.integers(0, 700), min_size=1, max_size=40), st.sampled_from([1, 4, 64, 128]))
def test_layout_matches_plain_python_oracle(sizes, block_m):
    assert L.make_group_starts(sizes, padded=False, block_m=block_m).tolist() == layout_ref.group_starts(sizes, False, block_m)
    assert L.make_group_starts(sizes, padded=True, block_m=block_m).tolist() == layout_ref.group_starts(sizes, True, block_m)
    ref = layout_ref.grouped_layout(sizes, block_m)
    lay = L.make_grouped_layout(sizes, block_m)
    assert lay.starts.tolist() == ref["starts"] and lay.padded_sizes.tolist() == ref["padded_sizes"]
    assert L.make_deep_gemm_grouped_layout(sizes, block_m=block_m).tolist() == layout_ref.deep_gemm_grouped_layout(sizes, block_m)
    assert L.make_deep_gemm_psum_layout(sizes, block_m=block_m).tolist() == layout_ref.deep_gemm_psum_layout(sizes, block_m)


def test_metadata_builder_matches_oracle():
    from triton_grouped_gemm_amd.gemm.BF16.m_grouped_gemm import _build_m_grouped_metadata
    sizes = [3, 0, 130, 128, 1, 257]
    ps, pe, gs, ge, idx, mpad = _build_m_grouped_metadata(torch.tensor(sizes, dtype=torch.int32))
    rps, rpe, rgs, rge, ridx, rmpad = layout_ref.m_grouped_metadata(sizes)
    assert ps.tolist() == rps and pe.tolist() == rpe and gs.tolist() == rgs and ge.tolist() == rge
    assert idx[: len(ridx)].tolist() == ridx and int(mpad) == rmpad
    assert idx.numel() == sum(sizes) // 128 + len(sizes) and idx.dtype == torch.int32
    assert ps.dtype == torch.int32 and gs.dtype == torch.int64


def test_sizes_from_explicit_layouts():
    # both explicit layout forms give back the valid rows they were built from (reference gemm/layout.py:73-119)
    from triton_grouped_gemm_amd.gemm.deep_gemm_ops import sizes_from_layout
    for sizes, block_m in ([[3, 5, 0, 7], 4], [[0, 0, 9], 8], [[128, 1, 127, 256, 0], 128], [[5], 128]):
        rows = L.make_deep_gemm_grouped_layout(sizes, block_m=block_m)
        ends = L.make_deep_gemm_psum_layout(sizes, block_m=block_m)
        assert sizes_from_layout(rows, len(sizes), block_m, False).tolist() == sizes
        assert sizes_from_layout(ends, len(sizes), block_m, True).tolist() == sizes
        assert sizes_from_layout(rows.to(torch.int64), len(sizes), block_m, False).dtype == torch.int32


def test_placement_from_per_row_layout_in_any_expert_order():
    # a per-row layout whose experts are not in ascending order: rows per expert and their first row, by hand
    from triton_grouped_gemm_amd.gemm.deep_gemm_ops import placement_from_layout
    lay = torch.tensor([2, 2, 2, -1, 0, 0, -1, -1, 3, -1, -1, -1], dtype=torch.int32)  # block_m = 4; expert 1 absent
    rows, first, expert = placement_from_layout(lay, 4)
    assert rows.tolist() == [2, 0, 3, 1] and first.tolist() == [4, 0, 0, 8] and expert is None
    assert rows.dtype == torch.int32 and first.dtype == torch.int32
    # ascending layouts give the padded starts the builders use
    sizes = [128, 1, 127, 256, 0]
    rows, first, expert = placement_from_layout(L.make_deep_gemm_grouped_layout(sizes), len(sizes))
    assert rows.tolist() == sizes and first.tolist() == [0, 128, 256, 384, 0] and expert is None


def test_placement_from_per_row_layout_with_an_expert_in_several_regions():
    # expert 2 owns rows 0..3 and 8..9, expert 0 rows 4..5 and row 11: one entry per region, in row order, by hand
    from triton_grouped_gemm_amd.gemm.deep_gemm_ops import placement_from_layout
    lay = torch.tensor([2, 2, 2, 2, 0, 0, -1, -1, 2, 2, -1, 0], dtype=torch.int64)
    rows, first, expert = placement_from_layout(lay, 3)
    assert rows.tolist() == [4, 2, 2, 1] and first.tolist() == [0, 4, 8, 11] and expert.tolist() == [2, 0, 2, 0]
    assert rows.dtype == torch.int32 and first.dtype == torch.int32 and expert.dtype == torch.int64
    # two regions of one expert that touch are one region; neighbours of different experts are two
    rows, first, expert = placement_from_layout(torch.tensor([1, 1, 1, 1, 0, 0, 0, -1]), 2)
    assert rows.tolist() == [3, 4] and first.tolist() == [4, 0] and expert is None
    with pytest.raises(ValueError, match=r"outside \[-1, 2\)"):
        placement_from_layout(torch.tensor([0, 0, 2, -1]), 2)
    with pytest.raises(ValueError, match=r"outside \[-1, 2\)"):
        placement_from_layout(torch.tensor([0, 0, -3, -1]), 2)


def test_layout_ids_that_name_no_expert_count_as_padding_where_nothing_can_be_checked():
    """sizes_from_layout never reads back (it is what a captured call uses): ids below -1 or beyond the experts must
    not index outside its table; their rows belong to no group."""
    from triton_grouped_gemm_amd.gemm.deep_gemm_ops import sizes_from_layout
    lay = torch.tensor([0, 0, 7, -1, 1, -5, 1, 1], dtype=torch.int32)
    assert sizes_from_layout(lay, 2, 4, False).tolist() == [2, 3]


def test_reference_named_helpers():
    """gemm/BF16/utils.py of the reference: the per-group torch loop, the group-size draw and the two checks."""
    import random

    import torch

    from triton_grouped_gemm_amd.gemm.BF16.utils import allclose, generate_random_list, gmm, row_max_normalization
    random.seed(3)
    for length, total in [(8, 1000), (1, 17), (128, 655360), (5, 4)]:
        sizes = generate_random_list(length, total)
        assert len(sizes) == length and sum(sizes) == total and min(sizes[:-1] + [0]) >= 0
    sizes = [3, 0, 5]
    a, b = torch.randn(8, 6), torch.randn(3, 6, 4)
    out = gmm(a, b, torch.tensor(sizes))
    assert out.shape == (8, 4)
    assert torch.equal(out[:3], a[:3] @ b[0]) and torch.equal(out[3:], a[3:] @ b[2])
    assert torch.equal(gmm(a, b.transpose(1, 2).contiguous(), torch.tensor(sizes), trans_b=True), out)
    assert allclose(out, out) and not allclose(out, out + 1.0)
    assert float(row_max_normalization(a).abs().max(dim=-1).values.max()) <= 1.0
