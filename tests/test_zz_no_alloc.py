"""The allocation-free sort entry point (tgg_moe_permute_map_static) against tgg_moe_permute_map, through the C ABI,
bit for bit, on two calls in a row (the second smaller, so stale contents of the shared scratch array would show),
plus its size limit."""
import ctypes

import pytest
import torch

from oracle import permute_ref
from triton_grouped_gemm_amd import _native

pytestmark = pytest.mark.gpu


def _indices(tokens, experts, topk, seed, drop=False):
    g = torch.Generator().manual_seed(seed)
    idx = torch.rand(tokens, experts, generator=g).topk(topk, dim=1).indices.to(torch.int32)
    if drop:
        idx[torch.rand(tokens, topk, generator=g) < 0.05] = -1
    return idx


def _both(dev, idx, experts, num_out_tokens=0, counts_dtype=torch.int32):
    tokens, topk = idx.shape
    d = idx.to(dev)
    stream = _native.stream_of(d)
    need = ctypes.c_int64(0)
    _native.call("tgg_moe_sort_workspace_bytes", tokens, topk, experts, ctypes.byref(need))
    ws = torch.empty(need.value, dtype=torch.uint8, device=dev)
    map_a = torch.full((tokens * topk,), -7, dtype=torch.int32, device=dev)
    cnt_a = torch.full((experts,), -7, dtype=counts_dtype, device=dev)
    _native.call("tgg_moe_permute_map", d.data_ptr(), tokens, topk, experts, num_out_tokens, map_a.data_ptr(),
                 cnt_a.data_ptr(), int(counts_dtype == torch.int64), ws.data_ptr(), need.value, stream)
    map_b = torch.full_like(map_a, -9)
    cnt_b = torch.full_like(cnt_a, -9)
    _native.call("tgg_moe_permute_map_static", d.data_ptr(), tokens, topk, experts, num_out_tokens, map_b.data_ptr(),
                 cnt_b.data_ptr(), int(counts_dtype == torch.int64), stream)
    torch.cuda.synchronize()
    assert torch.equal(map_a, map_b) and torch.equal(cnt_a, cnt_b)
    return map_b.cpu(), cnt_b.cpu()


def test_static_scratch_sort_equals_workspace_sort(dev):
    big = _indices(81920, 128, 8, 1)                       # 655360 assignments, 640 chunks
    m, c = _both(dev, big, 128)
    assert torch.equal(m, permute_ref.row_id_map(big)) and c.tolist() == permute_ref.tokens_per_expert(big, 128).tolist()
    small = _indices(777, 1024, 3, 2, drop=True)           # smaller, more experts, dropped assignments, int64 counts
    m, c = _both(dev, small, 1024, num_out_tokens=2000, counts_dtype=torch.int64)
    assert torch.equal(m, permute_ref.row_id_map(small, 2000))
    assert c.tolist() == permute_ref.tokens_per_expert(small, 1024).tolist()
    tiny = _indices(5, 3, 1, 3)
    m, c = _both(dev, tiny, 3)
    assert torch.equal(m, permute_ref.row_id_map(tiny))
    # the largest problem the scratch array holds
    full = _indices(1 << 17, 1024, 8, 4)
    _both(dev, full, 1024)


def test_static_scratch_sort_rejects_what_does_not_fit(dev):
    lib = _native.load()
    idx = torch.zeros(8, dtype=torch.int32, device=dev)
    out = torch.zeros(8, dtype=torch.int32, device=dev)
    rc = lib.tgg_moe_permute_map_static(idx.data_ptr(), (1 << 20) + 1, 1, 8, 0, out.data_ptr(), None, 0, None)
    assert rc == 1 and "exceeds" in _native.last_error()
    rc = lib.tgg_moe_permute_map_static(idx.data_ptr(), 8, 1, 1025, 0, out.data_ptr(), None, 0, None)
    assert rc == 1 and "num_experts" in _native.last_error()
