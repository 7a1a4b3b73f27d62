"""The entry points enqueue on the caller's stream and neither allocate nor synchronise, so a sequence of them can be
captured into a HIP graph and replayed.  Each replay is checked against the eager result, with eager work and
synchronisations between replays and changed inputs (the graph reads the same buffers)."""
import pytest
import torch

from triton_grouped_gemm_amd import _native
from triton_grouped_gemm_amd.gemm.BF16.k_grouped_gemm_TMA import k_grouped_gemm
from triton_grouped_gemm_amd.gemm.BF16.m_grouped_gemm_TMA import m_grouped_gemm

pytestmark = pytest.mark.gpu


def _randn(shape, seed, dev):
    g = torch.Generator().manual_seed(seed)
    return (torch.randn(shape, generator=g) * shape[-1] ** -0.5).to(torch.bfloat16).to(dev)


def test_forward_and_weight_gradient_in_one_graph(dev):
    sizes = torch.tensor([300, 0, 212, 512], dtype=torch.int32, device=dev)
    M, K, N = 1024, 256, 384
    a, b, g = _randn((M, K), 1, dev), _randn((4, N, K), 2, dev), _randn((M, N), 3, dev)
    out = torch.empty((M, N), dtype=torch.bfloat16, device=dev)
    dw = torch.empty((4, N, K), dtype=torch.bfloat16, device=dev)

    end = sizes.cumsum(0).to(torch.int32)
    start = (end - sizes).to(torch.int32)

    def step():
        # raw C-ABI calls into preallocated outputs: nothing inside allocates
        st = _native.stream_of(a)
        _native.call("tgg_m_grouped_gemm", a.data_ptr(), b.data_ptr(), out.data_ptr(), sizes.data_ptr(), 0, 4, M, N, K, 1,
                     _native.DTYPE_CODE[torch.bfloat16], -1, st)
        # weight gradient dW[g] = grad_g^T @ a_g : [N, K] per group
        _native.call("tgg_k_grouped_gemm", g.data_ptr(), a.data_ptr(), dw.data_ptr(), start.data_ptr(), end.data_ptr(), 4,
                     N, K, M, _native.DTYPE_CODE[torch.bfloat16], -1, st)

    step()  # first launches outside the capture (one-time function attributes)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        step()
    torch.cuda.current_stream().wait_stream(side)
    with torch.cuda.graph(graph):
        step()
    for it in range(4):
        a.copy_(_randn((M, K), 10 + it, dev))  # eager work between replays
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        ref = m_grouped_gemm(a, b, sizes, True)
        assert torch.equal(out, ref), f"replay {it}"
        assert torch.equal(dw, k_grouped_gemm(g, a, sizes)), f"replay {it} (weight gradient)"
