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


def test_group_sizes_may_change_between_replays(dev):
    """Group sizes are read on the device, so one captured graph serves any routing: between replays the sizes
    buffer is rewritten so that the kernels' device-side choices change (few narrow tiles; many half-empty tiles;
    large groups), for the 16-bit and the block-scaled FP8 M-grouped GEMM."""
    from triton_grouped_gemm_amd.quant.fp8_cast import per_block_cast_to_fp8, per_token_cast_to_fp8
    G, M, N, K = 64, 64 * 256, 1024, 512
    a, b = _randn((M, K), 21, dev), _randn((G, N, K), 22, dev)
    aq, sa = per_token_cast_to_fp8(a, scales_mn_major=True)
    wq, sb = per_block_cast_to_fp8(b)
    sizes = torch.zeros(G, dtype=torch.int32, device=dev)
    out16 = torch.empty((M, N), dtype=torch.bfloat16, device=dev)
    out8 = torch.empty((M, N), dtype=torch.bfloat16, device=dev)

    def step():
        st = _native.stream_of(a)
        _native.call("tgg_m_grouped_gemm", a.data_ptr(), b.data_ptr(), out16.data_ptr(), sizes.data_ptr(), 0, G, M, N, K, 1,
                     _native.DTYPE_CODE[torch.bfloat16], -1, st)
        _native.call("tgg_m_grouped_gemm_fp8_block", aq.data_ptr(), sa.data_ptr(), wq.data_ptr(), sb.data_ptr(),
                     out8.data_ptr(), sizes.data_ptr(), 0, G, M, N, K, 128, 1, -1, st)

    routings = [
        [128] * 3 + [0] * (G - 3),                 # 3 row tiles x 8 narrow column tiles: the narrow configuration
        [128] * G,                                  # every tile half empty: waves sit tiles out
        [256] * G,                                  # full tiles
        [1024, 0, 384] + [128] * 8 + [0] * (G - 11),
    ]
    sizes.copy_(torch.tensor(routings[0], dtype=torch.int32))
    step()
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        step()
    for it, routing in enumerate(routings * 2):
        sizes.copy_(torch.tensor(routing, dtype=torch.int32))
        out16.fill_(7.0)
        out8.fill_(7.0)
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        rows = sum(routing)
        ref16 = m_grouped_gemm(a, b, sizes, True)
        ref8 = torch.full_like(out8, 7.0)  # the same call, eagerly (the wrapper insists on M = sum of the padded sizes)
        _native.call("tgg_m_grouped_gemm_fp8_block", aq.data_ptr(), sa.data_ptr(), wq.data_ptr(), sb.data_ptr(),
                     ref8.data_ptr(), sizes.data_ptr(), 0, G, M, N, K, 128, 1, -1, _native.stream_of(a))
        assert torch.equal(out16[:rows], ref16[:rows]), f"replay {it}"
        placed = 0
        for n in routing:  # block-scaled layout: every group starts at a multiple of 128 rows
            assert torch.equal(out8[placed:placed + n], ref8[placed:placed + n]), f"replay {it} (fp8)"
            placed += (n + 127) // 128 * 128
        n0 = routing[0]
        ad = aq[:n0].float() * sa[:n0].repeat_interleave(128, dim=1)
        wd = wq[0].float() * sb[0].repeat_interleave(128, dim=0).repeat_interleave(128, dim=1)
        exact = ad @ wd.t()
        assert float((out8[:n0].float() - exact).abs().max()) <= 2.0 ** -7 * float(exact.abs().max()), f"replay {it} (fp8 values)"
        assert bool((out16[rows:] == 7.0).all()) and bool((out8[placed:] == 7.0).all()), f"replay {it}: rows past the groups"


def test_masked_counts_may_change_which_kernel_runs_between_replays(dev):
    """A masked launch of this size enqueues the four-wave kernel and the eight-wave kernel, and the counts decide on
    the device which of them does the work.  One captured graph holds both launches; between replays masked_m is
    rewritten so that the choice flips (counts near m_max: 256-row tiles pay; a few dozen rows per group: they do not)."""
    G, m_max, N, K = 72, 512, 1032, 256
    lhs = torch.randint(-1, 2, (G * m_max, K), generator=torch.Generator().manual_seed(41)).to(torch.bfloat16).to(dev)
    rhs = torch.randint(-1, 2, (G, N, K), generator=torch.Generator().manual_seed(42)).to(torch.bfloat16).to(dev)
    ref = torch.bmm(lhs.float().view(G, m_max, K), rhs.float().transpose(1, 2)).to(torch.bfloat16)  # exact: integers
    masked = torch.zeros(G, dtype=torch.int32, device=dev)
    out = torch.empty((G * m_max, N), dtype=torch.bfloat16, device=dev)

    def step():
        _native.call("tgg_m_grouped_gemm_masked", lhs.data_ptr(), rhs.data_ptr(), out.data_ptr(), masked.data_ptr(), 0, G,
                     m_max, G * m_max, N, K, 1, _native.DTYPE_CODE[torch.bfloat16], -1, _native.stream_of(lhs))

    counts = [
        [512 - (37 * g) % 200 for g in range(G)],
        [(53 * g) % 100 for g in range(G)],
        [(131 * g) % 513 for g in range(G)],
        [0] * G,
    ]
    masked.copy_(torch.tensor(counts[0], dtype=torch.int32))
    step()
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        step()
    for it, c in enumerate(counts * 2):
        masked.copy_(torch.tensor(c, dtype=torch.int32))
        out.fill_(-5.0)
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        got = out.view(G, m_max, N)
        for g, mm in enumerate(c):
            assert torch.equal(got[g, :mm], ref[g, :mm]), f"replay {it} group {g}"
            assert bool((got[g, mm:] == -5.0).all()), f"replay {it} group {g}: rows beyond masked_m were written"


def test_deep_gemm_shaped_wrappers_can_be_captured(dev):
    """m_grouped_bf16_nt_contiguous / m_grouped_fp8_nt_contiguous check M against the padded sizes on the host, as
    the reference does; under capture that read is left out, so the wrappers themselves can sit in a graph (with
    ``out=`` given).  Replays must equal the eager calls."""
    from triton_grouped_gemm_amd.gemm.deep_gemm_ops import m_grouped_bf16_nt_contiguous, m_grouped_fp8_nt_contiguous
    from triton_grouped_gemm_amd.quant.fp8_cast import per_block_cast_to_fp8, per_token_cast_to_fp8
    sizes_list = [100, 0, 256, 31, 128, 385]
    padded = [(s + 127) // 128 * 128 for s in sizes_list]
    G, M, N, K = len(sizes_list), sum(padded), 512, 256
    sizes = torch.tensor(sizes_list, dtype=torch.int32, device=dev)
    a, b = _randn((M, K), 31, dev), _randn((G, N, K), 32, dev)
    aq = per_token_cast_to_fp8(a, scales_mn_major=True)
    wq = per_block_cast_to_fp8(b)
    out16 = torch.zeros((M, N), dtype=torch.bfloat16, device=dev)
    out8 = torch.zeros((M, N), dtype=torch.bfloat16, device=dev)
    ref16 = m_grouped_bf16_nt_contiguous(a, b, sizes, out=torch.zeros_like(out16))
    ref8 = m_grouped_fp8_nt_contiguous(aq, wq, sizes, out=torch.zeros_like(out8))
    with pytest.raises(ValueError):  # eagerly the reference's check stays
        m_grouped_bf16_nt_contiguous(a[:-128], b, sizes)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        m_grouped_bf16_nt_contiguous(a, b, sizes, out=out16)
        m_grouped_fp8_nt_contiguous(aq, wq, sizes, out=out8)
    for it in range(3):
        out16.zero_()
        out8.zero_()
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(out16, ref16), f"replay {it}"
        assert torch.equal(out8, ref8), f"replay {it} (fp8)"


def test_k_grouped_wrapper_with_its_work_queue_can_be_captured(dev):
    """The K-grouped kernel finds its tile counters zero and leaves them zero.  A capture without a caller-owned queue
    gets a fresh zeroed tensor whose fill is part of the graph; with ``queue=`` the graph holds the GEMM kernel alone
    and nothing is allocated inside the call.  Replays with other token counts (read on the device) must equal the
    eager call."""
    G, Kt, Mdim, N = 6, 3072, 264, 520
    a, b = _randn((Kt, Mdim), 41, dev), _randn((Kt, N), 42, dev)
    sizes = torch.tensor([512] * G, dtype=torch.int32, device=dev)
    k_grouped_gemm(a, b, sizes)  # first launch outside the capture
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        out = k_grouped_gemm(a, b, sizes)
    for it, routing in enumerate([[512] * G, [3000, 0, 0, 8, 0, 64], [0, 1024, 1024, 0, 1000, 24], [512] * G]):
        sizes.copy_(torch.tensor(routing, dtype=torch.int32))
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(out, k_grouped_gemm(a, b, sizes)), f"replay {it}"
    from triton_grouped_gemm_amd import _native
    queue = torch.zeros(_native.QUEUE_WORDS, dtype=torch.int32, device=dev)
    torch.cuda.synchronize()
    graph2 = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph2):
        out2 = k_grouped_gemm(a, b, sizes, queue=queue)
    for it, routing in enumerate([[3000, 0, 0, 8, 0, 64], [512] * G, [0, 1024, 1024, 0, 1000, 24]]):
        sizes.copy_(torch.tensor(routing, dtype=torch.int32))
        torch.cuda.synchronize()
        graph2.replay()
        torch.cuda.synchronize()
        assert torch.equal(out2, k_grouped_gemm(a, b, sizes)), f"caller-owned queue, replay {it}"
        assert int(queue.abs().sum()) == 0
