"""GPU parity: BF16/FP16 M-grouped, masked and K-grouped GEMM through the C ABI vs the CPU oracle."""
import pytest
import torch

from oracle import gemm_ref
from tests._util import check_16bit_gemm
from triton_grouped_gemm_amd import _native, workloads
from triton_grouped_gemm_amd.gemm.BF16.k_grouped_gemm_TMA import k_grouped_gemm
from triton_grouped_gemm_amd.gemm.BF16.m_grouped_gemm_masked_TMA import m_grouped_gemm_masked
from triton_grouped_gemm_amd.gemm.BF16.m_grouped_gemm_TMA import m_grouped_gemm
from triton_grouped_gemm_amd.gemm.deep_gemm_ops import m_grouped_bf16_nt_contiguous

pytestmark = pytest.mark.gpu


def _randn(shape, scale, seed, dtype=torch.bfloat16):
    g = torch.Generator().manual_seed(seed)
    return (torch.randn(shape, generator=g) * scale).to(dtype)


def _ints(shape, seed, dtype=torch.bfloat16, lo=-1, hi=1):
    g = torch.Generator().manual_seed(seed)
    return torch.randint(lo, hi + 1, shape, generator=g).to(dtype)


@pytest.fixture(params=[0, 1, 2, 3], ids=["tuned", "generic", "four_wave", "stream"])
def variant(request, dev):
    """tuned: what a call gets by default; generic: the shape-agnostic kernel; four_wave: the large-problem kernel
    forced onto every M-grouped NT shape it can take, whatever the size; stream: the weight-streaming configuration
    (128-row tiles, three B slab buffers) forced onto every M-grouped / masked launch, whatever the group sizes
    (other calls run as in `tuned`)."""
    _native.set_option("force_generic", int(request.param == 1))
    _native.set_option("four_wave", 2 if request.param == 2 else 1)
    _native.set_option("variant", 4 if request.param == 3 else 0)
    yield request.param
    _native.set_option("force_generic", 0)
    _native.set_option("four_wave", 1)
    _native.set_option("variant", 0)


def test_config1_tiny_reference_case(dev, variant):
    """BASELINE config 1: G=4, rows [64,128,32,96], K=256, N=512, seed 0, trans_b=True."""
    torch.manual_seed(0)
    sizes = torch.tensor([64, 128, 32, 96], dtype=torch.int32)
    a = (torch.randn(320, 256) / 16).to(torch.bfloat16)
    b = (torch.randn(4, 512, 256) / 16).to(torch.bfloat16)
    out = m_grouped_gemm(a.to(dev), b.to(dev), sizes.to(dev), True)
    rd = check_16bit_gemm(out, gemm_ref.gmm(a, b, sizes, True), gemm_ref.gmm_fp32(a, b, sizes, True), "config1")
    print(f"config1 max-norm rdiff vs bf16 torch reference: {rd:.3e}")
    assert rd <= 1e-3  # the stated BF16 target, max-norm, on the reference's own CPU-runnable case


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("trans_b", [True, False])
@pytest.mark.parametrize("sizes,N,K", [
    ([64, 128, 32, 96], 512, 256),
    ([1, 0, 127, 129, 256, 3, 0, 300], 136, 72),
    ([0, 0, 5], 8, 8),
    ([200] * 16, 264, 64),
    ([300, 0, 417], 2600, 128),  # 11 (tuned) / 21 (generic) column tiles: the tile order's last chunk is narrower
])
def test_m_grouped_exact_on_integer_inputs(dev, variant, dtype, trans_b, sizes, N, K):
    """Entries in {-1,0,1}: every partial sum is an integer <= K <= 256, exactly representable, so the
    result must equal the oracle bit for bit (catches any indexing / scheduling / masking slip)."""
    M = sum(sizes)
    a = _ints((M, K), 1, dtype)
    b = _ints((len(sizes), N, K) if trans_b else (len(sizes), K, N), 2, dtype)
    s = torch.tensor(sizes, dtype=torch.int32)
    out = m_grouped_gemm(a.to(dev), b.to(dev), s.to(dev), trans_b)
    ref = gemm_ref.gmm_fp32(a, b, sizes, trans_b).to(dtype)
    assert torch.equal(out.cpu(), ref)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("num_cu", [-1, 8, 3])  # few workgroups: each one's copy stream crosses many tile boundaries
@pytest.mark.parametrize("sizes,N,K,trans_b", [
    ([300, 0, 417, 256, 1, 700], 520, 256, True),   # four slabs per tile, the least the four-wave kernel takes; a column tail of 8
    ([129, 511, 0, 64], 1000, 384, True),
    ([1024, 77], 256, 1024, True),
    ([5, 0, 0, 250, 3], 136, 512, True),            # a single column tile whose right half lies beyond N
    ([300, 0, 417, 256, 1, 700], 512, 256, False),  # B as [G, K, N]: N a multiple of 256
    ([129, 511, 0, 64], 1024, 384, False),
    ([1024, 77], 256, 1024, False),
])
def test_four_wave_kernel_on_the_shapes_it_takes(dev, dtype, num_cu, sizes, N, K, trans_b):
    """K a multiple of 128 and at least 256 (and, with B as [G, K, N], N a multiple of 256): the four-wave kernel,
    forced, runs these itself (other shapes fall back to the eight-wave kernels, which is what the `four_wave`
    variant of the other tests exercises).  Integer inputs against the oracle bit for bit, then random inputs against
    the shape-agnostic kernel bit for bit."""
    M = sum(sizes)
    s = torch.tensor(sizes, dtype=torch.int32, device=dev)
    b_shape = (len(sizes), N, K) if trans_b else (len(sizes), K, N)
    a_i, b_i = _ints((M, K), 3, dtype), _ints(b_shape, 4, dtype)
    torch.manual_seed(K + N)
    a_r = (torch.randn(M, K, device=dev) * K ** -0.5).to(dtype)
    b_r = torch.randn(b_shape, device=dev).to(dtype)
    _native.set_option("force_generic", 1)
    try:
        ref_r = m_grouped_gemm(a_r, b_r, s, trans_b)
    finally:
        _native.set_option("force_generic", 0)
    _native.set_option("four_wave", 2)
    try:
        out_i = m_grouped_gemm(a_i.to(dev), b_i.to(dev), s, trans_b, numSM=num_cu)
        out_r = m_grouped_gemm(a_r, b_r, s, trans_b, numSM=num_cu)
        out_r2 = m_grouped_gemm(a_r, b_r, s, trans_b, numSM=num_cu)
    finally:
        _native.set_option("four_wave", 1)
    assert torch.equal(out_i.cpu(), gemm_ref.gmm_fp32(a_i, b_i, sizes, trans_b).to(dtype))
    assert torch.equal(out_r, ref_r) and torch.equal(out_r2, ref_r)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("trans_b", [True, False])
def test_m_grouped_decode_sized_groups(dev, dtype, trans_b):
    """No group above 128 rows and more narrow tiles than workgroups: the default launch picks the weight-streaming
    configuration on the device.  Integer inputs, so the result must equal the oracle bit for bit."""
    sizes = [(37 * g) % 129 for g in range(48)]  # 0 .. 128
    sizes[5], sizes[6], sizes[47] = 128, 0, 128  # full 128-row groups and an empty one
    assert max(sizes) == 128 and min(sizes) == 0
    M, N, K = sum(sizes), 1032, 200              # ragged last column tile, K tail
    a = _ints((M, K), 11, dtype)
    b = _ints((48, N, K) if trans_b else (48, K, N), 12, dtype)
    out = m_grouped_gemm(a.to(dev), b.to(dev), torch.tensor(sizes, dtype=torch.int32, device=dev), trans_b)
    assert torch.equal(out.cpu(), gemm_ref.gmm_fp32(a, b, sizes, trans_b).to(dtype))


def _device_choice(sizes, N, workgroups=256):
    """The configuration that the default launch picks on the device for these group sizes: narrow tiles when all
    of them fit one round of the workgroups; else 128-row tiles when their rounds, at 0.7 of a 256-row tile's cost,
    are no more than the 256-row tiles' rounds; else the 256x256 tiles."""
    t256 = sum((s + 255) // 256 for s in sizes)
    t128 = sum((s + 127) // 128 for s in sizes)
    if t256 * ((N + 127) // 128) <= workgroups:
        return "narrow"
    nb = (N + 255) // 256
    rounds = lambda tiles: (tiles * nb + workgroups - 1) // workgroups
    return "stream" if rounds(t128) * 7 <= rounds(t256) * 10 else "wide"


@pytest.mark.parametrize("case", [
    # (group sizes, N, expected choice): both sides of the rule, the 128-row cut with groups above 128 rows
    ([200, 64, 130, 8, 0, 129, 250, 100, 256, 31] * 4, 2048, "stream"),   # 128-row cut has 1.5x the tiles, same rounds
    ([300, 129, 257, 40, 385, 0, 130, 200] * 5, 3072, "stream"),                # three rounds against four shorter ones
    ([512, 384, 300, 256, 700, 0, 1024, 513] * 4, 1536, "wide"),
    ([256, 256, 255, 129] * 4, 4096, "wide"),                              # one round of 256-row tiles, two of 128-row tiles
])
@pytest.mark.parametrize("trans_b", [True, False])
def test_m_grouped_device_choice_of_tile_height(dev, case, trans_b):
    """Integer inputs through the default launch on problems that land on either side of the device-side rule
    (mirrored in _device_choice, which also documents what each problem is meant to exercise): bit-exact against
    the oracle, so a tile prefix that was switched to the 128-row cut wrongly would show as misplaced rows."""
    sizes, N, want = case
    assert _device_choice(sizes, N) == want
    G, M, K = len(sizes), sum(sizes), 136
    a = _ints((M, K), 21, torch.bfloat16)
    b = _ints((G, N, K) if trans_b else (G, K, N), 22, torch.bfloat16)
    out = m_grouped_gemm(a.to(dev), b.to(dev), torch.tensor(sizes, dtype=torch.int32, device=dev), trans_b)
    assert torch.equal(out.cpu(), gemm_ref.gmm_fp32(a, b, sizes, trans_b).to(torch.bfloat16))


@pytest.mark.parametrize("trans_b", [True, False])
@pytest.mark.parametrize("sizes_dtype", [torch.int32, torch.int64])
def test_m_grouped_random_ragged(dev, variant, trans_b, sizes_dtype):
    sizes = [130, 0, 1, 255, 384, 77, 128, 49]
    M, N, K = sum(sizes), 384, 320
    a = _randn((M, K), K ** -0.5, 3)
    b = _randn((8, N, K) if trans_b else (8, K, N), 1.0, 4)
    s = torch.tensor(sizes, dtype=sizes_dtype)
    out = m_grouped_gemm(a.to(dev), b.to(dev), s.to(dev), trans_b)
    check_16bit_gemm(out, gemm_ref.gmm(a, b, sizes, trans_b), gemm_ref.gmm_fp32(a, b, sizes, trans_b), "ragged")


def test_m_grouped_rows_past_sum_untouched_and_neighbours_do_not_leak(dev, variant):
    """sum(sizes) < M: trailing rows keep their previous contents; a NaN row next to a group
    boundary must not contaminate the neighbouring group's rows."""
    from triton_grouped_gemm_amd.gemm.BF16.m_grouped_gemm import _m_grouped_gemm_launch
    sizes = [100, 60]
    M, N, K = 192, 128, 64
    a = _randn((M, K), 0.125, 5)
    a[160:] = float("nan")
    b = _randn((2, N, K), 1.0, 6)
    c = torch.full((M, N), 7.0, dtype=torch.bfloat16, device=dev)
    _m_grouped_gemm_launch(a.to(dev), b.to(dev), c, torch.tensor(sizes, dtype=torch.int32, device=dev), True)
    c = c.cpu()
    assert torch.equal(c[160:], torch.full((32, N), 7.0, dtype=torch.bfloat16))
    check_16bit_gemm(c[:160], gemm_ref.gmm(a[:160], b, sizes, True), gemm_ref.gmm_fp32(a[:160], b, sizes, True), "leak")
    # group-to-expert mapping: swapping the experts changes the answer accordingly
    a2 = a.clone()
    a2[100] = float("nan")  # first row of group 1
    c2 = m_grouped_gemm(a2.to(dev), b.to(dev), torch.tensor(sizes, dtype=torch.int32, device=dev), True).cpu()
    assert torch.isnan(c2[100].float()).all() and torch.isfinite(c2[:100].float()).all()
    assert torch.isfinite(c2[101:160].float()).all()


def test_m_grouped_runs_on_callers_stream_and_with_cpu_sizes(dev):
    sizes = [256, 128]
    a = _randn((384, 128), 0.1, 7)
    b = _randn((2, 256, 128), 1.0, 8)
    st = torch.cuda.Stream(device=dev)
    with torch.cuda.stream(st):
        out = m_grouped_gemm(a.to(dev), b.to(dev), torch.tensor(sizes, dtype=torch.int32), True, numSM=16)
    st.synchronize()
    check_16bit_gemm(out, gemm_ref.gmm(a, b, sizes, True), gemm_ref.gmm_fp32(a, b, sizes, True), "stream")


def test_contiguous_padded_bf16(dev, variant):
    sizes = [100, 0, 128, 300]
    padded = [128, 0, 128, 384]
    Mp, N, K = sum(padded), 256, 128
    a = _randn((Mp, K), K ** -0.5, 9)
    b = _randn((4, N, K), 1.0, 10)
    out = torch.full((Mp, N), 3.0, dtype=torch.bfloat16, device=dev)
    m_grouped_bf16_nt_contiguous(a.to(dev), b.to(dev), torch.tensor(sizes, dtype=torch.int32, device=dev), out=out)
    out = out.cpu()
    start = 0
    for g, (s, p) in enumerate(zip(sizes, padded)):
        if s:
            check_16bit_gemm(out[start:start + s], a[start:start + s] @ b[g].t(),
                             a[start:start + s].float() @ b[g].float().t(), f"padded g{g}")
        assert torch.equal(out[start + s:start + p], torch.full((p - s, N), 3.0, dtype=torch.bfloat16))
        start += p


@pytest.mark.parametrize("psum", [False, True])
def test_contiguous_padded_bf16_explicit_layout(dev, psum):
    # the explicit layout, not size_per_group, says which rows are valid: same padded placement, fewer valid rows
    from triton_grouped_gemm_amd.gemm import layout as L
    sizes = [100, 0, 128, 300]
    in_layout = [90, 0, 128, 257]
    padded = [128, 0, 128, 384]
    Mp, N, K = sum(padded), 256, 128
    a = _randn((Mp, K), K ** -0.5, 19)
    b = _randn((4, N, K), 1.0, 20)
    lay = (L.make_deep_gemm_psum_layout(in_layout) if psum else L.make_deep_gemm_grouped_layout(in_layout)).to(dev)
    out = torch.full((Mp, N), 3.0, dtype=torch.bfloat16, device=dev)
    m_grouped_bf16_nt_contiguous(a.to(dev), b.to(dev), torch.tensor(sizes, dtype=torch.int32, device=dev), out=out,
                                 grouped_layout=lay, use_psum_layout=psum)
    out = out.cpu()
    start = 0
    for g, (s, p) in enumerate(zip(in_layout, padded)):
        if s:
            check_16bit_gemm(out[start:start + s], a[start:start + s] @ b[g].t(),
                             a[start:start + s].float() @ b[g].float().t(), f"layout g{g}")
        assert torch.equal(out[start + s:start + p], torch.full((p - s, N), 3.0, dtype=torch.bfloat16))
        start += p


def _shuffled_layout(sizes, order, block_m=128):
    """Per-row layout with the experts' padded regions laid down in `order`; returns (layout, start row per expert)."""
    lay, starts, pos = [], {}, 0
    for g in order:
        padded = (sizes[g] + block_m - 1) // block_m * block_m
        starts[g] = pos
        lay += [g] * sizes[g] + [-1] * (padded - sizes[g])
        pos += padded
    return torch.tensor(lay, dtype=torch.int32), starts


@pytest.mark.parametrize("layout_dtype", [torch.int32, torch.int64])
def test_contiguous_bf16_per_row_layout_in_any_expert_order(dev, variant, layout_dtype):
    """The reference forwards whatever per-row layout it is given (gemm/deep_gemm_ops.py:24-57): here the experts'
    regions follow one another in a shuffled order.  Checked row by row from the layout's definition
    (out[r] = a[r] . b[layout[r]]^T where layout[r] >= 0), integer inputs, bit for bit."""
    sizes = [100, 0, 128, 300, 7, 256]
    order = [3, 0, 5, 1, 4, 2]
    lay, _ = _shuffled_layout(sizes, order)
    Mp, N, K = lay.numel(), 264, 136
    a = _ints((Mp, K), 31)
    b = _ints((len(sizes), N, K), 32)
    out = torch.full((Mp, N), 3.0, dtype=torch.bfloat16, device=dev)
    m_grouped_bf16_nt_contiguous(a.to(dev), b.to(dev), torch.tensor(sizes, dtype=torch.int32, device=dev), out=out,
                                 grouped_layout=lay.to(layout_dtype).to(dev))
    out = out.cpu()
    valid = lay >= 0
    ref = torch.einsum("rk,rnk->rn", a[valid].float(), b[lay[valid].long()].float()).to(torch.bfloat16)
    assert torch.equal(out[valid], ref)
    assert bool((out[~valid] == 3.0).all()), "padding rows were written"


def test_contiguous_bf16_per_row_layout_with_experts_in_several_regions(dev, variant):
    """A per-row layout in which two experts own two separate regions each (whole 128-row blocks first, the rest
    later): every row still gets its own expert's weights, out[r] = a[r] . b[layout[r]]^T, integer inputs, bit
    for bit; the padded total is the one the reference's check expects (gemm/deep_gemm_ops.py:49-51)."""
    sizes = [300, 128, 0, 200]
    lay = [3] * 128 + [0] * 256 + [1] * 128 + [3] * 72 + [-1] * 56 + [0] * 44 + [-1] * 84
    lay = torch.tensor(lay, dtype=torch.int32)
    Mp, N, K = lay.numel(), 264, 136
    a = _ints((Mp, K), 33)
    b = _ints((len(sizes), N, K), 34)
    out = torch.full((Mp, N), 3.0, dtype=torch.bfloat16, device=dev)
    m_grouped_bf16_nt_contiguous(a.to(dev), b.to(dev), torch.tensor(sizes, dtype=torch.int32, device=dev), out=out,
                                 grouped_layout=lay.to(dev))
    out = out.cpu()
    valid = lay >= 0
    ref = torch.einsum("rk,rnk->rn", a[valid].float(), b[lay[valid].long()].float()).to(torch.bfloat16)
    assert torch.equal(out[valid], ref)
    assert bool((out[~valid] == 3.0).all()), "padding rows were written"


@pytest.mark.parametrize("trans_b", [True, False])
def test_masked_small(dev, variant, trans_b):
    G, m_max, N, K = 6, 256, 264, 192
    masked = [0, 256, 1, 129, 77, 200]
    lhs = _randn((G * m_max, K), K ** -0.5, 11)
    for g, mm in enumerate(masked):  # rows beyond masked_m are garbage
        lhs[g * m_max + mm:(g + 1) * m_max] = float("nan")
    rhs = _randn((G, N, K), 1.0, 12)
    rhs_in = rhs if trans_b else rhs.transpose(1, 2).contiguous()
    out = torch.full((G * m_max, N), -5.0, dtype=torch.bfloat16, device=dev)
    ret = m_grouped_gemm_masked(lhs.to(dev), rhs_in.to(dev), out, torch.tensor(masked, dtype=torch.int32, device=dev),
                                m_max, trans_b)
    assert ret is None
    out = out.cpu()
    refs = gemm_ref.masked_gmm(lhs, rhs, masked, m_max)
    refs32 = gemm_ref.masked_gmm(lhs, rhs, masked, m_max, fp32=True)
    for g, mm in enumerate(masked):
        blk = out[g * m_max:(g + 1) * m_max]
        if mm:
            check_16bit_gemm(blk[:mm], refs[g], refs32[g], f"masked g{g}")
        assert torch.equal(blk[mm:], torch.full((m_max - mm, N), -5.0, dtype=torch.bfloat16))


def test_masked_decode_sized_counts(dev):
    """Masked launch whose counts stay at or below 128 with m_max = 512 (decode): the weight-streaming
    configuration is picked on the device; exact on integer inputs, rows beyond masked_m untouched."""
    G, m_max, N, K = 40, 512, 1024, 136
    masked = [(53 * g) % 129 for g in range(G)]
    masked[3], masked[4] = 128, 0
    lhs = _ints((G * m_max, K), 21)
    rhs = _ints((G, N, K), 22)
    out = torch.full((G * m_max, N), -5.0, dtype=torch.bfloat16, device=dev)
    m_grouped_gemm_masked(lhs.to(dev), rhs.to(dev), out, torch.tensor(masked, dtype=torch.int32, device=dev), m_max)
    out = out.cpu().view(G, m_max, N)
    ref = torch.bmm(lhs.float().view(G, m_max, K), rhs.float().transpose(1, 2)).to(torch.bfloat16)
    for g, mm in enumerate(masked):
        assert torch.equal(out[g, :mm], ref[g, :mm]), f"group {g}"
        assert bool((out[g, mm:] == -5.0).all()), f"group {g}: rows beyond masked_m were written"


@pytest.mark.parametrize("trans_b", [True, False])
def test_m_grouped_launch_that_both_kernels_look_at(dev, trans_b):
    """An M-grouped launch with many tiles but fewer than 512 rows per group on average: like a masked one it enqueues
    the four-wave and the eight-wave kernel and the sizes decide on the device which runs (here: groups of up to 700
    rows, 256-row tiles pay).  Exact on integer inputs; the same bits as either kernel forced."""
    G, N, K = 96, 1024, 256
    sizes = [(131 * g) % 700 for g in range(G)]
    M = sum(sizes)
    assert M < 512 * G
    a = _ints((M, K), 51)
    b = _ints((G, N, K) if trans_b else (G, K, N), 52)
    ref = gemm_ref.gmm_fp32(a, b, sizes, trans_b).to(torch.bfloat16)
    s_dev, a_dev, b_dev = torch.tensor(sizes, dtype=torch.int32, device=dev), a.to(dev), b.to(dev)
    for four_wave in (1, 2, 0):
        _native.set_option("four_wave", four_wave)
        try:
            out = m_grouped_gemm(a_dev, b_dev, s_dev, trans_b)
        finally:
            _native.set_option("four_wave", 1)
        assert torch.equal(out.cpu(), ref), f"four_wave={four_wave}"


@pytest.mark.parametrize("counts", ["large", "small", "mixed"])
def test_masked_launch_that_both_kernels_look_at(dev, counts):
    """A masked launch large enough for the four-wave kernel (K a multiple of 128, many tiles): it and the eight-wave
    kernel are both enqueued and decide from the counts, on the device, which of them runs -- the four-wave kernel
    where 256-row tiles pay (large counts), the eight-wave kernels otherwise (small counts: 128-row tiles).  Exact on
    integer inputs in every regime, rows beyond masked_m untouched, and the same bits when either kernel is forced."""
    G, m_max, N, K = 72, 512, 1032, 256
    if counts == "large":
        masked = [512 - (37 * g) % 200 for g in range(G)]
    elif counts == "small":
        masked = [(53 * g) % 100 for g in range(G)]
    else:
        masked = [(131 * g) % 513 for g in range(G)]
    masked[5], masked[6] = 0, 512 if counts != "small" else 99
    lhs = _ints((G * m_max, K), 31)
    rhs = _ints((G, N, K), 32)
    ref = torch.bmm(lhs.float().view(G, m_max, K), rhs.float().transpose(1, 2)).to(torch.bfloat16)
    mm_dev = torch.tensor(masked, dtype=torch.int32, device=dev)
    lhs_d, rhs_d = lhs.to(dev), rhs.to(dev)
    outs = []
    for four_wave in (1, 2, 0):  # decided on the device; four-wave kernel forced; eight-wave kernels only
        _native.set_option("four_wave", four_wave)
        try:
            out = torch.full((G * m_max, N), -5.0, dtype=torch.bfloat16, device=dev)
            m_grouped_gemm_masked(lhs_d, rhs_d, out, mm_dev, m_max)
        finally:
            _native.set_option("four_wave", 1)
        outs.append(out.cpu().view(G, m_max, N))
    for out in outs:
        for g, mm in enumerate(masked):
            assert torch.equal(out[g, :mm], ref[g, :mm]), f"group {g}"
            assert bool((out[g, mm:] == -5.0).all()), f"group {g}: rows beyond masked_m were written"


def test_masked_full_mask_reduces_to_bmm_exact(dev, variant):
    G, m_max, N, K = 4, 128, 128, 64
    lhs = _ints((G * m_max, K), 13)
    rhs = _ints((G, N, K), 14)
    out = torch.empty((G * m_max, N), dtype=torch.bfloat16, device=dev)
    m_grouped_gemm_masked(lhs.to(dev), rhs.to(dev), out, torch.full((G,), m_max, dtype=torch.int64, device=dev), m_max)
    ref = torch.bmm(lhs.float().view(G, m_max, K), rhs.float().transpose(1, 2)).to(torch.bfloat16)
    assert torch.equal(out.cpu().view(G, m_max, N), ref)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("sizes,Mdim,N", [
    ([128, 256, 0, 64], 256, 128),
    ([1, 33, 0, 130, 7], 136, 72),
    ([512], 128, 384),
    ([40, 0, 200], 520, 2600),  # ragged last chunk of the tile order, three row tiles
])
def test_k_grouped_exact_on_integer_inputs(dev, variant, dtype, sizes, Mdim, N):
    """Entries in {-1,0,1} and every group <= 512 tokens... sums stay below 256 in magnitude with
    overwhelming probability; verified on the oracle side before comparing bit for bit."""
    Kt = sum(sizes)
    a = _ints((Kt, Mdim), 15, dtype)
    b = _ints((Kt, N), 16, dtype)
    ref32 = gemm_ref.gmm_dw(a, b, sizes, fp32=True)
    assert ref32.abs().max() <= 256
    s = torch.tensor(sizes, dtype=torch.int32, device=dev)
    out = k_grouped_gemm(a.to(dev), b.to(dev), s)
    assert out.shape == (len(sizes), Mdim, N)
    assert torch.equal(out.cpu(), ref32.to(dtype))


def test_k_grouped_random_with_explicit_bounds(dev, variant):
    sizes = [300, 0, 1000, 77, 128]
    Kt, Mdim, N = sum(sizes), 384, 264
    a = _randn((Kt, Mdim), 1.0, 17)
    b = _randn((Kt, N), 1.0, 18)
    s = torch.tensor(sizes, dtype=torch.int64, device=dev)
    end = s.cumsum(0)
    out = k_grouped_gemm(a.to(dev), b.to(dev), s, group_start=end - s, group_end=end)
    ref, ref32 = gemm_ref.gmm_dw(a, b, sizes), gemm_ref.gmm_dw(a, b, sizes, fp32=True)
    assert torch.count_nonzero(out[1]) == 0  # empty group -> zeros
    for g in (0, 2, 3, 4):
        check_16bit_gemm(out[g], ref[g], ref32[g], f"kgrouped g{g}")


def test_k_grouped_single_group_is_plain_transposed_matmul(dev, variant):
    a = _randn((640, 128), 1.0, 19)
    b = _randn((640, 256), 1.0, 20)
    out = k_grouped_gemm(a.to(dev), b.to(dev), torch.tensor([640], dtype=torch.int32, device=dev))
    check_16bit_gemm(out[0], a.t() @ b, a.float().t() @ b.float(), "kgrouped G=1")


def test_medium_dirichlet_config_shape(dev, variant):
    """Config-2 style draw at 1/16 scale: G=128 experts, 40960 rows in 128-row blocks, gate-up shape."""
    G, M, N, K = 128, 40960, 1536, 2048
    sizes = workloads.dirichlet_multinomial_sizes(G, M, 128, seed=21)
    assert int(sizes.sum()) == M
    a = workloads.randn_bf16((M, K), K ** -0.5, 22)
    b = workloads.randn_bf16((G, N, K), K ** -0.5, 23)
    out = m_grouped_gemm(a.to(dev), b.to(dev), sizes.to(dev), True)
    # oracle on a sample of groups (CPU time) -- the largest, the smallest non-empty, and two more
    order = torch.argsort(sizes)
    nz = [int(i) for i in order if sizes[i] > 0]
    starts = (sizes.cumsum(0) - sizes).tolist()
    for g in {nz[0], nz[-1], nz[len(nz) // 2], nz[len(nz) // 3]}:
        s0, n = starts[g], int(sizes[g])
        n = min(n, 512)
        ag = a[s0:s0 + n]
        check_16bit_gemm(out[s0:s0 + n], ag @ b[g].t(), ag.float() @ b[g].float().t(), f"medium g{g}")


@pytest.mark.parametrize("G", [384, 512, 600])  # up to 512 groups run on the tuned kernels, more on the shape-agnostic one
def test_many_groups_exact(dev, variant, G):
    pattern = [3, 0, 70, 129, 1, 256]
    sizes = [pattern[g % len(pattern)] for g in range(G)]
    M, N, K = sum(sizes), 136, 64
    a = _ints((M, K), 21, torch.bfloat16)
    b = _ints((G, N, K), 22, torch.bfloat16)
    out = m_grouped_gemm(a.to(dev), b.to(dev), torch.tensor(sizes, dtype=torch.int32, device=dev), True)
    assert torch.equal(out.cpu(), gemm_ref.gmm_fp32(a, b, sizes, True).to(torch.bfloat16))
    kt = k_grouped_gemm(a.to(dev), a.to(dev), torch.tensor(sizes, dtype=torch.int64, device=dev))
    ref = gemm_ref.gmm_dw(a, a, sizes, fp32=True)
    assert ref.abs().max() <= 256 and torch.equal(kt.cpu(), ref.to(torch.bfloat16))


@pytest.mark.parametrize("sizes", [
    [5000, 0, 64, 1200, 0, 0, 8, 300, 2048, 16, 700, 1],      # few long tiles, runs of empty and one-slab groups
    [64] * 40,                                                # one-slab tiles only: the copy stream looks furthest ahead
    [0, 0, 0, 9000],                                          # empty groups first in index order
    [(53 * g * g + 17 * g) % 3000 for g in range(96)],
])
@pytest.mark.parametrize("num_cu", [-1, 100, 64, 8])  # 100: not a multiple of 8, one counter; 8: one workgroup per XCD
def test_k_grouped_work_queue_equals_fixed_assignment(dev, sizes, num_cu):
    """tgg_k_grouped_gemm_queued (tile ids drawn from counters in device memory, largest groups first) against
    tgg_k_grouped_gemm (fixed assignment) and the oracle: same bits, whichever workgroup computes a tile; the
    kernel leaves the counters zero, so a second launch on the same words needs no clearing."""
    from triton_grouped_gemm_amd import _native
    G, Mdim, N = len(sizes), 520, 776
    Kt = sum(sizes)
    a, b = _randn((Kt, Mdim), 1.0, 31).to(dev), _randn((Kt, N), 1.0, 32).to(dev)
    s = torch.tensor(sizes, dtype=torch.int32, device=dev)
    end = s.cumsum(0).to(torch.int32)
    start = (end - s).to(torch.int32)
    fixed = torch.full((G, Mdim, N), float("nan"), dtype=torch.bfloat16, device=dev)
    drawn = torch.full((G, Mdim, N), float("nan"), dtype=torch.bfloat16, device=dev)
    queue = torch.zeros(_native.QUEUE_WORDS, dtype=torch.int32, device=dev)
    st = _native.stream_of(a)
    _native.call("tgg_k_grouped_gemm", a.data_ptr(), b.data_ptr(), fixed.data_ptr(), start.data_ptr(), end.data_ptr(),
                 G, Mdim, N, Kt, _native.BF16, num_cu, st)
    _native.call("tgg_k_grouped_gemm_queued", a.data_ptr(), b.data_ptr(), drawn.data_ptr(), start.data_ptr(),
                 end.data_ptr(), G, Mdim, N, Kt, _native.BF16, num_cu, queue.data_ptr(), st)
    assert torch.equal(fixed, drawn)
    assert int(queue.abs().sum()) == 0, "the last workgroup clears the queue"
    drawn.fill_(float("nan"))
    _native.call("tgg_k_grouped_gemm_queued", a.data_ptr(), b.data_ptr(), drawn.data_ptr(), start.data_ptr(),
                 end.data_ptr(), G, Mdim, N, Kt, _native.BF16, num_cu, queue.data_ptr(), st)
    assert torch.equal(fixed, drawn), "second launch on the same, uncleared words"
    assert int(queue.abs().sum()) == 0
    check_16bit_gemm(drawn, gemm_ref.gmm_dw(a.cpu(), b.cpu(), sizes), gemm_ref.gmm_dw(a.cpu(), b.cpu(), sizes, fp32=True),
                     "queued K-grouped")
