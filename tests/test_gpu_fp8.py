"""GPU parity: FP8 grouped GEMMs (per-channel x per-expert scales, block scales) through the C ABI.

Tolerance: rdiff = max|out-ref| / max(max|out|, max|ref|) <= 2e-2 against the fp32 matmul of the
dequantised operands (the stated FP8 target); integer-valued cases must be exact.
"""
import numpy as np
import pytest
import torch

from oracle import gemm_ref, quant_ref
from tests._util import to_np_f32
from triton_grouped_gemm_amd import _native
from triton_grouped_gemm_amd.gemm.deep_gemm_ops import m_grouped_fp8_nt_contiguous
from triton_grouped_gemm_amd.gemm.FP8.k_grouped_gemm_channel_expert import matmul
from triton_grouped_gemm_amd.gemm.FP8.m_grouped_gemm_channel_expert import gmm_fp8_act_per_channel_w_per_expert

pytestmark = pytest.mark.gpu
FP8_RDIFF = 2e-2
TORCH_FP8 = {"e4m3fn": torch.float8_e4m3fn, "e5m2": torch.float8_e5m2}


def _randn(shape, seed, scale=1.0):
    g = torch.Generator().manual_seed(seed)
    return (torch.randn(shape, generator=g) * scale).to(torch.bfloat16)


def _codes_to_torch(codes: np.ndarray, fmt: str) -> torch.Tensor:
    return torch.from_numpy(codes.copy()).view(TORCH_FP8[fmt])


@pytest.fixture(params=[0, 1, 2], ids=["tuned", "generic", "stream"])
def variant(request, dev):
    """tuned: what a call gets by default; generic: the shape-agnostic kernel; stream: the weight-streaming
    configuration (128-row tiles, three B slab buffers) forced onto every M-grouped launch, whatever the group sizes."""
    _native.set_option("force_generic", int(request.param == 1))
    _native.set_option("variant", 4 if request.param == 2 else 0)
    yield request.param
    _native.set_option("force_generic", 0)
    _native.set_option("variant", 0)


@pytest.mark.parametrize("fmt_a,fmt_b", [("e4m3fn", "e4m3fn"), ("e5m2", "e4m3fn"), ("e4m3fn", "e5m2"), ("e5m2", "e5m2")])
@pytest.mark.parametrize("dtype_out", [torch.bfloat16, torch.float16])
def test_fp8_channel_m_grouped(dev, variant, fmt_a, fmt_b, dtype_out):
    """The reference's own example layout (gemm/FP8/m_grouped_gemm_channel_expert.py:293-315) at small size:
    per-token activation scale, per-expert weight scale expanded to [G*N]."""
    sizes = [125, 0, 259, 128, 3]
    M, N, K = sum(sizes), 264, 256
    x = to_np_f32(_randn((M, K), 30))
    w = to_np_f32(_randn((len(sizes), N, K), 31))
    xq, xs = quant_ref.per_row_cast_to_fp8(x, fmt_a)
    wq, ws = quant_ref.per_expert_cast_to_fp8(w, fmt_b)
    ws_exp = np.repeat(ws, N, axis=1).reshape(-1)  # .view(-1,1).repeat(1,N)
    out = gmm_fp8_act_per_channel_w_per_expert(
        _codes_to_torch(xq, fmt_a).to(dev), torch.from_numpy(xs).to(dev), _codes_to_torch(wq, fmt_b).to(dev),
        torch.from_numpy(ws_exp).to(dev), torch.tensor(sizes, dtype=torch.int32, device=dev), dtype_out)
    assert out.dtype == dtype_out and out.shape == (M, N)
    ref = gemm_ref.fp8_channel_reference(torch.from_numpy(quant_ref.dequant(xq, fmt_a)), torch.from_numpy(xs),
                                         torch.from_numpy(quant_ref.dequant(wq, fmt_b)), torch.from_numpy(ws_exp), sizes)
    rd = gemm_ref.rdiff(out.cpu().float(), ref)
    assert rd <= FP8_RDIFF, rd
    # exactly representable products; the matrix instruction truncates them below 2^-13 of an instruction's largest
    # one, so the 16-bit output rounding dominates what remains
    assert rd <= (2.0 ** -7 if dtype_out == torch.bfloat16 else 2.0 ** -10)


@pytest.mark.parametrize("K", [128, 176, 48, 400])  # 176, 48, 400: the last 128-deep slab is cut short by K
def test_fp8_channel_exact_on_integer_codes(dev, variant, K):
    sizes = [64, 1, 191]
    M, N = 256, 128
    g = torch.Generator().manual_seed(32)
    xa = torch.randint(-2, 3, (M, K), generator=g).float()
    wb = torch.randint(-2, 3, (3, N, K), generator=g).float()
    sa = torch.tensor([0.5, 1.0, 2.0, 4.0])[torch.randint(0, 4, (M,), generator=g)]
    sb = torch.tensor([0.25, 1.0])[torch.randint(0, 2, (3 * N,), generator=g)]
    out = gmm_fp8_act_per_channel_w_per_expert(
        xa.to(torch.float8_e4m3fn).to(dev), sa.view(-1, 1).to(dev), wb.to(torch.float8_e4m3fn).to(dev), sb.to(dev),
        torch.tensor(sizes, dtype=torch.int64, device=dev), torch.bfloat16)
    ref = gemm_ref.fp8_channel_reference(xa, sa, wb, sb, sizes)
    # |codes| <= 2 and power-of-two scales: fp32 sums are exact; bf16 holds them exactly up to 256 units
    assert torch.equal(out.cpu(), ref.to(torch.bfloat16))
    if K == 128:
        assert ref.abs().max() <= 2048 and torch.equal(ref, ref.to(torch.bfloat16).float())


@pytest.mark.parametrize("dtype_a,dtype_b", [(1, 1), (2, 1)])
def test_fp8_k_grouped_channel(dev, variant, dtype_a, dtype_b):
    """Layout of the reference's generator (gemm/FP8/k_grouped_gemm_channel_expert.py:238-268): tokens of
    every expert zero-padded to 128, scales [rows, G] stored expert-major."""
    fa, fb = ("e4m3fn" if dtype_a == 1 else "e5m2"), ("e4m3fn" if dtype_b == 1 else "e5m2")
    tokens = [125, 300, 0, 128]
    padded = [(t + 127) // 128 * 128 for t in tokens]
    M, N, G = 136, 264, len(tokens)
    xq_l, xs_l, yq_l, ys_l = [], [], [], []
    for i, (t, p) in enumerate(zip(tokens, padded)):
        x = np.zeros((M, p), np.float32)
        y = np.zeros((N, p), np.float32)
        x[:, :t] = to_np_f32(_randn((M, t), 40 + i))
        y[:, :t] = to_np_f32(_randn((N, t), 50 + i))
        if p == 0:
            xq, xs = np.zeros((M, 0), np.uint8), np.full((M, 1), 1e-4 / 448, np.float32)
            yq, ys = np.zeros((N, 0), np.uint8), np.full((N, 1), 1e-4 / 448, np.float32)
        else:
            xq, xs = quant_ref.per_row_cast_to_fp8(x, fa)
            yq, ys = quant_ref.per_row_cast_to_fp8(y, fb)
        xq_l.append(xq); xs_l.append(xs); yq_l.append(yq); ys_l.append(ys)
    xq, yq = np.concatenate(xq_l, 1), np.concatenate(yq_l, 1)
    xs, ys = np.concatenate(xs_l, 1), np.concatenate(ys_l, 1)
    Kt = sum(padded)
    xs_t = torch.from_numpy(xs).t().contiguous().t().to(dev)  # [M, G] with strides (1, M), as the reference builds it
    ys_t = torch.from_numpy(ys).to(dev)                        # plain contiguous [N, G]: logical indexing must still hold
    out = matmul(_codes_to_torch(xq, fa).to(dev), xs_t, _codes_to_torch(yq, fb).to(dev), ys_t,
                 torch.tensor(padded, dtype=torch.int32, device=dev), M, N, Kt, G, dtype_a, dtype_b)
    assert out.shape == (G, M, N) and out.dtype == torch.bfloat16
    ref = gemm_ref.fp8_k_grouped_channel_reference(torch.from_numpy(quant_ref.dequant(xq, fa)), torch.from_numpy(xs),
                                                   torch.from_numpy(quant_ref.dequant(yq, fb)), torch.from_numpy(ys), padded)
    assert torch.count_nonzero(out[2]) == 0
    rd = gemm_ref.rdiff(out.cpu().float(), ref)
    assert rd <= FP8_RDIFF and rd <= 2.0 ** -7, rd


def _k_grouped_unpadded_case(tokens, M, N, seed):
    """Per-expert blocks quantised per row (one scale per row and expert) and laid side by side WITHOUT padding."""
    xq_l, xs_l, yq_l, ys_l = [], [], [], []
    for i, t in enumerate(tokens):
        if t == 0:
            xq, xs = np.zeros((M, 0), np.uint8), np.full((M, 1), 1e-4 / 448, np.float32)
            yq, ys = np.zeros((N, 0), np.uint8), np.full((N, 1), 1e-4 / 448, np.float32)
        else:
            xq, xs = quant_ref.per_row_cast_to_fp8(to_np_f32(_randn((M, t), seed + i)))
            yq, ys = quant_ref.per_row_cast_to_fp8(to_np_f32(_randn((N, t), seed + 50 + i)))
        xq_l.append(xq); xs_l.append(xs); yq_l.append(yq); ys_l.append(ys)
    return np.concatenate(xq_l, 1), np.concatenate(xs_l, 1), np.concatenate(yq_l, 1), np.concatenate(ys_l, 1)


@pytest.mark.parametrize("tokens,tuned_runs", [
    ([125, 300, 0, 128, 7], False),      # not multiples of 16: the shape-agnostic kernel takes the call
    ([112, 304, 0, 128, 16], True),      # multiples of 16, not of 128: the tuned kernel cuts every group's last slab
    ([128, 384, 0, 256], True),
    ([16, 16, 16, 0, 48], True),
])
@pytest.mark.parametrize("M,N", [(136, 264), (512, 256)])
def test_fp8_channel_k_grouped_unpadded_counts(dev, tokens, tuned_runs, M, N):
    """Token counts as they are (the reference pads every expert to 128 with zero data,
    gemm/FP8/k_grouped_gemm_channel_expert.py:238-260; here a segment simply ends where its count says): tuned and
    shape-agnostic path against the oracle, and the device-side choice between them seen from outside."""
    G, Kt = len(tokens), sum(tokens)
    xq, xs, yq, ys = _k_grouped_unpadded_case(tokens, M, N, 60)
    ref = gemm_ref.fp8_k_grouped_channel_reference(torch.from_numpy(quant_ref.dequant(xq)), torch.from_numpy(xs),
                                                   torch.from_numpy(quant_ref.dequant(yq)), torch.from_numpy(ys), tokens)
    args = (_codes_to_torch(xq, "e4m3fn").to(dev), torch.from_numpy(xs).to(dev), _codes_to_torch(yq, "e4m3fn").to(dev),
            torch.from_numpy(ys).to(dev), torch.tensor(tokens, dtype=torch.int32, device=dev), M, N, Kt, G)
    outs = {}
    for name, opts in (("default", {}), ("generic", {"force_generic": 1}), ("tuned_only", {"kg_second_launch": 0})):
        for k, v in opts.items():
            _native.set_option(k, v)
        try:
            if name == "tuned_only":
                # call the C ABI on a sentinel-filled output to see whether the tuned kernel ran
                out = torch.full((G, M, N), -77.0, dtype=torch.bfloat16, device=dev)
                xs_e = args[1].t().contiguous()
                ys_e = args[3].t().contiguous()
                _native.call("tgg_k_grouped_gemm_fp8_channel", args[0].data_ptr(), xs_e.data_ptr(), args[2].data_ptr(),
                             ys_e.data_ptr(), out.data_ptr(), args[4].data_ptr(), G, M, N, Kt, _native.E4M3, _native.E4M3,
                             -1, _native.stream_of(out))
                torch.cuda.synchronize()
            else:
                out = matmul(*args)
        finally:
            for k in opts:
                _native.set_option(k, 1 if k == "kg_second_launch" else 0)
        outs[name] = out.cpu().float()
    for name in ("default", "generic"):
        rd = gemm_ref.rdiff(outs[name], ref)
        assert rd <= FP8_RDIFF and rd <= 2.0 ** -7, (name, rd)
        for g, t in enumerate(tokens):
            if t == 0:
                assert torch.count_nonzero(outs[name][g]) == 0
    if tuned_runs:
        assert torch.equal(outs["tuned_only"], outs["default"])
    else:
        assert bool((outs["tuned_only"] == -77.0).all())      # the tuned kernel saw the counts and left
        assert torch.equal(outs["default"], outs["generic"])  # ... to the shape-agnostic kernel


@pytest.mark.parametrize("tokens", [[512, 0, 128, 2048, 16, 0, 0, 640, 128, 128, 1024, 16], [128] * 24])
def test_fp8_k_grouped_work_queue_equals_fixed_assignment(dev, tokens):
    """tgg_k_grouped_gemm_fp8_channel_queued (tile ids drawn from counters in device memory) against the fixed
    assignment: same bits whichever workgroup computes a tile.  Token counts are multiples of 16, so the tuned
    kernel runs and draws; the wrapper's own result (queued as well) is checked against the oracle elsewhere."""
    from triton_grouped_gemm_amd import _native
    M, N, G = 264, 520, len(tokens)
    xq, xs, yq, ys = _k_grouped_unpadded_case(tokens, M, N, 90)
    Kt = sum(tokens)
    x = _codes_to_torch(xq, "e4m3fn").contiguous().to(dev)
    y = _codes_to_torch(yq, "e4m3fn").contiguous().to(dev)
    xs_t = torch.from_numpy(np.ascontiguousarray(xs.T)).to(dev)  # element (row, g) at g * rows + row
    ys_t = torch.from_numpy(np.ascontiguousarray(ys.T)).to(dev)
    tok = torch.tensor(tokens, dtype=torch.int32, device=dev)
    fixed = torch.full((G, M, N), float("nan"), dtype=torch.bfloat16, device=dev)
    drawn = torch.full((G, M, N), float("nan"), dtype=torch.bfloat16, device=dev)
    queue = torch.zeros(_native.QUEUE_WORDS, dtype=torch.int32, device=dev)
    st = _native.stream_of(x)
    _native.call("tgg_k_grouped_gemm_fp8_channel", x.data_ptr(), xs_t.data_ptr(), y.data_ptr(), ys_t.data_ptr(),
                 fixed.data_ptr(), tok.data_ptr(), G, M, N, Kt, _native.E4M3, _native.E4M3, -1, st)
    _native.call("tgg_k_grouped_gemm_fp8_channel_queued", x.data_ptr(), xs_t.data_ptr(), y.data_ptr(), ys_t.data_ptr(),
                 drawn.data_ptr(), tok.data_ptr(), G, M, N, Kt, _native.E4M3, _native.E4M3, -1, queue.data_ptr(), st)
    assert not bool(torch.isnan(fixed.float()).any())
    assert torch.equal(fixed, drawn)
    assert int(queue.abs().sum()) == 0, "the last workgroup clears the queue"
    drawn.fill_(float("nan"))
    _native.call("tgg_k_grouped_gemm_fp8_channel_queued", x.data_ptr(), xs_t.data_ptr(), y.data_ptr(), ys_t.data_ptr(),
                 drawn.data_ptr(), tok.data_ptr(), G, M, N, Kt, _native.E4M3, _native.E4M3, -1, queue.data_ptr(), st)
    assert torch.equal(fixed, drawn), "second launch on the same, uncleared words"


def _block_scaled_case(sizes, N, K, seed):
    padded = [(s + 127) // 128 * 128 for s in sizes]
    Mp, G = sum(padded), len(sizes)
    a = to_np_f32(_randn((Mp, K), seed))
    w = to_np_f32(_randn((G, N, K), seed + 1))
    aq, sa = quant_ref.per_token_cast_to_fp8(a)
    wq = np.zeros((G, N, K), np.uint8)
    sb = np.zeros((G, (N + 127) // 128, K // 128), np.float32)
    for g in range(G):
        wq[g], sb[g] = quant_ref.per_block_cast_to_fp8(w[g])
    return padded, aq, sa, wq, sb


@pytest.mark.parametrize("sizes,N,K", [([128, 0, 100, 300], 256, 512), ([5], 200, 128), ([256, 256], 384, 1024)])
def test_fp8_block_scaled(dev, variant, sizes, N, K):
    """BASELINE config 5 recipe at small size: 1x128 activation scales, 128x128 weight scales, bf16 out,
    compared with the fp32 matmul of the dequantised operands."""
    padded, aq, sa, wq, sb = _block_scaled_case(sizes, N, K, 60)
    Mp = sum(padded)
    out = torch.full((Mp, N), 9.0, dtype=torch.bfloat16, device=dev)
    ret = m_grouped_fp8_nt_contiguous((_codes_to_torch(aq, "e4m3fn").to(dev), torch.from_numpy(sa).to(dev)),
                                      (_codes_to_torch(wq, "e4m3fn").to(dev), torch.from_numpy(sb).to(dev)),
                                      torch.tensor(sizes, dtype=torch.int32, device=dev), out=out)
    assert ret is out
    ref = gemm_ref.fp8_block_scaled_reference(torch.from_numpy(quant_ref.dequant(aq)), torch.from_numpy(sa),
                                              torch.from_numpy(quant_ref.dequant(wq)), torch.from_numpy(sb), sizes)
    out = out.cpu().float()
    start = 0
    for s, p in zip(sizes, padded):
        assert torch.equal(out[start + s:start + p], torch.full((p - s, N), 9.0))  # pad rows untouched
        out[start + s:start + p] = 0
        start += p
    rd = gemm_ref.rdiff(out, ref)
    assert rd <= FP8_RDIFF and rd <= 2.0 ** -7, rd


@pytest.mark.parametrize("K", [384, 320, 64])  # 320, 64: K ends inside a 128-wide scale block
def test_fp8_block_scaled_exact_with_power_of_two_scales(dev, variant, K):
    """Small-integer codes and power-of-two scales: every product and partial sum is exact, so the
    kernel must reproduce the closed form bit for bit (pins the scale indexing: a swapped or
    transposed scale changes the answer)."""
    g = torch.Generator().manual_seed(70)
    sizes = [100, 128, 28]
    padded = [128, 128, 128]
    Mp, N, G = 384, 256, 3
    kb = (K + 127) // 128
    aq = torch.randint(-3, 4, (Mp, K), generator=g).float()
    bq = torch.randint(-3, 4, (G, N, K), generator=g).float()
    pw = torch.tensor([0.25, 0.5, 1.0, 2.0])
    sa = pw[torch.randint(0, 4, (Mp, kb), generator=g)]
    sb = pw[torch.randint(0, 4, (G, N // 128, kb), generator=g)]
    out = m_grouped_fp8_nt_contiguous((aq.to(torch.float8_e4m3fn).to(dev), sa.to(dev)),
                                      (bq.to(torch.float8_e4m3fn).to(dev), sb.to(dev)),
                                      torch.tensor(sizes, dtype=torch.int32, device=dev))
    # all fp32 operations are exact here, so the only rounding is the final one to bf16
    ref = gemm_ref.fp8_block_scaled_reference(aq, sa, bq, sb, sizes).to(torch.bfloat16)
    out = out.cpu()
    start = 0
    for s, p in zip(sizes, padded):
        assert torch.equal(out[start:start + s], ref[start:start + s])
        start += p


@pytest.mark.parametrize("sizes,N", [
    ([200, 64, 130, 8, 0, 129, 250, 100, 256, 31] * 4, 2048),    # the device picks 128-row tiles; groups above 128 rows
    ([300, 129, 257, 40, 385, 0, 130, 200] * 5, 3072),           # likewise, three rounds against four shorter ones
    ([512, 384, 300, 256, 700, 0, 1024, 513] * 4, 1536),         # 256-row tiles
])
def test_fp8_block_scaled_device_choice_of_tile_height(dev, sizes, N):
    """The default launch on problems on either side of the device-side choice of tile height (the same rule as in
    the 16-bit kernels, see test_gpu_bf16._device_choice): small-integer codes and power-of-two scales, so the
    result must equal the closed form bit for bit; a tile prefix switched to the 128-row cut wrongly, or scales
    fetched for the wrong rows, would show."""
    g = torch.Generator().manual_seed(71)
    padded = [(s + 127) // 128 * 128 for s in sizes]
    Mp, G, K = sum(padded), len(sizes), 256
    aq = torch.randint(-3, 4, (Mp, K), generator=g).float()
    bq = torch.randint(-3, 4, (G, N, K), generator=g).float()
    pw = torch.tensor([0.25, 0.5, 1.0, 2.0])
    sa = pw[torch.randint(0, 4, (Mp, K // 128), generator=g)]
    sb = pw[torch.randint(0, 4, (G, N // 128, K // 128), generator=g)]
    out = m_grouped_fp8_nt_contiguous((aq.to(torch.float8_e4m3fn).to(dev), sa.to(dev)),
                                      (bq.to(torch.float8_e4m3fn).to(dev), sb.to(dev)),
                                      torch.tensor(sizes, dtype=torch.int32, device=dev))
    ref = gemm_ref.fp8_block_scaled_reference(aq, sa, bq, sb, sizes).to(torch.bfloat16)
    out = out.cpu()
    start = 0
    for s_, p_ in zip(sizes, padded):
        assert torch.equal(out[start:start + s_], ref[start:start + s_])
        start += p_


def test_fp8_block_scaled_per_row_layout_in_any_expert_order(dev, variant):
    """Experts' regions in a shuffled order, stated by a per-row layout (gemm/deep_gemm_ops.py:60-100 forwards any):
    small-integer codes and power-of-two scales, so the closed form is exact; checked row by row from the layout."""
    g = torch.Generator().manual_seed(71)
    sizes, order, K, N = [100, 128, 0, 300, 28], [3, 1, 4, 0, 2], 384, 256
    lay = []
    for e in order:
        lay += [e] * sizes[e] + [-1] * ((sizes[e] + 127) // 128 * 128 - sizes[e])
    lay = torch.tensor(lay, dtype=torch.int32)
    Mp, G, kb = lay.numel(), len(sizes), K // 128
    aq = torch.randint(-3, 4, (Mp, K), generator=g).float()
    bq = torch.randint(-3, 4, (G, N, K), generator=g).float()
    pw = torch.tensor([0.25, 0.5, 1.0, 2.0])
    sa = pw[torch.randint(0, 4, (Mp, kb), generator=g)]
    sb = pw[torch.randint(0, 4, (G, N // 128, kb), generator=g)]
    out = torch.full((Mp, N), 9.0, dtype=torch.bfloat16, device=dev)
    m_grouped_fp8_nt_contiguous((aq.to(torch.float8_e4m3fn).to(dev), sa.to(dev)),
                                (bq.to(torch.float8_e4m3fn).to(dev), sb.to(dev)),
                                torch.tensor(sizes, dtype=torch.int32, device=dev), out=out, grouped_layout=lay.to(dev))
    out = out.cpu()
    valid = lay >= 0
    e = lay[valid].long()
    ad = (aq * sa.repeat_interleave(128, dim=1))[valid]                                         # dequantised rows
    wd = bq * sb.repeat_interleave(128, dim=1).repeat_interleave(128, dim=2)                    # dequantised weights
    ref = torch.einsum("rk,rnk->rn", ad, wd[e]).to(torch.bfloat16)                              # exact in fp32 here
    assert torch.equal(out[valid], ref)
    assert bool((out[~valid] == 9.0).all()), "padding rows were written"


def test_fp8_block_scaled_per_row_layout_with_experts_in_several_regions(dev, variant):
    """Two experts own two separate regions each: every row gets its own expert's weights and weight scales
    (small-integer codes and power-of-two scales: the closed form is exact)."""
    g = torch.Generator().manual_seed(72)
    sizes, K, N = [300, 128, 0, 200], 384, 256
    lay = torch.tensor([3] * 128 + [0] * 256 + [1] * 128 + [3] * 72 + [-1] * 56 + [0] * 44 + [-1] * 84, dtype=torch.int32)
    Mp, G, kb = lay.numel(), len(sizes), K // 128
    aq = torch.randint(-3, 4, (Mp, K), generator=g).float()
    bq = torch.randint(-3, 4, (G, N, K), generator=g).float()
    pw = torch.tensor([0.25, 0.5, 1.0, 2.0])
    sa = pw[torch.randint(0, 4, (Mp, kb), generator=g)]
    sb = pw[torch.randint(0, 4, (G, N // 128, kb), generator=g)]
    out = torch.full((Mp, N), 9.0, dtype=torch.bfloat16, device=dev)
    m_grouped_fp8_nt_contiguous((aq.to(torch.float8_e4m3fn).to(dev), sa.to(dev)),
                                (bq.to(torch.float8_e4m3fn).to(dev), sb.to(dev)),
                                torch.tensor(sizes, dtype=torch.int32, device=dev), out=out, grouped_layout=lay.to(dev))
    out = out.cpu()
    valid = lay >= 0
    ad = (aq * sa.repeat_interleave(128, dim=1))[valid]
    wd = bq * sb.repeat_interleave(128, dim=1).repeat_interleave(128, dim=2)
    ref = torch.einsum("rk,rnk->rn", ad, wd[lay[valid].long()]).to(torch.bfloat16)
    assert torch.equal(out[valid], ref)
    assert bool((out[~valid] == 9.0).all()), "padding rows were written"


def test_fp8_matrix_instruction_truncates_products_below_2_to_minus_13_of_the_largest(dev, variant):
    """Characterisation of gfx950's FP8 MFMA that the FP8 tolerances rest on: within one instruction the products
    are aligned to the largest one and bits below 2^-13 of it are dropped (truncated, not rounded), while the
    accumulator operand is added in full fp32.  Rows hold 448*1, -448*1 and x*1 inside one 16-deep K step, so both
    the 32x32x16 (generic) and the 16x16x128 (tuned) instruction see the three products together."""
    xs = [2.0 ** -j for j in range(0, 10)] + [1.75 * 2.0 ** -4]
    M, N, K = len(xs), 8, 128
    a, w = torch.zeros(M, K), torch.zeros(1, N, K)
    a[:, 0], a[:, 1], a[:, 2] = 448.0, -448.0, torch.tensor(xs)
    w[0, :, :3] = 1.0
    one_m, one_n = torch.ones(M, 1, device=dev), torch.ones(N, device=dev)
    out = gmm_fp8_act_per_channel_w_per_expert(a.to(dev).to(torch.float8_e4m3fn), one_m, w.to(dev).to(torch.float8_e4m3fn),
                                               one_n, torch.tensor([M], dtype=torch.int32, device=dev), torch.float16)
    got = out[:, 0].float().cpu().tolist()
    kept = [x if x >= 2.0 ** -5 else 0.0 for x in xs[:10]] + [1.5 * 2.0 ** -4]  # 448 = 1.75 * 2^8: cut-off at 2^(8-13)
    assert got == kept, got
    # the accumulator itself is full fp32: +448*448 in the first 128-deep slab, x in the second, -448*448 in the third
    K3 = 384
    a3, w3 = torch.zeros(M, K3), torch.zeros(1, N, K3)
    a3[:, 0], a3[:, 128], a3[:, 256] = 448.0, torch.tensor(xs), -448.0
    w3[0, :, 0], w3[0, :, 128], w3[0, :, 256] = 448.0, 1.0, 448.0
    out3 = gmm_fp8_act_per_channel_w_per_expert(a3.to(dev).to(torch.float8_e4m3fn), one_m, w3.to(dev).to(torch.float8_e4m3fn),
                                                one_n, torch.tensor([M], dtype=torch.int32, device=dev), torch.float16)
    # 448^2 = 200704 has an fp32 ulp of 2^-6: x survives the round trip exactly when it is a multiple of that
    want = [x if x >= 2.0 ** -6 else 0.0 for x in xs[:10]] + [1.75 * 2.0 ** -4]
    assert out3[:, 0].float().cpu().tolist() == want, out3[:, 0].tolist()
