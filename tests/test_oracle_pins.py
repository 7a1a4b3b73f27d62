"""CPU: pin the oracle (tests' checker) against the reference's known answers, library
routines and brute force, so that a wrong index / sign / dropped term in it fails here."""
import numpy as np
import pytest
import torch

from oracle import fp8_soft, gemm_ref, layout_ref, quant_ref


# ---- layout: the reference's own known answers (tests/test_layout_backend.py:23-52) ----
def test_layout_known_answers():
    assert layout_ref.round_up([0, 1, 127, 128, 129], 128) == [0, 128, 128, 128, 256]
    assert layout_ref.group_starts([3, 5, 0, 7], padded=False, block_m=4) == [0, 3, 8, 8]
    assert layout_ref.group_starts([3, 5, 0, 7], padded=True, block_m=4) == [0, 4, 12, 12]
    lay = layout_ref.grouped_layout([3, 5, 0, 7], block_m=4)
    assert lay["sizes"] == [3, 5, 0, 7] and lay["padded_sizes"] == [4, 8, 0, 8]
    assert lay["starts"] == [0, 4, 12, 12] and lay["total_m"] == 15 and lay["total_padded_m"] == 20
    assert layout_ref.deep_gemm_grouped_layout([3, 5], 4) == [0, 0, 0, -1, 1, 1, 1, 1, 1, -1, -1, -1]
    assert layout_ref.deep_gemm_psum_layout([3, 5], 4) == [3, 9]
    layout_ref.validate_total_m([2, 3, 4], 9)
    with pytest.raises(ValueError, match=r"sum\(size_per_group\)"):
        layout_ref.validate_total_m([2, 3, 4], 10)


def test_tile_rows_cover_every_row_once():
    sizes = [3, 0, 130, 128, 1, 257]
    seen = []
    for g, row0, rows in layout_ref.tile_rows(sizes, 128):
        assert 0 < rows <= 128
        seen += [(g, r) for r in range(row0, row0 + rows)]
    want, start = [], 0
    for g, s in enumerate(sizes):
        want += [(g, r) for r in range(start, start + s)]
        start += s
    assert seen == want


# ---- fp8 encoders: exhaustive against torch's CPU cast, and closed-form round trips ----
def _all_bf16_as_f32():
    return fp8_soft.bf16_bits_to_f32(np.arange(65536, dtype=np.uint16))


@pytest.mark.parametrize("fmt,tdt,enc", [("e4m3fn", torch.float8_e4m3fn, fp8_soft.encode_e4m3fn),
                                         ("e5m2", torch.float8_e5m2, fp8_soft.encode_e5m2)])
def test_fp8_encode_matches_torch_cast(fmt, tdt, enc):
    rng = np.random.default_rng(0)
    x = np.concatenate([_all_bf16_as_f32(),
                        (rng.standard_normal(200000) * np.exp(rng.uniform(-25, 12, 200000))).astype(np.float32),
                        np.array([448.0, 464.0, 463.99, 465.0, 57344.0, 61440.0, 61439.0, 2.0 ** -9, 2.0 ** -10,
                                  1.5 * 2.0 ** -10, 2.0 ** -16, 2.0 ** -17, 0.0, -0.0], dtype=np.float32)])
    with np.errstate(all="ignore"):
        mine = enc(x)
    ref = torch.from_numpy(x).to(tdt).view(torch.uint8).numpy()
    nan_mine = np.isnan(quant_ref.dequant(mine, fmt))
    nan_ref = np.isnan(quant_ref.dequant(ref, fmt))
    assert np.array_equal(nan_mine, nan_ref)
    assert np.array_equal(mine[~nan_ref], ref[~nan_ref])


def test_fp8_decode_encode_roundtrip_and_spacing():
    codes = np.arange(256, dtype=np.uint8)
    v = fp8_soft.decode_e4m3fn(codes)
    ok = ~np.isnan(v)
    assert np.array_equal(fp8_soft.encode_e4m3fn(v[ok]), codes[ok])
    assert v[0x7E] == 448.0 and v[0x01] == 2.0 ** -9 and v[0x08] == 2.0 ** -6 and np.isnan(v[0x7F])
    v5 = fp8_soft.decode_e5m2(codes)
    ok5 = np.isfinite(v5)
    assert np.array_equal(fp8_soft.encode_e5m2(v5[ok5]), codes[ok5])
    assert v5[0x7B] == 57344.0 and v5[0x01] == 2.0 ** -16 and np.isinf(v5[0x7C])
    # ties go to even: halfway between codes 0x40 (2.0) and 0x41 (2.25) -> 0x40; next tie -> 0x42
    assert fp8_soft.encode_e4m3fn(np.array([2.125, 2.375], np.float32)).tolist() == [0x40, 0x42]


def test_bf16_rounding_matches_torch():
    rng = np.random.default_rng(1)
    x = (rng.standard_normal(100000) * np.exp(rng.uniform(-30, 30, 100000))).astype(np.float32)
    ref = torch.from_numpy(x).to(torch.bfloat16).view(torch.int16).numpy().view(np.uint16)
    assert np.array_equal(fp8_soft.f32_to_bf16_bits(x), ref)


# ---- quantizers: brute force per element on tiny inputs + invariants ----
def _bf16_randn(shape, seed, scale=1.0):
    g = torch.Generator().manual_seed(seed)
    return (torch.randn(shape, generator=g) * scale).to(torch.bfloat16).float().numpy()


def test_trans_quant_bruteforce_and_invariants():
    sizes = [5, 0, 130, 128]
    M, N = sum(sizes), 256
    x = _bf16_randn((M, N), 3)
    codes, scales, padded = quant_ref.trans_per_block_quant_expand_128x(x, sizes)
    ME = M + 128 * len(sizes) - M % 128
    assert codes.shape == (N, ME) and scales.shape == (N // 128, ME // 128)
    assert padded.tolist() == [128, 0, 256, 128]
    # brute force: element by element with Python scalars
    src, dst = 0, 0
    for s, p in zip(sizes, padded.tolist()):
        for r in range(p):
            for n in range(0, N, 37):
                blk_r0 = src + (r // 128) * 128
                blk = x[blk_r0:min(blk_r0 + 128, src + s), (n // 128) * 128:(n // 128 + 1) * 128]
                amax = np.float32(np.abs(blk).max()) if blk.size else np.float32(0)
                sc = np.float32(max(np.float32(amax / np.float32(448.0)), np.float32(1e-12)))
                assert scales[n // 128, (dst + r) // 128] == sc
                val = x[src + r, n] if r < s else np.float32(0)
                q = np.float32(min(max(np.float32(val / sc), -448.0), 448.0))
                want = torch.tensor([q]).to(torch.float8_e4m3fn).view(torch.uint8).item()
                assert codes[n, dst + r] == want
        src += s
        dst += p
    # tail beyond the padded groups is zero
    assert not codes[:, dst:].any() and not scales[:, dst // 128:].any()
    # dequantised codes sit within half an e4m3 ulp (2^-4 relative of the block max) of x
    deq = quant_ref.dequant(codes[:, :128], "e4m3fn") * scales[:, 0:1].repeat(128, axis=0)
    err = np.abs(deq[:, :5].T - x[:5])
    assert err.max() <= np.abs(x[:5]).max() * 2.0 ** -4


def test_trans_quant_matches_reference_torch_oracle_on_full_blocks():
    """The reference's own torch oracle (quant/...:222-273) restated inline with torch ops."""
    sizes = [128, 256]
    M, N = 384, 128
    x = _bf16_randn((M, N), 4)
    codes, scales, _ = quant_ref.trans_per_block_quant_expand_128x(x, sizes)
    xt = torch.from_numpy(x).to(torch.bfloat16)
    outs, scs = [], []
    for part in torch.split(xt, sizes, dim=0):
        t = part.T
        d, s = t.shape
        blocks = t.reshape(d // 128, 128, s // 128, 128).transpose(1, 2).reshape(-1, 128 * 128)
        sc = blocks.abs().amax(-1, True).float() / 448.0
        q = (blocks / sc).clamp(-448, 448).to(torch.float8_e4m3fn)
        outs.append(q.reshape(d // 128, s // 128, 128, 128).transpose(1, 2).reshape(d, s))
        scs.append(sc.reshape(d // 128, s // 128))
    ref_codes = torch.cat(outs, -1).view(torch.uint8).numpy()
    ref_scales = torch.cat(scs, -1).numpy()
    assert np.array_equal(codes[:, :M], ref_codes)
    assert np.array_equal(scales[:, :M // 128], ref_scales)


def test_cast_recipes_match_torch_expressions():
    x = _bf16_randn((16, 256), 5, scale=3.0)
    xt = torch.from_numpy(x).to(torch.bfloat16)
    codes, scales = quant_ref.per_token_cast_to_fp8(x)
    v = xt.view(16, -1, 128)
    amax = v.abs().float().amax(dim=2).view(16, -1).clamp(1e-4)
    ref = (v * (448.0 / amax.unsqueeze(2))).to(torch.float8_e4m3fn).view(16, 256).view(torch.uint8).numpy()
    assert np.array_equal(codes, ref) and np.array_equal(scales, (amax / 448.0).numpy())
    xb = _bf16_randn((130, 200), 6)
    cb, sb = quant_ref.per_block_cast_to_fp8(xb)
    assert cb.shape == (130, 200) and sb.shape == (2, 2)
    blk = xb[128:, 128:]
    assert sb[1, 1] == np.float32(np.float32(np.abs(blk).max()) / np.float32(448.0))
    # a block of zeros hits the 1e-4 clamp
    cz, sz = quant_ref.per_block_cast_to_fp8(np.zeros((128, 128), np.float32))
    assert sz[0, 0] == np.float32(np.float32(1e-4) / np.float32(448.0)) and not cz.any()


@pytest.mark.parametrize("shape", [(130, 200), (256, 384), (300, 520), (128, 8192)])
def test_per_block_cast_matches_the_torch_expression_codes_and_scales(shape):
    """quant_ref.per_block_cast_to_fp8 against the torch expression of the reference's per_block_cast_to_fp8
    (gemm/FP8/m_grouped_gemm_channel_expert.py:237-245), evaluated by torch on the CPU: every code and every scale.
    A division in place of torch's reciprocal-then-multiply for `448.0 / amax` changes codes and fails here."""
    m, n = shape
    x = _bf16_randn(shape, 60 + m, scale=2.0)
    x[5, 7] = 0.0
    if m > 256:
        x[256:, 384:] *= 1e-3   # a ragged corner block of small values
    xt = torch.from_numpy(x).to(torch.bfloat16)
    x = xt.float().numpy()
    codes, scales = quant_ref.per_block_cast_to_fp8(x)
    mp, np_ = -(-m // 128) * 128, -(-n // 128) * 128
    x_padded = torch.zeros((mp, np_), dtype=xt.dtype)
    x_padded[:m, :n] = xt
    x_view = x_padded.view(-1, 128, np_ // 128, 128)
    x_amax = x_view.abs().float().amax(dim=(1, 3), keepdim=True).clamp(1e-4)
    x_scaled = (x_view * (448.0 / x_amax)).to(torch.float8_e4m3fn)
    ref_codes = x_scaled.view_as(x_padded)[:m, :n].contiguous().view(torch.uint8).numpy()
    ref_scales = (x_amax / 448.0).view(x_view.size(0), x_view.size(2)).numpy()
    assert codes.shape == (m, n) and scales.shape == ref_scales.shape
    assert np.array_equal(codes, ref_codes)
    assert np.array_equal(scales.view(np.uint32), ref_scales.view(np.uint32))
    if shape != (128, 8192):
        return
    # the pin bites: with 64 blocks, one IEEE division instead of reciprocal * 448 changes hundreds of codes
    amax = np.maximum(np.abs(np.pad(x, ((0, mp - m), (0, np_ - n)))).reshape(mp // 128, 128, np_ // 128, 128).max(axis=(1, 3), keepdims=True), np.float32(1e-4)).astype(np.float32)
    wrong = (np.pad(x, ((0, mp - m), (0, np_ - n))).reshape(mp // 128, 128, np_ // 128, 128) * (np.float32(448.0) / amax)).astype(np.float32)
    from oracle import fp8_soft
    assert not np.array_equal(fp8_soft.encode_e4m3fn(wrong).reshape(mp, np_)[:m, :n], ref_codes)


def test_row_and_expert_cast_recipes_match_torch_expressions():
    """per_row_cast_to_fp8 / per_expert_cast_to_fp8 against the torch expressions of the reference's
    per_channel_cast_to_fp8 and per_expert_cast_to_fp8 (gemm/FP8/m_grouped_gemm_channel_expert.py:224-234, :247-261):
    torch's own fp8 cast and its `fmax / amax` (reciprocal then multiply) stand against the numpy encoder."""
    for fmt, tdt in (("e4m3fn", torch.float8_e4m3fn), ("e5m2", torch.float8_e5m2)):
        fmax = torch.finfo(tdt).max
        x = _bf16_randn((12, 256), 21, scale=2.5)
        x[3] = 0.0                       # a whole row at the 1e-4 clamp
        x[4] *= 1e-3
        xt = torch.from_numpy(x).to(torch.bfloat16)
        x = xt.float().numpy()           # the oracle takes fp32 arrays holding bf16 values
        codes, scales = quant_ref.per_row_cast_to_fp8(x, fmt)
        v = xt.view(12, -1, 256)
        amax = v.abs().float().amax(dim=2).view(12, -1).clamp(1e-4)
        ref = (v * (fmax / amax.unsqueeze(2))).to(tdt).view(12, 256).view(torch.uint8).numpy()
        assert codes.shape == (12, 256) and scales.shape == (12, 1)
        assert np.array_equal(codes, ref) and np.array_equal(scales, (amax / fmax).numpy())
        # the scale is per ROW: scaling one row by 4 changes that row's scale only
        x2 = x.copy()
        x2[5] *= 4.0
        _, s2 = quant_ref.per_row_cast_to_fp8(x2, fmt)
        assert s2[5, 0] == np.float32(4.0) * scales[5, 0] and np.array_equal(np.delete(s2, 5, 0), np.delete(scales, 5, 0))

        w = _bf16_randn((3, 24, 40), 22, scale=0.3)
        w[1] *= 8.0
        wt = torch.from_numpy(w).to(torch.bfloat16)
        w = wt.float().numpy()
        cw, sw = quant_ref.per_expert_cast_to_fp8(w, fmt)
        wv = wt.view(3, 24, 1, 40)
        wamax = wv.abs().float().amax(dim=(1, 3), keepdim=True).clamp(1e-4)
        wref = (wv * (fmax / wamax)).to(tdt).view(3, 24, 40).view(torch.uint8).numpy()
        assert cw.shape == (3, 24, 40) and sw.shape == (3, 1)
        assert np.array_equal(cw, wref) and np.array_equal(sw, (wamax / fmax).view(3, 1).numpy())
        assert sw[1, 0] > 4 * sw[0, 0]   # one scale per EXPERT matrix, not a global one


def test_fp8_channel_reference_pins():
    """fp8_channel_reference (gemm/FP8/m_grouped_gemm_channel_expert.py:119-136): unit scales reduce it to gmm;
    with power-of-two scales folded into integer operands every product is exact, so it must EQUAL the plain
    per-group matmul of the pre-scaled operands; a brute-force triple loop on a tiny case; scales chosen so that
    reading b_scale as [N, G] instead of [G, N], or a_scale by group instead of by row, changes the result."""
    g = torch.Generator().manual_seed(31)
    sizes = [5, 0, 7]
    M, K, G, N = 12, 16, 3, 4
    aq = torch.randint(-6, 7, (M, K), generator=g).float()
    bq = torch.randint(-6, 7, (G, N, K), generator=g).float()
    ones_a, ones_b = torch.ones(M, 1), torch.ones(G * N)
    assert torch.equal(gemm_ref.fp8_channel_reference(aq, ones_a, bq, ones_b, sizes), gemm_ref.gmm(aq, bq, sizes, trans_b=True))
    sa = 2.0 ** torch.randint(-3, 4, (M, 1), generator=g).float()          # distinct per row
    sb = 2.0 ** torch.arange(G * N).float().remainder(7).sub(3)            # flattened [G*N], g-major: index g*N + n
    out = gemm_ref.fp8_channel_reference(aq, sa, bq, sb, sizes)
    folded = gemm_ref.gmm(aq * sa, bq * sb.view(G, N, 1), sizes, trans_b=True)
    assert torch.equal(out, folded)
    wrong = gemm_ref.gmm(aq * sa, bq * sb.view(N, G).t().reshape(G, N, 1), sizes, trans_b=True)
    assert not torch.equal(out, wrong)                                      # the test can tell [G,N] from [N,G]
    starts = [0, 5, 5]
    for gi, (st, sz) in enumerate(zip(starts, sizes)):
        for r in range(st, st + sz):
            for n in range(N):
                acc = sum(float(aq[r, k]) * float(bq[gi, n, k]) for k in range(K))
                assert float(out[r, n]) == acc * float(sa[r, 0]) * float(sb[gi * N + n])
    assert gemm_ref.fp8_channel_reference(aq, sa.view(-1), bq, sb, sizes).equal(out)   # [M] and [M,1] scales alike


def test_fp8_k_grouped_channel_reference_pins():
    """fp8_k_grouped_channel_reference (gemm/FP8/k_grouped_gemm_channel_expert.py:104-140: scale element (m, g) at
    g*M + m, accumulate over the group's token segment, multiply by a_s * b_s^T once at the end)."""
    g = torch.Generator().manual_seed(32)
    tokens = [4, 0, 6]
    M, N, G = 3, 5, 3
    Kt = sum(tokens)
    xq = torch.randint(-6, 7, (M, Kt), generator=g).float()
    yq = torch.randint(-6, 7, (N, Kt), generator=g).float()
    ones = gemm_ref.fp8_k_grouped_channel_reference(xq, torch.ones(M, G), yq, torch.ones(N, G), tokens)
    assert ones.shape == (G, M, N)
    assert torch.equal(ones[0], xq[:, :4] @ yq[:, :4].t()) and torch.count_nonzero(ones[1]) == 0
    assert torch.equal(ones.sum(0), xq @ yq.t())                            # segments partition the token axis
    assert torch.equal(ones, gemm_ref.gmm_dw(xq.t().contiguous(), yq.t().contiguous(), tokens))  # == bf16 K-grouped on A^T
    xs = 2.0 ** torch.randint(-3, 4, (M, G), generator=g).float()
    ys = 2.0 ** (torch.arange(N * G).float().remainder(5).sub(2)).view(N, G)
    out = gemm_ref.fp8_k_grouped_channel_reference(xq, xs, yq, ys, tokens)
    start = 0
    for gi, t in enumerate(tokens):
        seg = slice(start, start + t)
        folded = (xq[:, seg] * xs[:, gi:gi + 1]) @ (yq[:, seg] * ys[:, gi:gi + 1]).t()
        assert torch.equal(out[gi], folded)
        for m in range(M):
            for n in range(N):
                acc = sum(float(xq[m, k]) * float(yq[n, k]) for k in range(start, start + t))
                assert float(out[gi, m, n]) == acc * float(xs[m, gi]) * float(ys[n, gi])
        start += t
    # the column-major storage the kernel reads (element (m, g) at g*M + m) is what xs[:, g] addresses
    flat = xs.t().contiguous().view(-1)
    assert all(float(flat[gi * M + m]) == float(xs[m, gi]) for gi in range(G) for m in range(M))
    swapped = gemm_ref.fp8_k_grouped_channel_reference(xq, xs.t().reshape(M, G), yq, ys, tokens)
    assert not torch.equal(swapped, out)


# ---- GEMM references: reduce to library routines ----
def test_gmm_reduces_to_matmul_and_bmm():
    g = torch.Generator().manual_seed(7)
    a = torch.randn(96, 32, generator=g)
    b = torch.randn(3, 48, 32, generator=g)
    assert torch.equal(gemm_ref.gmm(a, b[:1], [96], trans_b=True), a @ b[0].t())
    out = gemm_ref.gmm(a, b, [32, 32, 32], trans_b=True)
    assert torch.allclose(out.view(3, 32, 48), torch.bmm(a.view(3, 32, 32), b.transpose(1, 2)), atol=1e-5)
    bn = b.transpose(1, 2).contiguous()
    assert torch.allclose(gemm_ref.gmm(a, bn, [10, 0, 86], trans_b=False), gemm_ref.gmm(a, b, [10, 0, 86], trans_b=True), atol=1e-5)
    # permuting experts permutes output blocks
    perm = gemm_ref.gmm(torch.cat([a[64:], a[:64]]), b[[2, 0, 1]], [32, 32, 32], trans_b=True)
    assert torch.allclose(perm[:32], out[64:], atol=1e-6)


def test_gmm_dw_and_masked_special_cases():
    g = torch.Generator().manual_seed(8)
    a = torch.randn(40, 16, generator=g)
    b = torch.randn(40, 24, generator=g)
    assert torch.allclose(gemm_ref.gmm_dw(a, b, [40])[0], a.t() @ b, atol=1e-5)
    out = gemm_ref.gmm_dw(a, b, [10, 0, 30])
    assert torch.count_nonzero(out[1]) == 0
    assert torch.allclose(out[0] + out[2], a.t() @ b, atol=1e-4)
    lhs = torch.randn(4 * 8, 16, generator=g)
    rhs = torch.randn(4, 12, 16, generator=g)
    outs = gemm_ref.masked_gmm(lhs, rhs, [8, 8, 8, 8], 8)
    assert torch.allclose(torch.stack(outs), torch.bmm(lhs.view(4, 8, 16), rhs.transpose(1, 2)), atol=1e-5)
    assert gemm_ref.masked_gmm(lhs, rhs, [0, 3, 8, 1], 8)[1].shape == (3, 12)


def test_block_scaled_reference_exact_on_power_of_two_scales():
    g = torch.Generator().manual_seed(9)
    sizes = [100, 128]
    Mp, K, N = 256, 256, 128
    aq = torch.randint(-4, 5, (Mp, K), generator=g).float()
    bq = torch.randint(-4, 5, (2, N, K), generator=g).float()
    sa = torch.tensor([0.5, 2.0]).repeat(Mp, 1)
    sb = torch.tensor([4.0, 0.25]).view(1, 1, 2).repeat(2, 1, 1)
    out = gemm_ref.fp8_block_scaled_reference(aq, sa, bq, sb, sizes)
    want0 = 2.0 * (aq[:100, :128] @ bq[0][:, :128].t()) + 0.5 * (aq[:100, 128:] @ bq[0][:, 128:].t())
    assert torch.equal(out[:100], want0)
    assert torch.count_nonzero(out[100:128]) == 0
    assert torch.equal(out[128:], 2.0 * (aq[128:, :128] @ bq[1][:, :128].t()) + 0.5 * (aq[128:, 128:] @ bq[1][:, 128:].t()))


def test_metrics():
    x = torch.tensor([1.0, -2.0, 4.0])
    assert gemm_ref.rdiff(x, x) == 0.0 and gemm_ref.cos_diff(x, x) == pytest.approx(0.0, abs=1e-15)
    assert gemm_ref.rdiff(x, x + torch.tensor([0.0, 0.0, 0.4])) == pytest.approx(0.4 / 4.4)
    assert torch.allclose(gemm_ref.row_max_normalization(torch.tensor([[1.0, -4.0]])), torch.tensor([[0.25, -1.0]]))


# ---------------------------------------------------------------------------------------------------------------
# MoE permute / unpermute oracle: brute force on tiny inputs
# ---------------------------------------------------------------------------------------------------------------
def test_permute_oracle_against_brute_force():
    import torch
    from oracle import permute_ref
    indices = torch.tensor([[2, 0], [1, 2], [-1, 0], [2, 1]], dtype=torch.int32)  # 4 tokens, top-2, one dropped
    x = torch.arange(4 * 3, dtype=torch.float32).reshape(4, 3)
    # kept assignments in (expert, flat position) order: written out by hand
    order = [(0, 1), (2, 1), (1, 0), (3, 1), (0, 0), (1, 1), (3, 0)]  # (token, k) for experts 0,0,1,1,2,2,2
    m = permute_ref.row_id_map(indices)
    for pos, (t, k) in enumerate(order):
        assert int(m[k * 4 + t]) == pos
    assert int(m[0 * 4 + 2]) == -1  # the dropped assignment (token 2, k 0)
    m5 = permute_ref.row_id_map(indices, 5)
    assert [int(v) for v in m5] == [v if 0 <= v < 5 else -1 for v in m.tolist()]
    assert permute_ref.tokens_per_expert(indices, 4).tolist() == [2, 2, 3, 0]
    # permute / unpermute without drops: a round trip with unit weights multiplies by topk
    ind2 = torch.tensor([[1, 0], [0, 1], [1, 0]], dtype=torch.int32)
    xs = torch.arange(3 * 2, dtype=torch.float32).reshape(3, 2) + 1
    p, so = permute_ref.permute(xs, ind2)
    assert p.tolist() == [xs[0].tolist(), xs[1].tolist(), xs[2].tolist(), xs[0].tolist(), xs[1].tolist(), xs[2].tolist()]
    probs = torch.tensor([[0.25, 0.75], [0.5, 0.5], [1.0, 0.0]])
    u = permute_ref.unpermute(p, so, probs)
    assert torch.allclose(u, xs * probs.sum(1, keepdim=True))
    u2 = permute_ref.unpermute(p * torch.tensor([[1.], [1.], [1.], [2.], [2.], [2.]]), so, probs)
    # expert-1 copies were doubled: token 0 used expert 1 at k=0 (weight .25), token 1 at k=1 (.5), token 2 at k=0 (1.0)
    assert torch.allclose(u2, xs * torch.tensor([[0.25 * 2 + 0.75], [0.5 + 0.5 * 2], [2.0]]))
