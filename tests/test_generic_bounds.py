"""Host-side bounds walk of the shape-agnostic kernel (no GPU): for every GEMM entry point, at group counts up to
the 1024 its table holds, every tile's accesses to A, B, C and the scale arrays stay inside the tensors.  The walk
runs the kernel's own scheduler and address functions (csrc/sched.hpp, csrc/generic_addr.hpp) through
tgg_debug_generic_extents.  The reference relies on Triton's masked loads / TMA bounds for the same guarantee
(gemm/BF16/m_grouped_gemm.py:83-116, gemm/FP8/m_grouped_gemm_channel_expert.py:119-136,
gemm/FP8/k_grouped_gemm_channel_expert.py:104-140)."""
import numpy as np
import pytest

from triton_grouped_gemm_amd import _native

A, B, C, SCALE_M, SCALE_N, SA, SB = range(7)
UNTOUCHED = (np.iinfo(np.int64).max, -1)


def extents(kind, sizes, G, M, aux, N, K, row_start=None):
    lib = _native.load()
    s = np.asarray(sizes, dtype=np.int64)
    rs = None if row_start is None else np.asarray(row_start, dtype=np.int32)
    out = np.zeros((7, 2), dtype=np.int64)
    rc = lib.tgg_debug_generic_extents(kind, s.ctypes.data, None if rs is None else rs.ctypes.data, G, M, aux, N, K,
                                       out.ctypes.data)
    assert rc == 0, _native.last_error()
    return [tuple(int(v) for v in row) for row in out]


def inside(ext, n_elements):
    return ext == UNTOUCHED or (0 <= ext[0] <= ext[1] < n_elements)


def sizes_for(G, seed, top=300):
    rng = np.random.default_rng(seed)
    s = rng.choice([0, 0, 3, 16, 40, 128, 129, top], size=G)
    s[min(511, G - 1)], s[min(512, G - 1)] = 77, 130
    return [int(x) for x in s]


GROUPS = [4, 256, 257, 512, 513, 600, 1024]
SHAPES = [(264, 136), (128, 256), (520, 72)]  # (N, K): column and K tails, exact tiles, several column tiles


@pytest.mark.parametrize("G", GROUPS)
@pytest.mark.parametrize("N,K", SHAPES)
def test_m_grouped_both_layouts(G, N, K):
    sizes = sizes_for(G, G)
    M = sum(sizes)
    for kind in (0, 1):
        e = extents(kind, sizes, G, M, 0, N, K)
        assert e[A] == (0, M * K - 1) and e[C] == (0, M * N - 1)
        assert inside(e[B], G * N * K)
        assert e[SCALE_M] == e[SCALE_N] == e[SA] == e[SB] == UNTOUCHED


@pytest.mark.parametrize("G", GROUPS)
@pytest.mark.parametrize("N,K", SHAPES)
def test_masked(G, N, K):
    m_stride = 256
    sizes = sizes_for(G, G + 1, m_stride)
    e = extents(2, sizes, G, G * m_stride, m_stride, N, K)
    assert inside(e[A], G * m_stride * K) and inside(e[B], G * N * K) and inside(e[C], G * m_stride * N)
    last = max(g for g in range(G) if sizes[g] > 0)
    assert e[C][1] == ((last * m_stride + sizes[last] - 1) * N + N - 1)  # the last valid row's last column, nothing beyond


@pytest.mark.parametrize("G", GROUPS)
@pytest.mark.parametrize("N,K", SHAPES)
def test_padded_and_placed(G, N, K):
    sizes = sizes_for(G, G + 2)
    padded = [-(-s // 128) * 128 for s in sizes]
    M = sum(padded)
    e = extents(3, sizes, G, M, 128, N, K)
    assert inside(e[A], M * K) and inside(e[B], G * N * K) and inside(e[C], M * N)
    # placed: the same regions in reverse order
    starts, at = [0] * G, 0
    for g in reversed(range(G)):
        starts[g] = at
        at += padded[g]
    e = extents(4, sizes, G, M, 0, N, K, row_start=starts)
    assert inside(e[A], M * K) and inside(e[B], G * N * K) and inside(e[C], M * N)
    assert e[A][0] == starts[max(g for g in range(G) if sizes[g] > 0)] * K  # the group placed first


@pytest.mark.parametrize("G", GROUPS)
@pytest.mark.parametrize("N", [264, 128, 520])
def test_k_grouped_16bit(G, N):
    tokens = sizes_for(G, G + 3)
    ktot, mdim = sum(tokens), 136
    e = extents(5, tokens, G, mdim, ktot, N, 0)
    assert e[A] == (0, ktot * mdim - 1) and e[B] == (0, ktot * N - 1)
    assert e[C] == (0, G * mdim * N - 1)  # every group's output is written, empty groups included


@pytest.mark.parametrize("G", GROUPS)
@pytest.mark.parametrize("N,K", [(264, 144), (128, 256), (520, 80)])
def test_fp8_channel_m_grouped(G, N, K):
    sizes = sizes_for(G, G + 4)
    M = sum(sizes)
    e = extents(6, sizes, G, M, 0, N, K)
    assert e[A] == (0, M * K - 1) and e[C] == (0, M * N - 1) and inside(e[B], G * N * K)
    assert e[SCALE_M] == (0, M - 1) and inside(e[SCALE_N], G * N)


@pytest.mark.parametrize("G", GROUPS)
@pytest.mark.parametrize("N", [264, 128])
def test_fp8_channel_k_grouped(G, N):
    tokens = [16 * (s % 13) for s in sizes_for(G, G + 5)]
    ktot, M = sum(tokens), 136
    e = extents(7, tokens, G, M, ktot, N, 0)
    assert inside(e[A], M * ktot) and inside(e[B], N * ktot)
    assert e[C] == (0, G * M * N - 1)
    assert e[SCALE_M] == (0, G * M - 1) and e[SCALE_N] == (0, G * N - 1)


@pytest.mark.parametrize("G", GROUPS)
@pytest.mark.parametrize("N,K", [(264, 256), (128, 144), (520, 4096)])
def test_fp8_block_scaled(G, N, K):
    sizes = sizes_for(G, G + 6)
    padded = [-(-s // 128) * 128 for s in sizes]
    M, kb, nb = sum(padded), -(-K // 128), -(-N // 128)
    for kind in (8, 9):
        e = extents(kind, sizes, G, M, 128, N, K)
        assert inside(e[A], M * K) and inside(e[B], G * N * K) and inside(e[C], M * N)
        assert inside(e[SA], M * kb) and inside(e[SB], G * nb * kb)
        assert e[SB][0] == 0 or sizes[0] == 0
    starts, at = [0] * G, 0
    for g in reversed(range(G)):
        starts[g] = at
        at += padded[g]
    e = extents(10, sizes, G, M, 128, N, K, row_start=starts)
    assert inside(e[A], M * K) and inside(e[C], M * N) and inside(e[SA], M * kb) and inside(e[SB], G * nb * kb)
