"""The persistent kernels' tile scheduler, run on the host through the library's test hook (no GPU):
every output tile of the grouped tile space is visited exactly once, whatever the group sizes, grid size,
walk and chunking.  This is the invariant the reference's tile enumeration provides
(gemm/BF16/m_grouped_gemm_TMA.py:55-71 grouped_launch, :297-326 m_indices_pad); results do not depend on
the order, only on the cover."""
import ctypes

import numpy as np
import pytest

from triton_grouped_gemm_amd import _native

MG, MG_PAD, MASKED, KG_COUNT = 0, 1, 2, 4


def tile_order(sizes, mode, m_total, aux, N, tile, grid, split, n_chunk=0):
    lib = _native.load()
    _native.set_option("n_chunk", n_chunk)
    try:
        s = np.asarray(sizes, dtype=np.int64)
        cap = 1 << 16
        out = np.zeros((cap, 6), dtype=np.int64)
        n = ctypes.c_int64(0)
        rc = lib.tgg_debug_tile_order(s.ctypes.data, len(s), mode, m_total, aux, N, tile, grid, split,
                                      out.ctypes.data, cap, ctypes.byref(n))
        assert rc == 0, lib.tgg_last_error().decode()
        return out[:n.value], n.value
    finally:
        _native.set_option("n_chunk", 0)


def expected_m_grouped_tiles(sizes, starts, tile, N, m_total):
    exp = set()
    for g, (sz, st) in enumerate(zip(sizes, starts)):
        sz = max(0, min(sz, m_total - st))
        for mt in range(-(-sz // tile)):
            rows = min(tile, sz - mt * tile)
            for nt in range(-(-N // tile)):
                exp.add((g, st + mt * tile, rows, nt * tile))
    return exp


@pytest.mark.parametrize("tile", [256, 128])
@pytest.mark.parametrize("split", [0, 1])
@pytest.mark.parametrize("grid", [256, 64, 7, 1])
@pytest.mark.parametrize("n_chunk", [0, 1, 3])
@pytest.mark.parametrize("sizes,N", [
    ([64, 128, 32, 96], 512),
    ([1, 0, 127, 129, 256, 3, 0, 300], 136),
    ([300, 0, 417], 2600),
    ([5120] * 16, 1536),
    ([0, 0, 0], 256),
])
def test_m_grouped_cover(tile, split, grid, n_chunk, sizes, N):
    starts = np.concatenate([[0], np.cumsum(sizes)[:-1]]).tolist()
    rows, n = tile_order(sizes, MG, sum(sizes), 0, N, tile, grid, split, n_chunk)
    exp = expected_m_grouped_tiles(sizes, starts, tile, N, sum(sizes))
    got = [tuple(r[2:6]) for r in rows.tolist()]
    assert n == len(exp) == len(got)
    assert set(got) == exp and len(set(got)) == len(got)
    # positions inside a workgroup's walk are 0, 1, 2, ... and workgroup ids stay below the grid
    for b in range(grid):
        pos = rows[rows[:, 0] == b][:, 1]
        assert pos.tolist() == list(range(len(pos)))
    assert rows[:, 0].max(initial=0) < grid


def test_padded_and_masked_starts():
    sizes = [100, 0, 130, 128]
    rows, n = tile_order(sizes, MG_PAD, 128 + 0 + 256 + 128, 128, 256, 256, 256, 1)
    exp = expected_m_grouped_tiles(sizes, [0, 128, 128, 384], 256, 256, 512)
    assert {tuple(r[2:6]) for r in rows.tolist()} == exp and n == len(exp)
    masked = [512, 0, 77, 300]
    rows, n = tile_order(masked, MASKED, 4 * 512, 512, 4096, 256, 256, 1)
    exp = expected_m_grouped_tiles(masked, [0, 512, 1024, 1536], 256, 4096, 2048)
    assert {tuple(r[2:6]) for r in rows.tolist()} == exp and n == len(exp)


def test_rows_past_the_end_of_a_are_clipped():
    """sizes that sum past m_total: the last group is cut, later ones vanish (never touch rows outside A)."""
    rows, n = tile_order([200, 200, 200], MG, 300, 0, 256, 256, 256, 1)
    assert {tuple(r[2:6]) for r in rows.tolist()} == {(0, 0, 200, 0), (1, 200, 100, 0)}


@pytest.mark.parametrize("tile", [256, 128])
@pytest.mark.parametrize("grid", [256, 24])
def test_k_grouped_cover(tile, grid):
    """K-grouped: every (group, row tile, column tile) of the [G, Mdim, N] output once, empty groups included
    (their tiles must be written with zeros)."""
    sizes, mdim, N = [40, 0, 200, 64], 520, 2600
    rows, n = tile_order(sizes, KG_COUNT, mdim, sum(sizes), N, tile, grid, 0)
    exp = {(g, mt * tile, min(tile, mdim - mt * tile), nt * tile)
           for g in range(len(sizes)) for mt in range(-(-mdim // tile)) for nt in range(-(-N // tile))}
    got = [tuple(r[2:6]) for r in rows.tolist()]
    assert n == len(exp) and set(got) == exp and len(set(got)) == len(got)


def test_k_grouped_tile_space_runs_over_groups_by_decreasing_size():
    """A K-grouped tile costs what its group has tokens and every group has equally many tiles, so the tile space
    lists the groups by decreasing token count (ties by index): with a fixed stride every workgroup then sees a
    fair mix, and the launch ends on its cheapest tiles."""
    sizes, mdim, N = [40, 0, 200, 64, 200, 8, 0, 512], 256, 512
    rows, n = tile_order(sizes, KG_COUNT, mdim, sum(sizes), N, 256, 1, 0)  # one workgroup: it walks the ids in order
    per_group = 2
    assert n == len(sizes) * per_group
    walked = [int(r[2]) for r in rows.tolist()]
    want = sorted(range(len(sizes)), key=lambda g: (-sizes[g], g))
    assert walked == [g for g in want for _ in range(per_group)]
    # the loads of 4 workgroups that take every fourth tile: within one largest group of each other
    sizes = [(37 * g * g + 11 * g) % 2000 for g in range(64)]
    rows, n = tile_order(sizes, KG_COUNT, 256, sum(sizes), 768, 256, 4, 0)  # 3 tiles per group, grid of 4
    load = [0] * 4
    for b, _, g, *_ in rows.tolist():
        load[int(b)] += sizes[int(g)]
    assert max(load) - min(load) <= max(sizes)


def test_runs_of_an_xcd_are_near_square():
    """With 256 workgroups dealt round robin to 8 XCDs, the 32 tiles an XCD works on at the same time should
    span few distinct row panels and column panels (this is what keeps operand re-reads inside one L2)."""
    sizes, N = [5120] * 128, 4096  # 16 column tiles -> chunks of 8
    rows, _ = tile_order(sizes, MG, sum(sizes), 0, N, 256, 256, 1)
    first = rows[rows[:, 1] == 0]
    for x in range(8):
        mine = first[first[:, 0] % 8 == x]
        assert len(mine) == 32
        assert len(set(mine[:, 3].tolist())) * len(set(mine[:, 5].tolist())) == 32  # a full rectangle
        assert len(set(mine[:, 3].tolist())) + len(set(mine[:, 5].tolist())) <= 12   # 4 x 8


def row_tiles(sizes, mode, m_total, aux, tile, n_chunk=0):
    lib = _native.load()
    s = np.asarray(sizes, dtype=np.int64)
    cap = 1 << 14
    out = np.zeros((cap, 3), dtype=np.int64)
    n = ctypes.c_int64(0)
    rc = lib.tgg_debug_row_tiles(s.ctypes.data, len(s), mode, m_total, aux, tile, n_chunk, out.ctypes.data, cap,
                                 ctypes.byref(n))
    assert rc == 0, lib.tgg_last_error().decode()
    return out[:n.value].tolist()


@pytest.mark.parametrize("tile", [128, 256])
@pytest.mark.parametrize("n_chunk", [0, 1, 2, 8])
@pytest.mark.parametrize("sizes", [
    [300, 0, 130, 128],          # the case on which the transposing quantizer once read the wrong row block
    [1, 0, 127, 129, 256, 3, 0, 300],
    [2048] * 32,
    [0, 0, 5],
    list(range(0, 700, 37)),
])
def test_row_tile_lookup(tile, n_chunk, sizes):
    """The lookup the transposing quantizer uses (global row tile -> group, first row, valid rows) against a plain
    Python enumeration of the groups' tiles; it must not depend on the column-chunk option of the GEMM tile order."""
    exp, start = [], 0
    for g, sz in enumerate(sizes):
        for mt in range(-(-sz // tile)):
            exp.append([g, start + mt * tile, min(tile, sz - mt * tile)])
        start += sz
    assert row_tiles(sizes, MG, sum(sizes), 0, tile, n_chunk) == exp


def test_row_tile_lookup_padded_and_masked():
    sizes = [100, 0, 130, 128]
    assert row_tiles(sizes, MG_PAD, 512, 128, 128) == [[0, 0, 100], [2, 128, 128], [2, 256, 2], [3, 384, 128]]
    assert row_tiles([512, 0, 77, 300], MASKED, 2048, 512, 256) == [
        [0, 0, 256], [0, 256, 256], [2, 1024, 77], [3, 1536, 256], [3, 1792, 44]]


@pytest.mark.parametrize("grid", [8, 64, 104, 256])
def test_work_queue_deals_every_tile_once_and_each_counter_in_growing_order(grid):
    """The K-grouped kernels draw tile ids from eight counters (one per XCD).  A counter is taken for exhausted at
    its first id beyond the tile space, and workgroups then steal from the other counters: that is only right if
    each counter's ids grow with the number of draws and the eight sequences together are a permutation of the ids.
    The deal hands out runs of grid/8 neighbouring tiles, eight runs per pass, forwards and backwards in turn."""
    lib = _native.load()
    R, draws = grid // 8, 7 * (grid // 8) + 3
    out = np.full((8, draws), -1, dtype=np.int32)
    assert lib.tgg_debug_queue_order(grid, draws, out.ctypes.data) == 0, _native.last_error()
    assert (np.diff(out, axis=1) > 0).all()
    full = 7 * grid  # the first seven passes are dealt completely
    ids = np.sort(out[out < full])
    assert np.array_equal(ids, np.arange(full))
    runs = out[:, :7 * R].reshape(8, 7, R)
    assert (np.diff(runs, axis=2) == 1).all(), "a run is R neighbouring tiles"
    first = runs[:, :, 0] // R  # run number in the tile space, by counter and pass
    for k in range(7):
        order = np.argsort(first[:, k])
        assert np.array_equal(first[order, k], 8 * k + np.arange(8))
        assert np.array_equal(order, np.arange(8) if k % 2 == 0 else np.arange(8)[::-1]), "back and forth"
    bad = np.zeros((8, 4), dtype=np.int32)
    assert lib.tgg_debug_queue_order(100, 4, bad.ctypes.data) == 1  # not a multiple of 8: one counter, ids in order


def _many_group_sizes(G, seed, top):
    rng = np.random.default_rng(seed)
    sizes = rng.choice([0, 0, 3, 16, 40, 128, 129, 300, top], size=G)
    sizes[G // 2 - 1], sizes[G // 2] = 77, 130  # rows on both sides of the middle of the table
    sizes[511], sizes[512] = 77, 130             # ... and of entry 512
    return [int(x) for x in sizes]


@pytest.mark.parametrize("tile", [128, 256])
@pytest.mark.parametrize("G", [513, 600, 1024])
@pytest.mark.parametrize("mode", [MG, MG_PAD, MASKED, KG_COUNT])
def test_cover_with_more_than_512_groups(tile, G, mode):
    """Group counts beyond the tuned kernels' 512-entry table, which the shape-agnostic kernel's 1024-entry table
    takes: every tile exactly once, rows inside each group's range and inside the operand, for every way the groups
    can be laid out (contiguous, padded, masked, K-grouped by counts)."""
    N, grid = 264, 256
    if mode == MASKED:
        m_stride = 256
        sizes = _many_group_sizes(G, G + tile, m_stride)  # holds counts above m_stride: the kernel clips them
        rows, n = tile_order(sizes, MASKED, G * m_stride, m_stride, N, tile, grid, 1)
        starts = [g * m_stride for g in range(G)]
        exp = expected_m_grouped_tiles([min(s, m_stride) for s in sizes], starts, tile, N, G * m_stride)
    elif mode == KG_COUNT:
        sizes = [16 * (s % 13) for s in _many_group_sizes(G, G + tile, 192)]
        mdim = 136
        rows, n = tile_order(sizes, KG_COUNT, mdim, sum(sizes), N, tile, grid, 0)
        exp = {(g, mt * tile, min(tile, mdim - mt * tile), nt * tile)
               for g in range(G) for mt in range(-(-mdim // tile)) for nt in range(-(-N // tile))}
    else:
        sizes = _many_group_sizes(G, G + tile, 517)
        align = 128 if mode == MG_PAD else 1
        padded = [-(-s // align) * align for s in sizes]
        starts = np.concatenate([[0], np.cumsum(padded)[:-1]]).tolist()
        m_total = sum(padded)
        rows, n = tile_order(sizes, mode, m_total, align if mode == MG_PAD else 0, N, tile, grid, 1)
        exp = expected_m_grouped_tiles(sizes, starts, tile, N, m_total)
    got = [tuple(r[2:6]) for r in rows.tolist()]
    assert n == len(exp) == len(got)
    assert set(got) == exp and len(set(got)) == len(got)
    assert 0 <= rows[:, 2].min() and rows[:, 2].max() < G


def test_a_negative_row_start_gives_the_group_no_rows():
    """Placed groups take their first row from device memory: a start in front of the operand must not be computed on
    (the upper end was always clipped)."""
    lib = _native.load()
    sizes = np.asarray([100, 50, 30], dtype=np.int64)
    starts = np.asarray([200, -64, 0], dtype=np.int32)
    out = np.zeros((7, 2), dtype=np.int64)
    assert lib.tgg_debug_generic_extents(4, sizes.ctypes.data, starts.ctypes.data, 3, 300, 0, 128, 64, out.ctypes.data) == 0
    assert out[0, 0] == 0 and out[0, 1] == 299 * 64 + 63         # A: rows 0..29 and 200..299 only
    assert out[2, 0] == 0 and out[2, 1] == 299 * 128 + 127       # C likewise
    assert out[1, 0] == 0 and out[1, 1] == 3 * 128 * 64 - 1      # weights of groups 0 and 2 (group 1 is never touched,
    #                                                              but it lies between them)
