// Per-workgroup tile scheduler for grouped GEMMs.
//
// Every workgroup rebuilds the same small table in LDS from the per-group sizes
// (an exclusive prefix sum of rows and of M-tiles) and then walks the tile space
// with a persistent, XCD-aware stride.  No host-side metadata, no workspace, no
// host/device synchronisation.
#pragma once
#include "common.hpp"

namespace tgg {

constexpr int kMaxGroups = 1024;

template <int MAXG>
struct SchedTableT {
  int64_t row0[MAXG];      // first row of the group in A/C (M modes) or first k (K modes)
  int32_t rows[MAXG];      // valid rows (M modes) or k extent (K modes)
  int32_t tile0[MAXG + 1]; // M modes: exclusive prefix of ceil(rows / BM); K modes: the groups in the order of the tile space (sched_order_groups)
  int32_t pad_;            // how many tiles more a cut at half the tile height has (set by sched_init)
  int64_t scan_[16];       // per-wave totals of the workgroup-wide prefix sums that build the table
};
typedef SchedTableT<kMaxGroups> SchedTable;

struct Tile {
  int g;
  int64_t row0;   // first row of this tile in A and C (M modes); first m within the group (K modes)
  int rows;       // valid rows in this tile (<= BM)
  int n0;
  int64_t k0;     // reduction range [k0, k1)
  int64_t k1;
};

// The functions below that are marked TGG_HD contain no device-only construct: the library also runs them
// on the host to report the tile order (a test hook), so what the tests check is what the kernels execute.
#define TGG_HD __host__ __device__ __forceinline__

TGG_HD int64_t load_size(const void* p, int is64, int i) {
  int64_t v = is64 ? ((const int64_t*)p)[i] : (int64_t)((const int32_t*)p)[i];
  return v < 0 ? 0 : v;
}

// Entry g of the table before the prefix pass: the group's raw extent.
template <class Table>
TGG_HD void sched_load_group(const GemmParams& p, Table& t, int g) {
  if (p.mode == MODE_KG) {
    int64_t s = p.k_start[g], e = p.k_end[g];
    if (s < 0) s = 0;
    if (e > p.k_total) e = p.k_total;
    t.row0[g] = s;
    t.rows[g] = e > s ? (int32_t)(e - s) : 0;
  } else {
    t.rows[g] = (int32_t)load_size(p.sizes, p.sizes_i64, g);
  }
}

// Serial prefix pass over the loaded extents (every mode but MODE_KG, whose ranges are explicit).
template <int BM, class Table>
TGG_HD void sched_prefix(const GemmParams& p, Table& t) {
  const int G = p.G;
  int64_t row = 0;
  int32_t tile = 0;
  for (int g = 0; g < G; ++g) {
    int64_t sz = t.rows[g];
    int64_t start;
    if (p.mode == MODE_MASKED) {
      start = (int64_t)g * p.m_stride;
      if (sz > p.m_stride) sz = p.m_stride;
    } else {
      start = (p.mode == MODE_MG_PAD && p.row_start) ? (int64_t)p.row_start[g] : row;
      row += (p.mode == MODE_MG_PAD) ? ((sz + p.align - 1) / p.align) * p.align : sz;
    }
    const int64_t limit = (p.mode == MODE_KG_COUNT) ? p.k_total : p.m_total;
    if (start < 0 || start >= limit) sz = 0;  // never touch rows (or k) outside the operands (a negative start can only come from row_start)
    else if (start + sz > limit) sz = limit - start;
    t.row0[g] = start;
    t.rows[g] = (int32_t)sz;
    t.tile0[g] = tile;
    tile += (int32_t)((sz + BM - 1) / BM);
  }
  t.tile0[G] = tile;
}

// K-grouped tile space: a tile costs what its group has tokens, every group has the same number of tiles, and the
// persistent workgroups take tile ids with a fixed stride -- so with 192 tiles per group and 256 workgroups each
// workgroup misses every fourth group, and which fourth decides its load.  The tile space therefore runs over the
// groups in order of decreasing token count (ties by index): the sums over every fourth group of a sorted sequence
// differ by less than the largest group, and the launch ends on its cheapest tiles.  t.tile0[i] = the group whose
// tiles come i-th.  Position of group g = number of groups that precede it in that order.
template <class Table>
TGG_HD int sched_group_rank(const Table& t, int G, int g) {
  const int32_t mine = t.rows[g];
  int rank = 0;
  for (int h = 0; h < G; ++h) {
    const int32_t other = t.rows[h];
    rank += (other > mine) || (other == mine && h < g);
  }
  return rank;
}

// Serial form (host hook, and kernels whose workgroups have fewer threads than there are groups).
template <class Table>
TGG_HD void sched_order_groups_serial(const GemmParams& p, Table& t) {
  for (int g = 0; g < p.G; ++g) t.tile0[sched_group_rank(t, p.G, g)] = g;
}

// Exclusive prefix sum over the workgroup's threads (in thread order) and the total; all threads must call it.
// Wave-wide scan by lane exchange, the waves' totals through the table's scratch words.
template <class Table>
TGG_DEV int64_t sched_block_scan(int64_t v, Table& t, int64_t& total) {
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, waves = ((int)blockDim.x + 63) >> 6;
  int64_t inc = v;
#pragma unroll
  for (int d = 1; d < 64; d <<= 1) {
    const int64_t o = __shfl_up(inc, d, 64);
    if (lane >= d) inc += o;
  }
  if (lane == 63) t.scan_[wave] = inc;
  __syncthreads();
  int64_t base = 0, tot = 0;
  for (int w = 0; w < waves; ++w) {
    const int64_t s = t.scan_[w];
    if (w < wave) base += s;
    tot += s;
  }
  __syncthreads();  // the scratch words are free again
  total = tot;
  return base + inc - v;
}

// K modes only (a no-op otherwise): fills t.tile0 with the groups in tile-space order once t.rows is final.  All
// threads of the workgroup must call this; ends with a barrier when it does anything.
template <class Table>
TGG_DEV void sched_order_groups(const GemmParams& p, Table& t) {
  if (p.mode != MODE_KG && p.mode != MODE_KG_COUNT) return;
  for (int g = threadIdx.x; g < p.G; g += blockDim.x) t.tile0[sched_group_rank(t, p.G, g)] = g;
  __syncthreads();
}

// Builds the table.  All threads of the workgroup must call this; ends with a barrier.
// With one thread per group (G <= workgroup size <= 1024) the two prefix sums of sched_prefix -- group starts, then
// tiles of the clipped sizes -- are workgroup-wide scans: about a microsecond, where the serial pass of one thread
// takes 0.2 us per group (15 us at 128 groups, a tenth of a decode-sized launch).  Same values as sched_prefix.
// The tile scan carries the prefix for tiles of half the height along in its upper word: the calling thread's group
// would start at the returned tile id under that cut, and t.pad_ receives how many tiles more that cut has in all
// (see sched_use_half_height).  Where the serial pass runs instead, t.pad_ is set so large that no caller prefers
// the half-height cut.
template <int BM, class Table>
TGG_DEV int32_t sched_init(const GemmParams& p, Table& t) {
  if (p.mode == MODE_KG || p.G > (int)blockDim.x || blockDim.x > 1024) {
    for (int g = threadIdx.x; g < p.G; g += blockDim.x) sched_load_group(p, t, g);
    __syncthreads();
    if (p.mode != MODE_KG) {
      if (threadIdx.x == 0) {
        sched_prefix<BM>(p, t);
        t.pad_ = 1 << 30;
      }
      __syncthreads();
    }
    sched_order_groups(p, t);
    return 0;
  }
  const int g = threadIdx.x;
  const bool live = g < p.G;
  int64_t sz = live ? load_size(p.sizes, p.sizes_i64, g) : 0;
  int64_t start;
  if (p.mode == MODE_MASKED) {
    start = (int64_t)g * p.m_stride;
    if (sz > p.m_stride) sz = p.m_stride;
  } else {
    const int64_t step = (p.mode == MODE_MG_PAD) ? ((sz + p.align - 1) / p.align) * p.align : sz;
    int64_t all;
    start = sched_block_scan(step, t, all);
    if (p.mode == MODE_MG_PAD && p.row_start && live) start = (int64_t)p.row_start[g];
  }
  const int64_t limit = (p.mode == MODE_KG_COUNT) ? p.k_total : p.m_total;
  if (start < 0 || start >= limit) sz = 0;  // never touch rows (or k) outside the operands (a negative start can only come from row_start)
  else if (start + sz > limit) sz = limit - start;
  constexpr int HALF = BM / 2;
  int64_t total;
  const int64_t both = sched_block_scan((sz + BM - 1) / BM + (((sz + HALF - 1) / HALF) << 32), t, total);
  if (live) {
    t.row0[g] = start;
    t.rows[g] = (int32_t)sz;
    t.tile0[g] = (int32_t)(both & 0xffffffff);
  }
  if (threadIdx.x == 0) {
    t.tile0[p.G] = (int32_t)(total & 0xffffffff);
    t.pad_ = (int32_t)(total >> 32) - (int32_t)(total & 0xffffffff);
  }
  __syncthreads();
  sched_order_groups(p, t);
  return (int32_t)(both >> 32);
}

// Switches a table built by sched_init<BM> to tiles of half that height: half_tile0 is what sched_init returned
// to this thread.  All threads of the workgroup must call this; starts and ends with a barrier (other threads may
// still be reading the totals that it overwrites).
template <class Table>
TGG_DEV void sched_use_half_height(const GemmParams& p, Table& t, int32_t half_tile0) {
  __syncthreads();
  if ((int)threadIdx.x < p.G) t.tile0[threadIdx.x] = half_tile0;
  if (threadIdx.x == 0) t.tile0[p.G] += t.pad_;
  __syncthreads();
}

// K-grouped by counts: does the launch pass its gate (GemmParams::kg_gate)?  All threads of the workgroup must call
// this after sched_init; the answer is the same in every workgroup of the launch.
template <class Table>
TGG_DEV bool sched_kg_gate_open(const GemmParams& p, const Table& t) {
  if (p.kg_gate == 0) return true;
  int bad = 0;
  for (int g = threadIdx.x; g < p.G; g += blockDim.x) bad |= (t.rows[g] & 15) != 0;
  const int n_bad = __syncthreads_count(bad);
  return p.kg_gate == 1 ? n_bad == 0 : n_bad != 0;
}

template <int BM, int BN, class Table>
TGG_HD int64_t sched_num_tiles(const GemmParams& p, const Table& t) {
  const int tiles_n = (p.N + BN - 1) / BN;
  if (p.mode == MODE_KG || p.mode == MODE_KG_COUNT) {
    const int tiles_m = (int)((p.m_total + BM - 1) / BM);
    return (int64_t)p.G * tiles_m * tiles_n;
  }
  return (int64_t)t.tile0[p.G] * tiles_n;
}

// Whether tiles of half the table's tile height pay for an M-grouped launch.  t.pad_ holds the tiles that the half
// height cut has over the table's cut (sched_init leaves it there).  The persistent workgroups work in rounds (one
// tile each per round), a half-height tile costs about 0.7 of a full one (measured over group counts 8-256 and
// 64-2048 rows per group, for both operand widths), and what decides is whole rounds: a launch whose full-height
// tiles just fit one round loses by going to two rounds of short tiles, whatever their number.
template <int BN, class Table>
__device__ __forceinline__ bool sched_short_tiles_pay(const GemmParams& p, const Table& t) {
  const int64_t tiles_n = (p.N + BN - 1) / BN, wgs = gridDim.x;
  const int64_t rounds_full = ((int64_t)t.tile0[p.G] * tiles_n + wgs - 1) / wgs;
  const int64_t rounds_half = ((int64_t)(t.tile0[p.G] + t.pad_) * tiles_n + wgs - 1) / wgs;
  return rounds_half * 7 <= rounds_full * 10;
}

// Whether a launch of 256-row tiles is neither small enough for the narrow tiles (all of them fit one round of the
// persistent workgroups) nor made of groups so small that 128-row tiles pay: the case in which the eight-wave kernels
// run their BM x BN configuration.  t: a table built by sched_init<BM> with one thread per group.
template <int BM, int BN, class Table>
__device__ __forceinline__ bool sched_wide_tiles_chosen(const GemmParams& p, const Table& t) {
  return sched_num_tiles<BM, BN / 2>(p, t) > (int64_t)gridDim.x && !sched_short_tiles_pay<BN>(p, t);
}

// Tile order.  Consecutive tile ids are handed to workgroups that run at the same time on one XCD
// (see sched_walk), so a run of ids should cover a near-square block of tiles: a run of R tiles spanning
// w column tiles touches R / w row panels of A plus w column panels of B per K slab.  The N tiles are
// therefore cut into chunks of at most eight columns and ids run over (chunk, row tile, column within
// chunk), innermost last.  Eight rather than the square root of an XCD's 32 workgroups: B panels
// (weights) are reused by the following row tiles of the group, A panels are streamed once, so the
// wider side goes to B.
TGG_HD int sched_chunk_width(int tiles_n, int n_chunk) {
  if (n_chunk > 0) return n_chunk < tiles_n ? n_chunk : tiles_n;
  const int chunks = (tiles_n + 7) / 8;
  return (tiles_n + chunks - 1) / chunks;
}

// Splits the position `r` inside a block of `rows_m` row tiles x `tiles_n` column tiles into (row tile, column tile).
TGG_HD void sched_split(int r, int rows_m, int tiles_n, int nc, int& mt, int& nt) {
  const int chunk_tiles = rows_m * nc;
  int c = r / chunk_tiles;
  const int full = tiles_n / nc;
  int width = nc;
  if (c >= full) {  // the last, narrower chunk
    c = full;
    width = tiles_n - full * nc;
  }
  const int q = r - c * chunk_tiles;
  mt = q / width;
  nt = c * nc + (q - mt * width);
}

// Row-tile lookup shared by every consumer of the group table (every mode but the K-grouped ones): which group
// owns the global BM-row tile `mt_glob` (counted over the groups' tiles in order, independent of the tile-id
// order that sched_tile lays over the (row tile, column tile) space), where its rows start and how many are valid.
// g_hint: a group at or before the tile's group, if the caller knows one (a workgroup's walk visits tiles in
// increasing order, and within a column chunk their groups never decrease): the lookup then checks the hinted
// group and its successor before it falls back to the binary search, each probe being a dependent LDS read.
struct RowTile {
  int g;
  int64_t row0;
  int rows;
};

template <int BM, class Table>
TGG_HD RowTile sched_row_tile(const Table& t, int G, int mt_glob, int g_hint = -1) {
  int lo = 0, hi = G;  // last g with tile0[g] <= mt_glob
  if (g_hint >= 0 && g_hint < G && t.tile0[g_hint] <= mt_glob) {
    lo = g_hint;
    if (t.tile0[lo + 1] > mt_glob) hi = lo + 1;            // tile0 has G + 1 entries
    else if (lo + 2 <= G && t.tile0[lo + 2] > mt_glob) { lo = lo + 1; hi = lo + 1; }
    else lo = lo + 1;                                      // further on: search [lo, G)
  }
  while (hi - lo > 1) {
    const int mid = (lo + hi) >> 1;
    if (t.tile0[mid] <= mt_glob) lo = mid; else hi = mid;
  }
  RowTile r;
  r.g = lo;
  const int mt = mt_glob - t.tile0[lo];
  r.row0 = t.row0[lo] + (int64_t)mt * BM;
  const int left = t.rows[lo] - mt * BM;
  r.rows = left < BM ? left : BM;
  return r;
}

template <int BM, int BN, class Table>
TGG_HD Tile sched_tile(const GemmParams& p, const Table& t, int64_t tile_id, int g_hint = -1) {
  Tile r;
  const int tiles_n = (p.N + BN - 1) / BN;
  const int nc = sched_chunk_width(tiles_n, p.n_chunk);
  const int tid32 = (int)tile_id;  // the tile space is far below 2^31; 32-bit division is much cheaper
  if (p.mode == MODE_KG || p.mode == MODE_KG_COUNT) {
    const int tiles_m = (int)((p.m_total + BM - 1) / BM);
    const int per_group = tiles_m * tiles_n;
    const int slot = tid32 / per_group;
    r.g = t.tile0[slot];  // groups in order of decreasing size, see sched_group_rank
    int mt, nt;
    sched_split(tid32 - slot * per_group, tiles_m, tiles_n, nc, mt, nt);
    r.n0 = nt * BN;
    r.row0 = (int64_t)mt * BM;
    const int64_t left = p.m_total - r.row0;
    r.rows = left < BM ? (int)left : BM;
    r.k0 = t.row0[r.g];
    r.k1 = r.k0 + t.rows[r.g];
    return r;
  }
  int mt_glob, nt;
  sched_split(tid32, t.tile0[p.G], tiles_n, nc, mt_glob, nt);
  const RowTile rt = sched_row_tile<BM>(t, p.G, mt_glob, g_hint);
  r.n0 = nt * BN;
  r.g = rt.g;
  r.row0 = rt.row0;
  r.rows = rt.rows;
  r.k0 = 0;
  r.k1 = p.K;
  return r;
}

// Persistent walk of the tile space by workgroup b of P.  Consecutive workgroup ids land on
// different XCDs (round robin over 8), each with its own L2, so the walk is laid out per XCD:
//   split = true   XCD x owns the contiguous tile range [x*T/8, (x+1)*T/8) and its P/8 workgroups
//                  sweep it in runs of P/8 neighbouring tiles.  Neighbours share activation rows and
//                  expert weights, and an expert's weights are fetched by one or two XCDs only.
//                  Right when all tiles cost the same (M-grouped: K is fixed).
//   split = false  every sweep hands each XCD a run of P/8 neighbouring tiles, sweeps interleaved over
//                  the whole space.  Used when tile cost varies along the tile order (K-grouped:
//                  cost follows the group's token count), so that every XCD sees every group.
struct TileWalk {
  int64_t first, end, stride;
};

TGG_HD TileWalk sched_walk_of(int64_t num_tiles, bool split, int P, int b) {
  TileWalk w;
  if ((P & 7) != 0) {
    w.first = b; w.end = num_tiles; w.stride = P;
  } else if (split) {
    const int x = b & 7;
    w.first = (num_tiles * x) / 8 + (b >> 3);
    w.end = (num_tiles * (x + 1)) / 8;
    w.stride = P >> 3;
  } else {
    w.first = (int64_t)(b & 7) * (P >> 3) + (b >> 3);
    w.end = num_tiles;
    w.stride = P;
  }
  return w;
}

TGG_DEV TileWalk sched_walk(int64_t num_tiles, bool split) {
  return sched_walk_of(num_tiles, split, (int)gridDim.x, (int)blockIdx.x);
}

// The tile id behind the n-th draw from XCD xq's counter (R = workgroups per XCD): run n / R of that XCD, which is run
// xq of the deal's pass n / R when the pass runs forwards (even) and run 7 - xq when it runs backwards.
TGG_HD int sched_queue_id(int n, int xq, int R) {
  const int pass = n / R;
  return (pass * 8 + ((pass & 1) ? 7 - xq : xq)) * R + n % R;
}

// Work queue of the K-grouped tuned kernels: eight counters in global memory, one per XCD (zero at launch).  The
// tile space is cut into runs of R neighbouring tiles (R = workgroups per XCD; neighbours are tiles of one group,
// which share operand panels in an XCD's L2), and the runs are dealt to the XCDs in order of decreasing cost, back
// and forth (0..7, 7..0, ...) so that no XCD always gets the dearest of eight.  Within an XCD a tile goes to
// whichever workgroup asks next: like the static interleaved walk the XCD works through runs of neighbours, but a
// workgroup that drew expensive tiles draws fewer.  A workgroup whose own XCD has nothing left takes from the
// next XCD's counter, and so on round the ring: what the deal leaves uneven is evened out at the end.  For every
// counter the ids grow with the number of draws, so one id at or beyond `total` means that counter is exhausted.
// `victim` (0 at first; kept by the drawing thread) counts the counters found exhausted so far; returns an id at
// or beyond `total` when all eight are.
TGG_DEV int sched_draw_tile(int32_t* queue, int total, int& victim) {
  const int P = (int)gridDim.x;
  if ((P & 7) != 0) return atomicAdd(queue, 1);
  const int x = (int)blockIdx.x & 7, R = P >> 3;
  while (victim < 8) {
    const int xq = (x + victim) & 7;
    const int id = sched_queue_id(atomicAdd(queue + xq, 1), xq, R);
    if (id < total) return id;
    ++victim;
  }
  return total;
}

// End of a queued launch: every workgroup reports here once it has drawn its last id (the draw that found all eight
// counters exhausted has returned by then), and the workgroup that reports last puts the nine words back to zero, so
// that the next launch on the same stream finds the queue as this one found it.  Thread 0 of each workgroup calls it.
constexpr int kQueueDoneWord = 8;
TGG_DEV void sched_queue_finish(int32_t* queue) {
  if (atomicAdd(queue + kQueueDoneWord, 1) == (int)gridDim.x - 1) {
    for (int i = 0; i <= kQueueDoneWord; ++i) atomicExch(queue + i, 0);
  }
}

}  // namespace tgg
