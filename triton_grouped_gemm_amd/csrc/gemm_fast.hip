// Tuned bf16/fp16 grouped GEMM kernels for gfx950.
//
// One kernel template covers the three operand layouts of the grouped-GEMM path:
//   NT  A [rows, K]      B [G, N, K]   (forward, masked/decode, contiguous-padded)
//   NN  A [rows, K]      B [G, K, N]   (activation gradient)
//   TN  A [Ktot, Mdim]   B [Ktot, N]   (K-grouped weight gradient, per-group token range)
//
// Persistent workgroups walk the grouped tile space (sched.hpp).  Per 256x256 (or smaller) tile:
//   * 64-deep K slabs of both operands stream HBM/L2 -> LDS with buffer_load_dwordx4 ... lds, no
//     VGPR staging.  Anything outside an operand (rows past the end of A, tokens past the end of
//     a group's range) reads as zero through the buffer descriptor's bounds check, so ragged
//     groups and token tails need no separate code path.
//   * Two slab buffers alternate in LDS with one workgroup barrier per slab.  The slabs of all of a
//     workgroup's tiles form one uninterrupted stream: the copies run two slabs ahead of the
//     multiplies across tile boundaries, and the fragment reads run one K step ahead across the
//     barrier, so neither the barrier nor the LDS latency behind it leaves the matrix pipe idle.
//   * A slab's copy instructions are issued between multiplies rather than back to back: the
//     address unit takes 16 cycles per copy and has a short queue, and a wave blocked on that queue
//     cannot issue its multiplies.
//   * LDS is XOR-swizzled at 16-byte granularity.  The direct-to-LDS copy is lane-linear on the
//     LDS side, so the swizzle is applied to the global address each lane fetches from.
//   * K-contiguous operands are read back as 16-byte MFMA fragments (ds_read_b128); operands whose
//     rows are tokens (MN-contiguous) are read with the transposing ds_read_b64_tr_b16, which hands
//     every lane 4 consecutive K values of one column.
//   * Each wave owns a (BM/WM) x (BN/WN) block of 16x16x32 MFMA tiles.  That shape is chosen for power: with
//     all 256 CUs multiplying random operands the chip is power-limited, and 16x16x32 delivers about 20 % more
//     flops per watt than 32x32x16 (a quarter of the accumulator traffic per multiply-add pair of operands);
//     it also keeps full issue rate with two waves per SIMD, which 32x32x16 with distinct operand registers
//     does not.  Multiplies are issued with the B operand as srcA and the A operand as srcB, so a lane ends up
//     with 4 consecutive output columns of one row; results are transposed one 16-row strip at a time through a
//     small per-wave LDS staging area (separate from the slab buffers, so the copy stream keeps running) and
//     leave as 16-byte stores that cover whole row segments of the wave's columns.
#include "fast_common.hpp"
#include "launch.hpp"
#include <atomic>
#include <type_traits>

namespace tgg {

namespace {

enum : int { LAYOUT_NT = 0, LAYOUT_NN = 1, LAYOUT_TN = 2 };
constexpr int BK = 64;  // K depth of a slab for 16-bit operands

template <int DT> struct Mma16;
template <> struct Mma16<DT_BF16> {
  static TGG_DEV f32x4_t run(i32x4_t w, i32x4_t x, f32x4_t c) {
    return __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8_t, w), __builtin_bit_cast(bf16x8_t, x), c, 0, 0, 0);
  }
};
template <> struct Mma16<DT_F16> {
  static TGG_DEV f32x4_t run(i32x4_t w, i32x4_t x, f32x4_t c) {
    return __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(f16x8_t, w), __builtin_bit_cast(f16x8_t, x), c, 0, 0, 0);
  }
};

// fp32 -> nearest 16-bit value of the output type (as fp32), and 16 bits -> fp32
template <int DT> TGG_DEV float round16(float x) {
  if (DT == DT_BF16) return (float)(__bf16)x;
  return (float)(_Float16)x;
}
template <int DT> TGG_DEV float from16(uint16_t h) {
  if (DT == DT_BF16) return __builtin_bit_cast(float, (uint32_t)h << 16);
  return (float)__builtin_bit_cast(_Float16, h);
}

// BST: slab buffers of the B operand.  2: A and B slabs of a stage sit together, two stages.  3: the A slabs keep
// two buffers, the B slabs get a ring of three of their own and their copies run a slab further ahead (the
// weight-streaming configuration, see gemm_fast_body).
template <int BM_, int BN_, int WM_, int WN_, int BST_ = 2>
struct FastCfg {
  static constexpr int BM = BM_, BN = BN_, WM = WM_, WN = WN_, BST = BST_;
  static constexpr int NWAVES = WM * WN;
  static constexpr int THREADS = NWAVES * 64;
  static constexpr int A_BYTES = BM * BK * 2, B_BYTES = BN * BK * 2;
  static constexpr int STAGE_BYTES = A_BYTES + B_BYTES;
  static constexpr int NI_A = A_BYTES / 1024, NI_B = B_BYTES / 1024;
  static constexpr int TM = BM / WM / 16, TN = BN / WN / 16;  // 16x16 blocks per wave
  static constexpr int EPI_PITCH = TN * 32 + 16;  // staged strip of 16 rows x (16 TN) 16-bit outputs: row pitch in bytes
  static constexpr int EPI_WAVE_BYTES = 16 * EPI_PITCH;
  static constexpr int SCHED_OFF = 2 * A_BYTES + BST * B_BYTES;
  // byte offsets of A buffer a (0, 1) and B buffer b (0 .. BST-1)
  static constexpr int a_off(int a) { return BST == 2 ? a * STAGE_BYTES : a * A_BYTES; }
  static constexpr int b_off(int b) { return BST == 2 ? b * STAGE_BYTES + A_BYTES : 2 * A_BYTES + b * B_BYTES; }
  static constexpr int EPI_OFF = SCHED_OFF + (((int)sizeof(SchedTableT<kFastMaxGroups>) + 255) & ~255);
  static constexpr int QMAX_OFF = EPI_OFF + NWAVES * EPI_WAVE_BYTES;  // fused quantisation: [WN][BM] 16-bit row maxima
  static constexpr int SMEM_BYTES = QMAX_OFF + WN * BM * 2;
  static_assert(NI_A % NWAVES == 0 && NI_B % NWAVES == 0, "copies must divide evenly over waves");
  static_assert(NWAVES % 8 == 0, "a wave keeps one swizzle pattern for all its copies");
  static_assert(BST == 2 || BST == 3, "B slab buffers");
  static_assert(SMEM_BYTES <= 160 * 1024, "LDS budget");
};

// The whole kernel but for the group table, which the caller has built at byte SCHED_AT of the workgroup's LDS
// (C::SCHED_OFF unless two tile configurations share one kernel, see gemm_fast_auto_kernel).
template <class C, int DT, int LAYOUT, bool QUANT, int SCHED_AT>
TGG_DEV void gemm_fast_body(const GemmParams& p) {
  constexpr bool A_KMAJOR = LAYOUT != LAYOUT_TN;
  constexpr bool B_KMAJOR = LAYOUT == LAYOUT_NT;
  // DEEP: three B slab buffers, B copies one slab further ahead than A copies.  For launches that stream weights
  // (few rows per group, decode): what limits them is how many bytes of B a CU has in flight, and a B slab of the
  // two-buffer scheme is requested only one slab period before it is needed.
  constexpr bool DEEP = C::BST == 3;
  static_assert(!DEEP || !QUANT, "the fused-quantisation epilogue uses the two-buffer configuration");
  typedef Operand<C::BM, A_KMAJOR> OpA;
  typedef Operand<C::BN, B_KMAJOR> OpB;

  extern __shared__ __attribute__((aligned(1024))) char smem[];
  auto& sched_rw = *reinterpret_cast<SchedTableT<kFastMaxGroups>*>(smem + SCHED_AT);
  const auto& sched = sched_rw;
  const int64_t num_tiles = sched_num_tiles<C::BM, C::BN>(p, sched);

  const uint32_t smem_addr = (uint32_t)(uintptr_t)(lds_ptr_t)smem;
  const int lane = lane_id();
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int wm0 = (wave / C::WN) * (C::BM / C::WM);
  const int wn0 = (wave % C::WN) * (C::BN / C::WN);
  const int l16 = lane & 15, lg = lane >> 4;

  // global row pitches in bytes
  const int64_t a_ld = (LAYOUT == LAYOUT_TN ? p.m_total : (int64_t)p.K) * 2;
  const int64_t b_ld = (LAYOUT == LAYOUT_NT ? (int64_t)p.K : (int64_t)p.N) * 2;

  // per-lane source offsets of this wave's copies (one swizzle pattern per wave, see FastCfg)
  const int a_voff = OpA::lane_voff(lane, wave % OpA::NPAT, (int)a_ld);
  const int b_voff = OpB::lane_voff(lane, wave % OpB::NPAT, (int)b_ld);
  // K tail (K not a multiple of the slab depth): in a tile's last slab the lanes whose 16-byte chunk of a
  // K-contiguous row starts at or beyond K fetch nothing (zeros); token-row operands end with the descriptor.
  const int tail_chunks = LAYOUT == LAYOUT_TN ? 0 : (p.K % BK) / 8;
  const int a_voff_tail = (A_KMAJOR && OpA::lane_chunk(lane, wave % OpA::NPAT) >= tail_chunks) ? kNoFetch : a_voff;
  const int b_voff_tail = (B_KMAJOR && OpB::lane_chunk(lane, wave % OpB::NPAT) >= tail_chunks) ? kNoFetch : b_voff;

  // per-lane LDS offsets of the fragment reads, relative to the operand's slab.  A fragment of the 16x16x32
  // multiply is 8 consecutive K values per lane: K = 32 ks + 8 lg + (0..7) of row or column (block + l16).
  //   K-contiguous: one 16-byte read
  //   token rows:   two transposing 8-byte reads (K 8 lg + 0..3 and + 4..7).  Lane L of a 16-lane group addresses
  //                 8 bytes (4 columns) of token row L / 4; the read returns to lane i the 4 tokens of column i.
  constexpr int KSTEPS = BK / 32;
  int a_rd[A_KMAJOR ? KSTEPS : C::TM];
  int b_rd[B_KMAJOR ? KSTEPS : C::TN];
  if (A_KMAJOR) {
#pragma unroll
    for (int ks = 0; ks < KSTEPS; ++ks) a_rd[ks] = (wm0 + l16) * 128 + (((4 * ks + lg) ^ ((l16 / 2) % 8)) << 4);
  } else {
#pragma unroll
    for (int i = 0; i < C::TM; ++i) {
      const int e = l16 >> 2, c = l16 & 3;
      const int chunk = ((wm0 + 16 * i) / 8 + (c >> 1)) ^ (e * 4) ^ ((lg & 1) * 2);
      a_rd[i] = (lg * 8 + e) * (C::BM * 2) + chunk * 16 + (c & 1) * 8;
    }
  }
  if (B_KMAJOR) {
#pragma unroll
    for (int ks = 0; ks < KSTEPS; ++ks) b_rd[ks] = (wn0 + l16) * 128 + (((4 * ks + lg) ^ ((l16 / 2) % 8)) << 4);
  } else {
#pragma unroll
    for (int j2 = 0; j2 < C::TN; ++j2) {
      const int e = l16 >> 2, c = l16 & 3;
      const int chunk = ((wn0 + 16 * j2) / 8 + (c >> 1)) ^ (e * 4) ^ ((lg & 1) * 2);
      b_rd[j2] = (lg * 8 + e) * (C::BN * 2) + chunk * 16 + (c & 1) * 8;
    }
  }
  // MFMA fragment of K step ks: block i of A / block j of B of the slab at s
  auto load_a = [&](const char* s, int ks, int i) -> i32x4_t {
    if (A_KMAJOR) return *(const i32x4_t*)(s + a_rd[ks] + i * 16 * 128);
    const char* q = s + a_rd[i] + ks * 32 * (C::BM * 2);
    const i16x4_t lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_i16x4_ptr_t)q);
    const i16x4_t hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_i16x4_ptr_t)(q + 4 * (C::BM * 2)));
    return __builtin_bit_cast(i32x4_t, __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7));
  };
  auto load_b = [&](const char* sb, int ks, int j) -> i32x4_t {  // sb: the B slab
    if (B_KMAJOR) return *(const i32x4_t*)(sb + b_rd[ks] + j * 16 * 128);
    const char* q = sb + b_rd[j] + ks * 32 * (C::BN * 2);
    const i16x4_t lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_i16x4_ptr_t)q);
    const i16x4_t hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_i16x4_ptr_t)(q + 4 * (C::BN * 2)));
    return __builtin_bit_cast(i32x4_t, __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7));
  };

  // Slab sequence of a tile, held in scalar registers: where the next slab of each operand starts and how far
  // the copies may reach from there (everything beyond reads as zero).  32-bit bookkeeping keeps the per-slab
  // scalar work short (eight waves share the CU's scalar unit):
  //   K-contiguous operand  rem = bytes left in the tile's window of rows (it shrinks by 128 per slab)
  //   token-row operand     rem = token rows left in the reduction range; a slab may touch
  //                         min(rem, BK) * row pitch - off bytes, off = byte offset of the tile inside a row
  struct TileIo {
    uint64_t a_base, b_base;
    int a_rem, b_rem, a_off, b_off;
    int kt_n, issued;
  };
  const int64_t a_step = A_KMAJOR ? BK * 2 : BK * a_ld;
  const int64_t b_step = B_KMAJOR ? BK * 2 : BK * b_ld;
  // Queued launches (see tile_at below) give the tiles of an empty group one slab of nothing instead of none: the
  // copy stream then advances by exactly one tile per tile, which bounds how far ahead of the multiplies it looks.
  const bool queued = LAYOUT == LAYOUT_TN && p.queue != nullptr;
  auto slabs_of = [&](const Tile& t) -> int {
    if (LAYOUT != LAYOUT_TN) return (p.K + BK - 1) / BK;
    const int n = (int)((t.k1 - t.k0 + BK - 1) / BK);
    return queued && n == 0 ? 1 : n;
  };
  auto make_io = [&](const Tile& t) {
    TileIo io;
    io.kt_n = slabs_of(t);
    io.a_off = io.b_off = 0;
    if (LAYOUT == LAYOUT_TN) {
      const int klen = (int)(t.k1 - t.k0);
      io.a_base = (uint64_t)p.A + (uint64_t)(t.k0 * a_ld + t.row0 * 2);
      io.a_rem = klen;
      io.a_off = (int)(t.row0 * 2);
      io.b_base = (uint64_t)p.B + (uint64_t)(t.k0 * b_ld + (int64_t)t.n0 * 2);
      io.b_rem = klen;
      io.b_off = t.n0 * 2;
    } else {
      // only the tile's valid rows are fetched: the rest of its 256 (another group's rows, or whatever lies beyond
      // masked_m) reads as zero and its products are never stored
      io.a_base = (uint64_t)p.A + (uint64_t)(t.row0 * a_ld);
      io.a_rem = t.rows * (int)a_ld;
      if (LAYOUT == LAYOUT_NT) {
        const int n_left = p.N - t.n0;
        io.b_base = (uint64_t)p.B + (uint64_t)(((int64_t)t.g * p.N + t.n0) * b_ld);
        io.b_rem = (n_left < C::BN ? n_left : C::BN) * (int)b_ld;
      } else {
        io.b_base = (uint64_t)p.B + (uint64_t)((int64_t)t.g * p.K * b_ld + (int64_t)t.n0 * 2);
        io.b_rem = p.K;
        io.b_off = t.n0 * 2;
      }
    }
    io.a_base = uniform64(io.a_base);
    io.b_base = uniform64(io.b_base);
    io.a_rem = __builtin_amdgcn_readfirstlane(io.a_rem);
    io.b_rem = __builtin_amdgcn_readfirstlane(io.b_rem);
    io.a_off = __builtin_amdgcn_readfirstlane(io.a_off);
    io.b_off = __builtin_amdgcn_readfirstlane(io.b_off);
    io.kt_n = __builtin_amdgcn_readfirstlane(io.kt_n);
    io.issued = 0;
    return io;
  };

  // The copy stream.  Slabs of all of this workgroup's tiles form one sequence (tiles without slabs,
  // i.e. empty K-grouped segments, contribute nothing); slab q of the sequence lives in LDS buffer
  // q % 2.  `feed` is the tile whose slabs are being requested, normally one tile ahead of the tile
  // being multiplied.  Once the sequence is exhausted the descriptors get length zero: nothing is
  // fetched, but every wave still issues the same number of copies, which keeps the waits uniform.
  const TileWalk walk = sched_walk(num_tiles, LAYOUT != LAYOUT_TN && p.tile_split);
  // The workgroup's pos-th tile (-1 past its last one).  Static: the walk above.  Queued (K-grouped, whose tiles
  // cost what their groups have tokens, with the groups in order of decreasing size): tile ids are drawn from a
  // counter in global memory, so a workgroup that drew expensive tiles simply draws fewer -- the greedy schedule
  // that evens out what no fixed assignment can.  Thread 0 draws and passes the ids to the other waves through a
  // ring of eight words in the group table's scan scratch; readers use plain LDS reads, so an id must be drawn a
  // workgroup barrier before anyone can ask for it.  Who asks first is the copy stream: it runs two slabs ahead of
  // the multiplies and looks the next tile up as soon as it has requested a tile's last slab.  Thread 0 draws once
  // per tile, right before the barrier of the tile's first slab (what it writes there is seen by all from the
  // next slab on at the latest), and draws on through short tiles until it has drawn one of at least
  // kLongTile slabs -- that one gives the next draw time enough -- or is kQueueAhead tiles ahead (enough for any
  // run of one-slab tiles).  So a workgroup commits itself to one expensive tile beyond the one in work, not more:
  // committing to several is what spoils the balance when a workgroup has only a dozen tiles in all.  Ids at or
  // beyond the tile count end the workgroup's sequence; the counter only grows, so all later ones are too.
  constexpr int kQueueAhead = 5, kLongTile = 5;
  int32_t* const qring = reinterpret_cast<int32_t*>(sched_rw.scan_);
  const int total_tiles = (int)num_tiles;
  auto tile_at = [&](int pos) -> int {
    if (queued) {
      const int id = __builtin_amdgcn_readfirstlane(qring[pos & 7]);
      return id < total_tiles ? id : -1;
    }
    const int64_t id = walk.first + (int64_t)pos * walk.stride;
    return id < walk.end ? (int)id : -1;
  };
  int q_drawn = 0, q_victim = 0;  // thread 0: ids drawn so far, counters found exhausted (see sched_draw_tile)
  // thread 0: makes sure the ids of tiles from..from+kQueueAhead-1 are drawn, up to the first long tile
  auto draw_from = [&](int from) {
    for (int j = from; j < from + kQueueAhead; ++j) {
      if (j >= q_drawn) {
        qring[j & 7] = sched_draw_tile(p.queue, total_tiles, q_victim);
        ++q_drawn;
      }
      const int id = qring[j & 7];
      if (id >= total_tiles || slabs_of(sched_tile<C::BM, C::BN>(p, sched, id)) >= kLongTile) break;
    }
  };
  if (queued) {
    if (threadIdx.x == 0) draw_from(0);
    __syncthreads();
  }
  TileIo feed;
  int feed_pos = 0;
  // The tile the feed last looked up is kept: it is the one the multiplying loop asks for a little later, which
  // saves that loop the lookup (a chain of dependent LDS reads right before a tile's first multiplies).
  Tile seen;
  int seen_id = -1;
  int seen_g = -1;
  // DEEP: the B copies have a cursor of their own, one slab ahead of `feed` (which then serves A only); it does
  // the tile lookups and `feed` reuses them.
  TileIo feedb;
  int feedb_pos = 0;
  Tile seenb;
  int seenb_id = -1;
  int seenb_g = -1;
  auto feedb_seek = [&](int pos) {
    feedb.kt_n = 0;
    feedb.issued = 0;
    feedb.a_base = feedb.b_base = (uint64_t)p.A;
    feedb.a_rem = feedb.b_rem = feedb.a_off = feedb.b_off = 0;
    for (int id; (id = tile_at(pos)) >= 0; ++pos) {
      const Tile tt = sched_tile<C::BM, C::BN>(p, sched, id, seenb_g);
      seenb = tt;
      seenb_id = id;
      seenb_g = tt.g;
      if (slabs_of(tt) > 0) {
        feedb = make_io(tt);
        break;
      }
    }
    feedb_pos = pos;
  };
  auto feed_seek = [&](int pos) {
    feed.kt_n = 0;
    feed.issued = 0;
    feed.a_base = feed.b_base = (uint64_t)p.A;
    feed.a_rem = feed.b_rem = feed.a_off = feed.b_off = 0;
    for (int id; (id = tile_at(pos)) >= 0; ++pos) {
      const Tile tt = (DEEP && id == seenb_id) ? seenb : sched_tile<C::BM, C::BN>(p, sched, id, seen_g);
      seen = tt;
      seen_id = id;
      seen_g = tt.g;
      if (slabs_of(tt) > 0) {
        feed = make_io(tt);
        break;
      }
    }
    feed_pos = pos;
  };
  // One slab's copies are requested in two halves, interleaved with multiplies (see the pipeline below):
  // begin_slab fixes the descriptors and moves the feed on, copy_k issues this wave's k-th copy.
  struct SlabCopy {
    i32x4_t ra, rb;
    uint32_t base, base_b;  // LDS addresses of the A slab and of the B slab
    bool tail, tail_b;      // the tile's last slab, cut short by K (DEEP: A and B are slabs of different numbers)
  };
  constexpr int CA = C::NI_A / C::NWAVES, CB = C::NI_B / C::NWAVES, NC = CA + CB;
  // multiplies between two copies: the first half of a slab's copies goes out right after the barrier, one per
  // multiply (the sooner they are out, the longer they have to land: +1.5-2 % over one per four multiplies;
  // not so with two token-row operands, where the denser issue measured 1.3 % slower), the second half one per
  // four multiplies during the following half step (all eight early: -2 %, the address unit's queue is short)
  constexpr int SP2 = (C::TM * C::TN / 2) / (NC / 2);
  constexpr int SP1 = LAYOUT == LAYOUT_TN ? SP2 : 1;
  static_assert(NC % 2 == 0 && SP2 >= 1, "a slab's copies are spread over the multiplies of two half K steps");
  // DEEP: the next B slab of the B cursor, into B buffer `buf_b`
  auto begin_b = [&](SlabCopy& sc, int buf_b) {
    const bool live = feedb.issued < feedb.kt_n;
    const int b_len = B_KMAJOR ? feedb.b_rem : min(feedb.b_rem, BK) * (int)b_ld - feedb.b_off;
    sc.rb = make_rsrc32(feedb.b_base, live ? b_len : 0);
    sc.base_b = smem_addr + C::b_off(buf_b);
    sc.tail_b = tail_chunks != 0 && feedb.issued + 1 == feedb.kt_n;
    feedb.b_base += b_step;
    feedb.b_rem -= B_KMAJOR ? BK * 2 : BK;
    feedb.issued += 1;
    if (live && feedb.issued >= feedb.kt_n) feedb_seek(feedb_pos + 1);
  };
  // buf: the A buffer (and, with two B buffers, the B buffer); buf_b: the B buffer of the deep ring
  auto begin_slab = [&](int buf, int buf_b = 0) {
    SlabCopy sc;
    const bool counted = feed.issued < feed.kt_n;
    // a queued launch's slab of nothing (empty group): counted like any slab, fetches nothing
    const bool live = counted && (LAYOUT != LAYOUT_TN || feed.a_rem > 0);
    const int a_len = A_KMAJOR ? feed.a_rem : min(feed.a_rem, BK) * (int)a_ld - feed.a_off;
    const int b_len = B_KMAJOR ? feed.b_rem : min(feed.b_rem, BK) * (int)b_ld - feed.b_off;
    sc.ra = make_rsrc32(feed.a_base, live ? a_len : 0);
    sc.base = smem_addr + C::a_off(buf);
    sc.tail = tail_chunks != 0 && feed.issued + 1 == feed.kt_n;
    if (!DEEP) {
      sc.rb = make_rsrc32(feed.b_base, live ? b_len : 0);
      sc.base_b = sc.base + C::A_BYTES;
      sc.tail_b = sc.tail;
    }
    feed.a_base += a_step;
    feed.a_rem -= A_KMAJOR ? BK * 2 : BK;
    feed.b_base += b_step;
    feed.b_rem -= B_KMAJOR ? BK * 2 : BK;
    feed.issued += 1;
    if (counted && feed.issued >= feed.kt_n) feed_seek(feed_pos + 1);
    if (DEEP) begin_b(sc, buf_b);
    return sc;
  };
  auto copy_k = [&](const SlabCopy& sc, int k) {
    if (k < CA) {
      const int idx = wave + k * C::NWAVES;  // wave-uniform
      copy_b128_to_lds(sc.ra, sc.base + idx * 1024, (sc.tail ? a_voff_tail : a_voff) + idx * OpA::RPI * (int)a_ld);
    } else {
      const int idx = wave + (k - CA) * C::NWAVES;
      copy_b128_to_lds(sc.rb, sc.base_b + idx * 1024, (sc.tail_b ? b_voff_tail : b_voff) + idx * OpB::RPI * (int)b_ld);
    }
  };

  // Software pipeline.  A slab is two K steps of 32, each issued as two halves (row blocks 0..TM/2-1, then the
  // rest).  Registers hold one K step of A fragments (replaced one by one: as soon as the multiplies of row
  // block i are issued, fragment i of the following step is read into its place; the last block alternates
  // between two registers so that its successor can be read early) and two K steps of B fragments.  Per slab r:
  //   step 0            multiply while reading step 1 of the same slab;
  //   step 1, 1st half  multiply only;
  //   then wait for this wave's share of slab r+1 and pass the workgroup barrier: slab r+1 is complete and
  //   nobody reads slab r any more, its last fragments are already in registers;
  //   step 1, 2nd half  multiply while reading step 0 of slab r+1 (first the fragments the 1st half skipped).
  // The copies of slab r+2 (into slab r's buffer) are issued between the multiplies of the half step after
  // the barrier and the half step after that, which leaves them a whole K step to land before they are waited
  // for.  They are spread out because the texture-address unit takes 16 cycles per copy instruction and its
  // queue is short: a wave that issues its copies back to back sits blocked behind the other waves' copies with
  // its multiplies queued up behind them.  Tile boundaries do not interrupt the stream.
  // DEEP: per slab r the A copies of slab r+2 and then the B copies of slab r+3 are issued; the wait in slab r+1
  // lets the most recent CB copies (those B copies) stay in flight: loads complete in order, so all older ones are done.
  constexpr int WAIT_N = DEEP ? CB : 0;
  if (DEEP) feedb_seek(0);
  feed_seek(0);
  {
    SlabCopy s0 = begin_slab(0, 0);
#pragma unroll
    for (int k = 0; k < NC; ++k) copy_k(s0, k);
    if (DEEP) {  // B slab 1 as well: from here on the B cursor is a slab ahead
      begin_b(s0, 1);
#pragma unroll
      for (int k = CA; k < NC; ++k) copy_k(s0, k);
    }
  }
  wait_vmcnt<0>();
  __syncthreads();
  SlabCopy sc = begin_slab(1, 2);
#pragma unroll
  for (int k = 0; k < NC / 2; ++k) copy_k(sc, k);
  i32x4_t fa[C::TM - 1], fa_last[2], fb[2][C::TN];
#pragma unroll
  for (int i = 0; i < C::TM - 1; ++i) fa[i] = load_a(smem + C::a_off(0), 0, i);
  fa_last[0] = load_a(smem + C::a_off(0), 0, C::TM - 1);
#pragma unroll
  for (int j = 0; j < C::TN; ++j) fb[0][j] = load_b(smem + C::b_off(0), 0, j);
  int ring = 0;
  int ring3 = 0;  // ring % 3 (DEEP: the B buffer of the current slab)

  // The accumulators start at zero and every epilogue path below clears each strip's registers right after it
  // has converted them: those moves then sit in the epilogue's LDS waits instead of in front of the next tile's
  // first multiplies.
  f32x4_t acc[C::TM][C::TN];
#pragma unroll
  for (int i = 0; i < C::TM; ++i)
#pragma unroll
    for (int j = 0; j < C::TN; ++j)
#pragma unroll
      for (int e = 0; e < 4; ++e) acc[i][j][e] = 0.f;
  auto clear_strip = [&](int i) {
#pragma unroll
    for (int j = 0; j < C::TN; ++j)
#pragma unroll
      for (int e = 0; e < 4; ++e) acc[i][j][e] = 0.f;
  };

  for (int tile_pos = 0, tile_id; (tile_id = tile_at(tile_pos)) >= 0; ++tile_pos) {
    const Tile cur = tile_id == seen_id ? seen : sched_tile<C::BM, C::BN>(p, sched, tile_id);
    const int kt_n = __builtin_amdgcn_readfirstlane(slabs_of(cur));

    // Half a K step: the multiplies of row blocks [h TM/2, (h+1) TM/2) with fragment set `cur_set`.  Meanwhile
    // fragments of K step ks_next of the slab at s_next are read into the other set:
    //   READ_EARLY    B fragments and the last A fragment right after the first multiply, A fragment i after the
    //                 multiplies of row block i;
    //   READ_ROLL     A fragment i after the multiplies of row block i;
    //   READ_NONE     nothing (the slab to read from is not complete yet);
    //   READ_CATCH_UP as READ_EARLY, plus the A fragments that the preceding READ_NONE half left out.
    // Copies [k0, k0 + NC/2) of `sc` are issued between the multiplies when k0 >= 0 (SP1, SP2 above).
    enum { READ_EARLY, READ_ROLL, READ_NONE, READ_CATCH_UP };
    SlabCopy sc_next;
    auto half = [&](int cur_set, int h, const char* s_next, const char* sb_next, int ks_next, int mode, int k0, bool prepare = false) {
      const int nxt = cur_set ^ 1;
      constexpr int HM = C::TM / 2;
#pragma unroll
      for (int ii = 0; ii < HM; ++ii) {
        const int i = h * HM + ii;
        const i32x4_t a = i == C::TM - 1 ? fa_last[cur_set] : fa[i];
        // Column blocks are visited in snake order (0..TN-1, then TN-1..0): one operand register changes per
        // multiply instead of both at every row-block boundary, which is worth 6 % more flops per watt in a
        // register-only loop.
#pragma unroll
        for (int jj = 0; jj < C::TN; ++jj) {
          const int j = (i & 1) ? C::TN - 1 - jj : jj;
          acc[i][j] = Mma16<DT>::run(fb[cur_set][j], a, acc[i][j]);
          const int n = ii * C::TN + jj;
          if (n == 0 && (mode == READ_EARLY || mode == READ_CATCH_UP)) {
            __builtin_amdgcn_sched_barrier(0);
#pragma unroll
            for (int j2 = 0; j2 < C::TN; ++j2) fb[nxt][j2] = load_b(sb_next, ks_next, j2);
            fa_last[nxt] = load_a(s_next, ks_next, C::TM - 1);
            if (mode == READ_CATCH_UP) {
#pragma unroll
              for (int i2 = 0; i2 < HM; ++i2) fa[i2] = load_a(s_next, ks_next, i2);
            }
            __builtin_amdgcn_sched_barrier(0);
          }
          if (prepare && n == 1) sc_next = begin_slab(ring & 1, ring3);  // scalar work, under the multiplies just issued
          const int sp = k0 == 0 ? SP1 : SP2;
          if (k0 >= 0 && (n + 1) % sp == 0 && (n + 1) / sp <= NC / 2) {
            __builtin_amdgcn_sched_barrier(0);
            copy_k(sc, k0 + (n + 1) / sp - 1);
            __builtin_amdgcn_sched_barrier(0);
          }
        }
        if (mode != READ_NONE && i < C::TM - 1) {
          __builtin_amdgcn_sched_barrier(0);
          fa[i] = load_a(s_next, ks_next, i);
          __builtin_amdgcn_sched_barrier(0);
        }
      }
      __builtin_amdgcn_sched_barrier(0);
    };

    // A wave whose whole block of the tile lies beyond the group's rows (a group of at most BM / WM rows leaves
    // the lower waves without work) or beyond N multiplies nothing: it keeps its share of the copy stream and the
    // barriers going, leaves the matrix pipe to the wave it shares a SIMD with, and ends with the fragment reads
    // the next tile expects.  Its accumulators are zero and stay zero, and it has nothing to store.
    if (!QUANT && LAYOUT != LAYOUT_TN && (wm0 >= cur.rows || cur.n0 + wn0 >= p.N)) {
      for (int kt = 0; kt < kt_n; ++kt) {
#pragma unroll
        for (int k = NC / 2; k < NC; ++k) {
          copy_k(sc, k);
          __builtin_amdgcn_s_sleep(1);  // paced: the address unit's queue is shared with the working waves
        }
        sc_next = begin_slab(ring & 1, ring3);
        wait_vmcnt<WAIT_N>();
        __syncthreads();
        sc = sc_next;
#pragma unroll
        for (int k = 0; k < NC / 2; ++k) {
          copy_k(sc, k);
          __builtin_amdgcn_s_sleep(1);
        }
        ++ring;
        ring3 = ring3 == 2 ? 0 : ring3 + 1;
      }
      if (kt_n > 0) {
        const char* sn = smem + C::a_off(ring & 1);
        const char* sbn = smem + C::b_off(DEEP ? ring3 : (ring & 1));
#pragma unroll
        for (int i = 0; i < C::TM - 1; ++i) fa[i] = load_a(sn, 0, i);
        fa_last[0] = load_a(sn, 0, C::TM - 1);
#pragma unroll
        for (int j = 0; j < C::TN; ++j) fb[0][j] = load_b(sbn, 0, j);
      }
      continue;
    }

    for (int kt = 0; kt < kt_n; ++kt) {
      const int ring3n = ring3 == 2 ? 0 : ring3 + 1;
      const char* sa = smem + C::a_off(ring & 1);
      const char* sn = smem + C::a_off((ring + 1) & 1);
      const char* sba = smem + C::b_off(DEEP ? ring3 : (ring & 1));
      const char* sbn = smem + C::b_off(DEEP ? ring3n : ((ring + 1) & 1));
      half(0, 0, sa, sba, 1, READ_EARLY, NC / 2);
      half(0, 1, sa, sba, 1, READ_ROLL, -1, true);
      half(1, 0, sn, sbn, 0, READ_NONE, -1);
      wait_vmcnt<WAIT_N>();
      // queued: this tile's draw, where this wave has no copies in flight (the wait for the counter's answer then
      // waits for nothing else) and in front of the barrier: wave 0 is the first-served wave of its SIMD and tends
      // to reach the barrier early, so part of the answer's latency falls into time it would spend waiting there
      if (LAYOUT == LAYOUT_TN && queued && kt == 0 && threadIdx.x == 0) draw_from(tile_pos + 1);
      __syncthreads();
      sc = sc_next;
      half(1, 1, sn, sbn, 0, READ_CATCH_UP, 0);
      ++ring;
      ring3 = ring3n;
    }

    // Epilogue.  A lane owns row l16 and columns 16 j + 4 lg + (0..3) of each 16-row block i: transpose one
    // 16-row strip (all of the wave's columns) at a time through the wave's LDS staging so that global stores
    // are 16 bytes per lane and cover whole row segments.  The lane id passes through an opaque statement so
    // that the address arithmetic below is redone per tile instead of being hoisted out of the tile loop, where
    // it would occupy registers (or spill) across the multiplies.
    int el = lane;
    asm volatile("" : "+v"(el));
    const int e16 = el & 15, eg = el >> 4;
    char* const stage_c = smem + C::EPI_OFF + wave * C::EPI_WAVE_BYTES;
    const int64_t c_row0 = (LAYOUT == LAYOUT_TN) ? ((int64_t)cur.g * p.m_total + cur.row0) : cur.row0;
    if (QUANT) {
      // Fused 1x128 quantisation, bit-identical to rounding the tile to the 16-bit type and quantising that:
      // round, take each row's |max| over the wave's columns (own 16 values, then the three lanes that hold the
      // rest of the row), exchange with the neighbouring wave that holds the other half of the 128-column block,
      // scale, convert, store codes and one scale per (row, block).  A 128-column block never straddles tiles
      // (N and the tile width are multiples of 128), and the maxima are exact 16-bit values, so they travel as
      // 16 bits.
      static_assert(!QUANT || (C::BN / C::WN == 64 && C::WN % 2 == 0), "two waves per 128-column block");
      uint16_t* const rowmax = (uint16_t*)(smem + C::QMAX_OFF);
      const int wn = wave % C::WN;
      const float fmax_ = p.q_fmt == DT_E4M3 ? 448.0f : 57344.0f;
      float rmax[C::TM];
#pragma unroll
      for (int i = 0; i < C::TM; ++i) {
        float m = 0.f;
#pragma unroll
        for (int j = 0; j < C::TN; ++j)
#pragma unroll
          for (int e = 0; e < 4; ++e) {
            const float v = round16<DT>(acc[i][j][e]);
            acc[i][j][e] = v;
            m = fmaxf(m, fabsf(v));
          }
        m = fmaxf(m, __shfl_xor(m, 16, 64));
        m = fmaxf(m, __shfl_xor(m, 32, 64));
        rmax[i] = m;
        if (eg == 0) rowmax[wn * C::BM + wm0 + 16 * i + e16] = Out16<DT>::cvt(m);
      }
      __syncthreads();
      char* const q_tile = (char*)p.C + (c_row0 + wm0) * (int64_t)p.N + cur.n0 + wn0;  // 1-byte codes
      const int blk = (cur.n0 + wn0) >> 7;
      const int st_row = el >> 2, st_chunk = el & 3;  // 16 rows x 64 one-byte codes are staged: 4 chunks of 16 bytes per row
      const bool col_ok = cur.n0 + wn0 + st_chunk * 16 < p.N;
#pragma unroll
      for (int i = 0; i < C::TM; ++i) {
        const float other = from16<DT>(rowmax[(wn ^ 1) * C::BM + wm0 + 16 * i + e16]);
        const float amax = fmaxf(fmaxf(rmax[i], other), 1e-4f);
        const float mult = (1.0f / amax) * fmax_;  // torch evaluates `448.0 / amax` as reciprocal * 448
#pragma unroll
        for (int j = 0; j < C::TN; ++j) {
          const float a0 = acc[i][j][0] * mult, a1 = acc[i][j][1] * mult;
          const float a2 = acc[i][j][2] * mult, a3 = acc[i][j][3] * mult;
          uint32_t w;
          if (p.q_fmt == DT_E4M3) {
            w = __builtin_amdgcn_cvt_pk_fp8_f32(a0, a1, 0u, false);
            w = __builtin_amdgcn_cvt_pk_fp8_f32(a2, a3, w, true);
          } else {
            w = __builtin_amdgcn_cvt_pk_bf8_f32(a0, a1, 0u, false);
            w = __builtin_amdgcn_cvt_pk_bf8_f32(a2, a3, w, true);
          }
          *(uint32_t*)(stage_c + e16 * C::EPI_PITCH + 16 * j + 4 * eg) = w;
        }
        clear_strip(i);
        const i32x4_t v = *(const i32x4_t*)(stage_c + st_row * C::EPI_PITCH + st_chunk * 16);
        if (col_ok && wm0 + 16 * i + st_row < cur.rows)
          store_c((i32x4_t*)(q_tile + (int64_t)(16 * i + st_row) * p.N + st_chunk * 16), v, 0);  // 64-byte row segments: half lines do worse non-temporally
        const int row = wm0 + 16 * i + e16;
        if ((wn & 1) == 0 && eg == 0 && row < cur.rows && cur.n0 + wn0 < p.N)
          p.q_scales[(c_row0 + row) * p.q_rs + (int64_t)blk * p.q_bs] = amax / fmax_;
      }
      continue;
    }
    char* const c_tile = (char*)p.C + ((c_row0 + wm0) * (int64_t)p.N + cur.n0 + wn0) * 2;
    constexpr int CPS = 2 * C::TN;        // 16-byte chunks per staged row
    constexpr int PASSES = 16 * CPS / 64;  // wave-wide reads per strip
    static_assert(16 * CPS % 64 == 0, "a strip is read back by whole waves");
    // Tiles that lie wholly inside the output (all but the last row tile of a group and a ragged last column
    // tile) take a path without per-store bounds checks: a wave-uniform base per strip plus a 32-bit lane offset.
    const bool full = cur.rows >= C::BM && cur.n0 + C::BN <= p.N;
    if (full) {
      const uint64_t base = uniform64((uint64_t)c_tile);
      const uint32_t strip_bytes = (uint32_t)__builtin_amdgcn_readfirstlane(16 * p.N * 2);
      uint32_t voff[PASSES];
#pragma unroll
      for (int it = 0; it < PASSES; ++it) {
        const int idx = it * 64 + el, r = idx / CPS, ch = idx % CPS;
        voff[it] = (uint32_t)(r * p.N * 2 + ch * 16);
      }
#pragma unroll
      for (int i = 0; i < C::TM; ++i) {
#pragma unroll
        for (int j = 0; j < C::TN; ++j)
          *(uint2*)(stage_c + e16 * C::EPI_PITCH + (16 * j + 4 * eg) * 2) =
              pack4<DT>(acc[i][j][0], acc[i][j][1], acc[i][j][2], acc[i][j][3]);
        clear_strip(i);
        const uint64_t strip = base + (uint64_t)i * strip_bytes;
#pragma unroll
        for (int it = 0; it < PASSES; ++it) {
          const int idx = it * 64 + el, r = idx / CPS, ch = idx % CPS;
          const i32x4_t v = *(const i32x4_t*)(stage_c + r * C::EPI_PITCH + ch * 16);
          store_c((i32x4_t*)(strip + voff[it]), v, p.store_nt);
        }
      }
      continue;
    }
#pragma unroll
    for (int i = 0; i < C::TM; ++i) {
#pragma unroll
      for (int j = 0; j < C::TN; ++j)
        *(uint2*)(stage_c + e16 * C::EPI_PITCH + (16 * j + 4 * eg) * 2) =
            pack4<DT>(acc[i][j][0], acc[i][j][1], acc[i][j][2], acc[i][j][3]);
      clear_strip(i);
#pragma unroll
      for (int it = 0; it < PASSES; ++it) {
        const int idx = it * 64 + el, r = idx / CPS, ch = idx % CPS;
        const i32x4_t v = *(const i32x4_t*)(stage_c + r * C::EPI_PITCH + ch * 16);
        if (cur.n0 + wn0 + ch * 8 < p.N && wm0 + 16 * i + r < cur.rows)
          store_c((i32x4_t*)(c_tile + ((int64_t)(16 * i + r) * p.N + ch * 8) * 2), v, p.store_nt);
      }
    }
  }
  if (LAYOUT == LAYOUT_TN && queued && threadIdx.x == 0) sched_queue_finish(p.queue);
  wait_vmcnt<0>();  // the trailing zero-length copies still write LDS: let them finish before the wave ends
}

template <class C, int DT, int LAYOUT, bool QUANT>
__global__ __launch_bounds__(C::THREADS) void gemm_fast_kernel(const GemmParams p) {
  extern __shared__ __attribute__((aligned(1024))) char smem[];
  sched_init<C::BM>(p, *reinterpret_cast<SchedTableT<kFastMaxGroups>*>(smem + C::SCHED_OFF));
  gemm_fast_body<C, DT, LAYOUT, QUANT, C::SCHED_OFF>(p);
}

// Several tile configurations in one kernel, chosen per launch from the group sizes, which only the device knows:
//   * the narrow tiles (half the columns) when all of them fit into a single round of the persistent workgroups
//     -- twice as many workgroups then have work, and a narrow tile costs about 0.7 of a wide one;
//   * otherwise, when the groups are small (the launch streams weights), the weight-streaming configuration
//     CS -- 128-row tiles and a ring of three B slabs whose copies run a slab further ahead, i.e. twice the weight
//     bytes in flight per CU: 5-30 % faster there (up to 6 TB/s of weights).  A 128-row tile costs about 0.7 of a
//     256-row one, so CS runs when its rounds of the persistent workgroups, times 0.7, are no more than the wide
//     configuration's rounds (see sched_short_tiles_pay): groups of up to about 200 rows on average;
//   * the wide tiles otherwise.
// Wide and narrow use BM-row tiles, so one group table serves both; for CS the table's tile prefix is rebuilt for
// its tile height when it differs (some group above 128 rows; sched_init has computed it alongside).  The table sits where the wide configuration keeps
// it, past everything the others touch.  CS = void: no weight-streaming configuration (K-grouped).
template <class CW, class CN, class CS, int DT, int LAYOUT>
__global__ __launch_bounds__(CW::THREADS) void gemm_fast_auto_kernel(const GemmParams p) {
  static_assert(CW::BM == CN::BM && CW::THREADS == CN::THREADS, "one group table, one launch shape");
  static_assert(CN::SMEM_BYTES <= CW::SCHED_OFF, "the narrow configuration must not reach the shared group table");
  extern __shared__ __attribute__((aligned(1024))) char smem[];
  auto& sched = *reinterpret_cast<SchedTableT<kFastMaxGroups>*>(smem + CW::SCHED_OFF);
  const int32_t half_tile0 = sched_init<CW::BM>(p, sched);
  bool stream = false;
  if constexpr (!std::is_void<CS>::value) {
    static_assert(CS::THREADS == CW::THREADS && CS::SCHED_OFF == CW::SCHED_OFF && CS::SMEM_BYTES <= CW::SMEM_BYTES,
                  "the weight-streaming configuration shares the launch shape and the group table's place");
    static_assert(CW::THREADS >= kFastMaxGroups && CS::BM * 2 == CW::BM, "sched_init's half-height prefix is CS's");
    stream = sched_short_tiles_pay<CW::BN>(p, sched);
  }
  if constexpr (!std::is_void<CS>::value) {
    // the four-wave kernel, launched in front of this one, has taken the launch (GemmParams::wide_gate)
    if (p.wide_gate == 2 && sched_wide_tiles_chosen<CW::BM, CW::BN>(p, sched)) return;
  }
  if (__builtin_expect(sched_num_tiles<CN::BM, CN::BN>(p, sched) > (int64_t)gridDim.x, 1)) {
    if constexpr (!std::is_void<CS>::value) {
      if (__builtin_expect(stream, 0)) {
        if (sched.pad_ != 0) {  // some group has more than one 128-row tile: the tile prefix for this tile height
          sched_use_half_height(p, sched, half_tile0);
        }
        gemm_fast_body<CS, DT, LAYOUT, false, CW::SCHED_OFF>(p);
        return;
      }
    }
    gemm_fast_body<CW, DT, LAYOUT, false, CW::SCHED_OFF>(p);
  } else {
    gemm_fast_body<CN, DT, LAYOUT, false, CW::SCHED_OFF>(p);
  }
}

template <class Kern>
int launch_kernel(Kern kern, int smem_bytes, int threads, bool& attr_done, const GemmParams& p, hipStream_t s, const char* what) {
  if (!attr_done) {
    if (hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize, smem_bytes) != hipSuccess)
      return check_launch("hipFuncSetAttribute(gemm_fast)");
    attr_done = true;
  }
  int grid = num_cus();
  if (p.grid_limit > 0 && p.grid_limit < grid) grid = p.grid_limit;
  hipLaunchKernelGGL(kern, dim3(grid), dim3(threads), smem_bytes, s, p);
  return check_launch(what);
}

// The attribute is per device: one flag per device ordinal and kernel (devices beyond the table set it every time).
inline bool& attr_flag(bool (&flags)[64]) {
  static thread_local bool unlisted;
  int dev = 0;
  (void)hipGetDevice(&dev);
  if (dev < 0 || dev >= 64) {
    unlisted = false;
    return unlisted;
  }
  return flags[dev];
}

template <class C, int DT, int LAYOUT, bool QUANT>
int launch_cfg(const GemmParams& p, hipStream_t s) {
  static bool attr_set[64] = {false};
  return launch_kernel(gemm_fast_kernel<C, DT, LAYOUT, QUANT>, C::SMEM_BYTES, C::THREADS, attr_flag(attr_set), p, s, "gemm_fast");
}

template <class CW, class CN, class CS, int DT, int LAYOUT>
int launch_auto(const GemmParams& p, hipStream_t s) {
  static bool attr_set[64] = {false};
  return launch_kernel(gemm_fast_auto_kernel<CW, CN, CS, DT, LAYOUT>, CW::SMEM_BYTES, CW::THREADS, attr_flag(attr_set), p, s, "gemm_fast");
}

std::atomic<int> g_variant{0};

template <int DT, int LAYOUT>
int launch_variant(const GemmParams& p, hipStream_t s) {
  typedef FastCfg<256, 256, 2, 4> Wide;
  typedef FastCfg<256, 128, 2, 4> Narrow;
  typedef FastCfg<128, 256, 2, 4, 3> Stream;
  typedef typename std::conditional<LAYOUT == LAYOUT_TN, void, Stream>::type StreamOrNone;
  switch (g_variant.load()) {
    default:
    case 0: return launch_auto<Wide, Narrow, StreamOrNone, DT, LAYOUT>(p, s);
    case 1: return launch_cfg<Narrow, DT, LAYOUT, false>(p, s);
    case 2: return launch_cfg<Wide, DT, LAYOUT, false>(p, s);
    case 4:
      if constexpr (LAYOUT != LAYOUT_TN) return launch_cfg<Stream, DT, LAYOUT, false>(p, s);
      else return launch_auto<Wide, Narrow, void, DT, LAYOUT>(p, s);
  }
}

template <int DT>
int launch_layout(const GemmParams& p, int layout, hipStream_t s) {
  if (layout == LAYOUT_NT) return launch_variant<DT, LAYOUT_NT>(p, s);
  if (layout == LAYOUT_NN) return launch_variant<DT, LAYOUT_NN>(p, s);
  return launch_variant<DT, LAYOUT_TN>(p, s);
}

}  // namespace

void set_fast_variant(int v) { g_variant = v; }

bool fast_supported(const GemmParams& p, int dt, int layout) {
  if (dt != DT_BF16 && dt != DT_F16) return false;
  if (p.G > kFastMaxGroups) return false;
  if ((p.N & 7) != 0) return false;
  if (layout == LAYOUT_TN) {
    if (p.mode != MODE_KG) return false;
    if ((p.m_total & 7) != 0) return false;
    return p.m_total * 2 * 64 < (1ll << 30) && (int64_t)p.N * 2 * 64 < (1ll << 30);
  }
  if (p.mode != MODE_MG && p.mode != MODE_MG_PAD && p.mode != MODE_MASKED) return false;
  if (p.K < 8 || (p.K & 7) != 0) return false;
  // per-lane source offsets stay far below the out-of-range marker
  if ((int64_t)p.K * 2 * 256 >= (1ll << 30)) return false;
  if (layout == LAYOUT_NN && (int64_t)p.N * 2 * 64 >= (1ll << 30)) return false;
  return layout == LAYOUT_NT || layout == LAYOUT_NN;
}

// Fused-quantisation launches: M-grouped NT / NN with N a multiple of 128 (see fast_quant_supported).
int launch_fast_16bit_quant(const GemmParams& p, int dt, int layout, hipStream_t s) {
  typedef FastCfg<256, 256, 2, 4> Cfg;
  if (dt == DT_BF16)
    return layout == LAYOUT_NT ? launch_cfg<Cfg, DT_BF16, LAYOUT_NT, true>(p, s) : launch_cfg<Cfg, DT_BF16, LAYOUT_NN, true>(p, s);
  return layout == LAYOUT_NT ? launch_cfg<Cfg, DT_F16, LAYOUT_NT, true>(p, s) : launch_cfg<Cfg, DT_F16, LAYOUT_NN, true>(p, s);
}

bool fast_quant_supported(const GemmParams& p, int dt, int layout) {
  if (layout != LAYOUT_NT && layout != LAYOUT_NN) return false;
  if (p.mode != MODE_MG && p.mode != MODE_MG_PAD) return false;
  if ((p.N & 127) != 0) return false;
  return fast_supported(p, dt, layout);
}

int launch_fast_16bit(const GemmParams& p, int dt, int layout, hipStream_t s) {
  if (dt == DT_BF16) return launch_layout<DT_BF16>(p, layout, s);
  return launch_layout<DT_F16>(p, layout, s);
}

}  // namespace tgg
