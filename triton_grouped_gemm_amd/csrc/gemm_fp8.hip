// Tuned FP8 (OCP e4m3fn / e5m2) grouped GEMM kernels for gfx950, K-contiguous operands.
//
// Same skeleton as the 16-bit kernels (persistent grouped tiles, one continuous direct-to-LDS slab
// stream across tiles, swizzled LDS, copies interleaved with multiplies, staged epilogue); a slab is
// 128 bytes = 128 K values of every row, i.e. exactly one 128-wide scale block.  The contraction runs
// on v_mfma_f32_16x16x128_f8f6f4: one multiply per 16x16 output block and slab, operands swapped as in the
// 16-bit kernels (a lane ends up with 4 consecutive columns of one row).  The shape is a power decision: with all
// CUs busy on random operands it buys about 9 % more flops per watt than 32x32x64.
//
//   EPI_BLOCK    out[r,n] = sum_kb (sum_{k in kb} a[r,k] b[g,n,k]) * sa[kb,r] * sb[g,n/128,kb]
//                Every slab is contracted into a fresh partial accumulator that is then folded into
//                the running fp32 accumulator with the slab's scale product (one VALU FMA per
//                element per 128 of K, overlapped with the next MFMAs).  The activation scales of
//                the slab's 256 rows travel with the slab (one extra 4-byte-per-lane LDS copy); the
//                weight scale is one scalar per wave and slab.
//   EPI_CHANNEL  out[r,n] = (sum_k a[r,k] b[g,n,k]) * scale_m[r] * scale_n[g*N + n], applied once in
//                the epilogue; used M-grouped and K-grouped (per-group token range along K).
#include "fast_common.hpp"
#include "launch.hpp"
#include <atomic>

namespace tgg {

namespace {

enum : int { EPI_CHANNEL = 1, EPI_BLOCK = 2 };
constexpr int BKB = 128;  // K depth of a slab in fp8 values (= bytes)

// One copy of 4 bytes per lane global -> LDS (destination m0 + lane * 4; s_nop 0 as in copy_b128_to_lds).
TGG_DEV void copy_b32_to_lds(i32x4_t rsrc, uint32_t lds_addr, int voff) {
  asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tbuffer_load_dword %1, %2, 0 offen lds" : : "s"(lds_addr), "v"(voff), "s"(rsrc) : "memory", "m0");
}

// BST: slab buffers of the B operand.  2: the A slab, the B slab and the activation scales of a stage sit together, two
// stages.  3 (the weight-streaming configuration, see gemm_fast.hip): A slabs and scales keep two buffers, the B
// slabs get a ring of three of their own and their copies run a slab further ahead.
template <int BM_, int BN_, int WM_, int WN_, int BST_ = 2>
struct Fp8Cfg {
  static constexpr int BM = BM_, BN = BN_, WM = WM_, WN = WN_, BST = BST_;
  static constexpr int NWAVES = WM * WN;
  static constexpr int THREADS = NWAVES * 64;
  static constexpr int A_BYTES = BM * 128, B_BYTES = BN * 128;
  static constexpr int SA_BYTES = BM * 4 + 256;  // activation scales of the slab's rows + a sink for spare waves' copies
  static constexpr int STAGE_BYTES = A_BYTES + B_BYTES + SA_BYTES;
  static constexpr int NI_A = A_BYTES / 1024, NI_B = B_BYTES / 1024;
  static constexpr int TM = BM / WM / 16, TN = BN / WN / 16;  // 16x16 blocks per wave
  static constexpr int EPI_PITCH = TN * 32 + 16;  // staged strip of 16 rows x (16 TN) 16-bit outputs: row pitch in bytes
  static constexpr int EPI_WAVE_BYTES = 16 * EPI_PITCH;
  static constexpr int SCHED_OFF = 2 * (A_BYTES + SA_BYTES) + BST * B_BYTES;
  // byte offsets of A buffer a (0, 1), its scales, and B buffer b (0 .. BST-1)
  static constexpr int a_off(int a) { return BST == 2 ? a * STAGE_BYTES : a * A_BYTES; }
  static constexpr int s_off(int a) { return BST == 2 ? a * STAGE_BYTES + A_BYTES + B_BYTES : 2 * A_BYTES + a * SA_BYTES; }
  static constexpr int b_off(int b) { return BST == 2 ? b * STAGE_BYTES + A_BYTES : 2 * (A_BYTES + SA_BYTES) + b * B_BYTES; }
  static constexpr int EPI_OFF = SCHED_OFF + (((int)sizeof(SchedTableT<kFastMaxGroups>) + 255) & ~255);
  static constexpr int SMEM_BYTES = EPI_OFF + NWAVES * EPI_WAVE_BYTES;
  static_assert(NI_A % NWAVES == 0 && NI_B % NWAVES == 0, "copies must divide evenly over waves");
  static_assert(NWAVES % 2 == 0 && BM / 64 <= NWAVES, "scale copies: one per wave");
  static_assert((BN / WN) <= 128, "a wave's columns must share one 128-wide weight scale block");
  static_assert(TM >= 4 && TM % 2 == 0 && TN >= 2, "the block schedule below alternates two A fragments");
  static_assert(SMEM_BYTES <= 160 * 1024, "LDS budget");
  static_assert(BST == 2 || BST == 3, "B slab buffers");
};

// s_waitcnt vmcnt(N) lgkmcnt(0): all LDS reads and all but the N most recent vector-memory operations are complete
template <int N> TGG_DEV void wait_vmcnt_lgkmcnt0() {
  static_assert(N >= 0 && N < 64, "vmcnt range");
  __builtin_amdgcn_s_waitcnt((N & 15) | ((N >> 4) << 14) | (7 << 4));
}

// FA / FB: 0 = e4m3fn, 1 = e5m2 (the cbsz / blgp format codes of the f8f6f4 MFMA).
// The whole kernel but for the group table, which the caller has built at byte SCHED_AT of the workgroup's LDS.
// IDLE: waves whose block of a tile has no rows or columns sit that tile out (see the tile loop).  A separate
// instantiation because the extra loop costs the plain one 1-1.5 % through register allocation alone.
template <class C, int FA, int FB, int EPI, int OUT, bool KGROUP, int SCHED_AT, bool IDLE>
TGG_DEV void gemm_fp8_body(const GemmParams& p) {
  typedef Operand<C::BM, true> OpA;
  typedef Operand<C::BN, true> OpB;
  constexpr bool BLOCK = EPI == EPI_BLOCK;
  constexpr bool DEEP = C::BST == 3;  // three B slab buffers, B copies a slab further ahead (see gemm_fast.hip)
  static_assert(!DEEP || !KGROUP, "the weight-streaming configuration is M-grouped");

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

  const int64_t ld = KGROUP ? p.k_total : (int64_t)p.K;  // bytes between consecutive rows of A and of B
  const int a_voff = OpA::lane_voff(lane, wave % OpA::NPAT, (int)ld);
  const int b_voff = OpB::lane_voff(lane, wave % OpB::NPAT, (int)ld);
  // K tail (see gemm_fast.hip): in a tile's last slab, chunks that start at or beyond K read as zero
  const int tail_chunks = KGROUP ? 0 : (p.K % BKB) / 16;
  const int a_voff_tail = OpA::lane_chunk(lane, wave % OpA::NPAT) >= tail_chunks ? kNoFetch : a_voff;
  const int b_voff_tail = OpB::lane_chunk(lane, wave % OpB::NPAT) >= tail_chunks ? kNoFetch : b_voff;
  // K-grouped: a group's last slab holds only the group's remaining tokens (a multiple of 16, see kg_gate); the
  // chunks beyond them belong to the next group and are not fetched
  const int a_chunk = OpA::lane_chunk(lane, wave % OpA::NPAT);
  const int b_chunk = OpB::lane_chunk(lane, wave % OpB::NPAT);
  const int kblocks = (p.K + 127) >> 7;
  const int nblocks = (p.N + 127) >> 7;

  // A fragment of the 16x16x128 multiply is 32 K values per lane.  Which 32 is free as long as both operands
  // agree (a dot product does not care about the order of its terms): lane group lg takes 16-byte chunks lg and
  // lg + 4 of the row's 128 bytes, so that each of the two reads has the lanes of a wave on four neighbouring
  // chunks, the access pattern of the 16-bit kernels.  Chunks 2 lg and 2 lg + 1 (the instruction's nominal K
  // order) collide in the LDS banks: 3.2 conflict cycles per read and 1.6 % slower overall.
  const int fsw = (l16 / 2) % 8;
  int rd[2];
#pragma unroll
  for (int h = 0; h < 2; ++h) rd[h] = l16 * 128 + (((lg + 4 * h) ^ fsw) << 4);
  // the fragment of the 16-row block starting at LDS address q
  auto load_frag = [&](const char* q) -> i32x8_t {
    const i32x4_t lo = *(const i32x4_t*)(q + rd[0]);
    const i32x4_t hi = *(const i32x4_t*)(q + rd[1]);
    return __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
  };

  // Slab sequence of a tile in scalar registers (see gemm_fast.hip): next slab's start and remaining bytes
  // of A, B and (block scaling) of the tile rows' activation scales, which are stored [K/128, m_total].
  struct TileIo {
    uint64_t a_base, b_base, s_base;
    int a_left, b_left;  // operand windows stay below 2^30 bytes: 32-bit scalar bookkeeping
    int s_bytes, kt_n, issued;
    int k_left;  // K-grouped: bytes of the group's token range not yet issued
  };
  // Queued launches (K-grouped, see tile_at below and gemm_fast.hip) give the tiles of an empty group one slab of
  // nothing instead of none, so that the copy stream advances by exactly one tile per tile.
  const bool queued = KGROUP && p.queue != nullptr;
  auto slabs_of = [&](const Tile& t) -> int {
    if (!KGROUP) return (p.K + BKB - 1) / BKB;
    const int n = (int)((t.k1 - t.k0 + BKB - 1) / BKB);
    return queued && n == 0 ? 1 : n;
  };
  auto make_io = [&](const Tile& t) {
    TileIo io;
    const int64_t k0 = KGROUP ? t.k0 : 0;
    io.kt_n = __builtin_amdgcn_readfirstlane(slabs_of(t));
    const int a_rows = t.rows;  // only the tile's valid rows are fetched, the others read as zero
    const int n_left = p.N - t.n0;
    io.a_base = uniform64((uint64_t)p.A + (uint64_t)(t.row0 * ld + k0));
    io.a_left = __builtin_amdgcn_readfirstlane((int)((int64_t)a_rows * ld - k0));
    io.b_base = uniform64((uint64_t)p.B + (uint64_t)((KGROUP ? (int64_t)t.n0 : ((int64_t)t.g * p.N + t.n0)) * ld + k0));
    io.b_left = __builtin_amdgcn_readfirstlane((int)((int64_t)(n_left < C::BN ? n_left : C::BN) * ld - k0));
    io.s_base = BLOCK ? uniform64((uint64_t)(p.sa + t.row0)) : 0;
    io.s_bytes = BLOCK ? __builtin_amdgcn_readfirstlane(a_rows * 4) : 0;
    io.issued = 0;
    io.k_left = KGROUP ? __builtin_amdgcn_readfirstlane((int)(t.k1 - t.k0)) : 0;
    return io;
  };
  // Weight scales of this wave's column block for every slab of a tile: lane kb holds block kb.
  // This is an ordinary vector load, so the compiler waits for *all* outstanding vector memory
  // traffic at its first use; it is therefore fetched one tile ahead and first touched right after
  // a point where this wave has waited for everything anyway.
  // With the deep ring a wave never waits for *everything* (its newest B copies stay in flight), so there the
  // load is inline assembly as well: loads complete in order, and the value is first used a tile later, behind
  // several of the stream's own waits.  It loads into the variable's own register ("+v"): the compiler, which
  // takes the statement's result for available at once, then has no reason to copy it anywhere before it has arrived.
  auto load_sbv = [&](const Tile& t, float& dst) {
    const int64_t idx = ((int64_t)t.g * nblocks + ((t.n0 + wn0) >> 7)) * kblocks;
    if (DEEP && BLOCK) {
      const float* src = p.sb + idx + (lane < kblocks ? lane : 0);
      asm volatile("global_load_dword %0, %1, off" : "+v"(dst) : "v"(src) : "memory");
    } else {
      dst = (BLOCK && lane < kblocks) ? p.sb[idx + lane] : 0.f;
    }
  };

  // The copy stream (see gemm_fast.hip): slab q of the workgroup's whole slab sequence lives in buffer q % 2.
  // M-grouped: every XCD owns a contiguous range of tiles, as in the 16-bit kernels (measured +2 % over
  // interleaved sweeps); K-grouped: interleaved, since a tile's cost follows its group's token count.
  const TileWalk walk64 = sched_walk(num_tiles, !KGROUP && p.tile_split);
  struct { int first, end, stride; } walk = {(int)walk64.first, (int)walk64.end, (int)walk64.stride};
  // The workgroup's pos-th tile (-1 past its last one): the static walk, or, queued, ids drawn from the counter in
  // global memory by thread 0 and passed on through a ring of eight words in the group table's scan scratch: one
  // draw per tile, on through short tiles up to the first one of kLongTile slabs or kQueueAhead tiles ahead (the
  // protocol and why it is safe are described in gemm_fast.hip).
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
  // The multiplying loop looks every tile up one tile ahead (it needs the tile's weight scales early); the feed
  // reaches that tile later and reuses the lookup instead of repeating its chain of dependent LDS reads.
  Tile nt;
  int nt_id = -1;
  // DEEP: the B copies have a cursor of their own, one slab ahead of `feed` (which then serves A and the scales)
  TileIo feedb;
  Tile seen;          // queued launches: the tile the feed looked up last
  int seen_id = -1;
  int feedb_pos = 0;
  auto feedb_seek = [&](int pos) {
    feedb.kt_n = 0;
    feedb.issued = 0;
    feedb.a_base = feedb.b_base = feedb.s_base = (uint64_t)p.A;
    feedb.a_left = feedb.b_left = 0;
    feedb.s_bytes = 0;
    feedb.k_left = 0;
    for (int id; (id = tile_at(pos)) >= 0; ++pos) {
      const Tile tt = id == nt_id ? nt : sched_tile<C::BM, C::BN>(p, sched, id);
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
    feed.a_base = feed.b_base = feed.s_base = (uint64_t)p.A;
    feed.a_left = feed.b_left = 0;
    feed.s_bytes = 0;
    feed.k_left = 0;
    for (int id; (id = tile_at(pos)) >= 0; ++pos) {
      const Tile tt = id == nt_id ? nt : sched_tile<C::BM, C::BN>(p, sched, id);
      if (queued) {  // no look-ahead by the multiplying loop there: it reuses this lookup instead
        seen = tt;
        seen_id = id;
      }
      if (slabs_of(tt) > 0) {
        feed = make_io(tt);
        break;
      }
    }
    feed_pos = pos;
  };
  struct SlabCopy {
    i32x4_t ra, rb, rs;
    uint32_t base, base_s, base_b;  // LDS addresses of the A slab, its scales and the B slab
    bool tail, tail_b;  // the tile's last slab, cut short by K (DEEP: A and B are slabs of different numbers)
    int chunks; // K-grouped: 16-byte chunks of this slab that belong to the group (8 but for a group's last slab)
  };
  constexpr int CA = C::NI_A / C::NWAVES, CB = C::NI_B / C::NWAVES, CS = BLOCK ? 1 : 0, NC = CS + CA + CB;
  auto begin_b = [&](SlabCopy& sc, int buf_b) {  // DEEP: the next B slab of the B cursor, into B buffer buf_b
    const bool live = feedb.issued < feedb.kt_n;
    sc.rb = make_rsrc32(feedb.b_base, live ? feedb.b_left : 0);
    sc.base_b = (uint32_t)__builtin_amdgcn_readfirstlane((int)(smem_addr + C::b_off(buf_b)));  // wave-uniform: goes into m0
    sc.tail_b = tail_chunks != 0 && feedb.issued + 1 == feedb.kt_n;
    feedb.b_base += BKB;
    feedb.b_left -= BKB;
    feedb.issued += 1;
    if (live && feedb.issued >= feedb.kt_n) feedb_seek(feedb_pos + 1);
  };
  auto begin_slab = [&](int buf, int buf_b = 0) {
    SlabCopy sc;
    const bool live = feed.issued < feed.kt_n;
    sc.ra = make_rsrc32(feed.a_base, live ? feed.a_left : 0);
    sc.rs = make_rsrc32(feed.s_base, live ? feed.s_bytes : 0);
    sc.base = (uint32_t)__builtin_amdgcn_readfirstlane((int)(smem_addr + C::a_off(buf)));
    sc.base_s = (uint32_t)__builtin_amdgcn_readfirstlane((int)(smem_addr + C::s_off(buf)));
    sc.tail = tail_chunks != 0 && feed.issued + 1 == feed.kt_n;
    if (!DEEP) {
      sc.rb = make_rsrc32(feed.b_base, live ? feed.b_left : 0);
      sc.base_b = (uint32_t)__builtin_amdgcn_readfirstlane((int)(smem_addr + C::b_off(buf)));
      sc.tail_b = sc.tail;
    }
    sc.chunks = KGROUP ? (feed.k_left >= BKB ? 8 : (feed.k_left > 0 ? feed.k_left >> 4 : 0)) : 8;
    feed.k_left -= BKB;
    feed.a_base += BKB;
    feed.a_left -= BKB;
    feed.b_base += BKB;
    feed.b_left -= BKB;
    feed.s_base += (uint64_t)p.m_total * 4;
    feed.issued += 1;
    if (live && feed.issued >= feed.kt_n) feed_seek(feed_pos + 1);
    if (DEEP) begin_b(sc, buf_b);
    return sc;
  };
  auto copy_k = [&](const SlabCopy& sc, int k) {
    if (k < CS) {
      // activation scales of the slab's rows: wave w fetches rows 64 w .. 64 w + 63; spare waves issue an
      // out-of-range copy into a sink so that every wave has the same number of copies in flight
      const bool mine = wave * 64 < C::BM;
      copy_b32_to_lds(sc.rs, sc.base_s + (mine ? wave * 256 : C::BM * 4),
                      mine ? (wave * 64 + lane) * 4 : kNoFetch);
    } else if (k < CS + CA) {
      const int idx = wave + (k - CS) * C::NWAVES;  // wave-uniform
      const int v0 = KGROUP ? (a_chunk >= sc.chunks ? kNoFetch : a_voff) : (sc.tail ? a_voff_tail : a_voff);
      copy_b128_to_lds(sc.ra, sc.base + idx * 1024, v0 + idx * OpA::RPI * (int)ld);
    } else {
      const int idx = wave + (k - CS - CA) * C::NWAVES;
      const int v0 = KGROUP ? (b_chunk >= sc.chunks ? kNoFetch : b_voff) : (sc.tail_b ? b_voff_tail : b_voff);
      copy_b128_to_lds(sc.rb, sc.base_b + idx * 1024, v0 + idx * OpB::RPI * (int)ld);
    }
  };

  // Software pipeline.  A slab is TM x TN multiplies, one per 16x16 block, row block by row block.  The B
  // fragments of all column blocks stay in registers for the slab; the A fragment of row block i + 1 is read
  // during row block i (two registers sets alternate).  Before the last row block: wait for this wave's share of
  // the next slab, workgroup barrier, read the next slab's first A fragment; each of the last row block's
  // multiplies is followed by the read of the next slab's B fragment into the registers it has just used.  The
  // copies of the slab after the next one are issued one per multiply from the barrier on: the sooner they are
  // out, the longer they have to land before the next wait (one per two multiplies measured 3 % slower, two per
  // multiply 4 % slower: the address unit's queue is short, see gemm_fast.hip).
  // Block scaling: every multiply starts from zero and its result is folded into the accumulators, scaled, three
  // multiplies later.
  // DEEP: per slab the scale, A and then B copies go out, the B copies for a slab one further ahead; the wait lets
  // the CB most recent copies -- those B copies -- stay in flight (loads complete in order).
  constexpr int WAIT_N = DEEP ? CB : 0;
  constexpr int kFoldLag = C::TN >= 3 ? 3 : 2;  // block scaling: a product is folded in this many multiplies after its own
  static_assert(kFoldLag >= 1 && kFoldLag <= 3 && kFoldLag <= C::TN, "four product buffers; the carried products share the last row block's scale");
  if (DEEP) feedb_seek(0);
  feed_seek(0);
  {
    SlabCopy s0 = begin_slab(0, 0);
#pragma unroll
    for (int k = 0; k < NC; ++k) copy_k(s0, k);
    if (DEEP) {  // B slab 1 as well: from here on the B cursor is a slab ahead
      begin_b(s0, 1);
#pragma unroll
      for (int k = CS + CA; k < NC; ++k) copy_k(s0, k);
    }
  }
  wait_vmcnt<0>();
  __syncthreads();
  SlabCopy sc = begin_slab(1, 2);
  // copy k of `sc`, if there is one (k is a compile-time constant at every call site)
  auto copy_at = [&](int k) {
    if (k < NC) {
      __builtin_amdgcn_sched_barrier(0);
      copy_k(sc, k);
      __builtin_amdgcn_sched_barrier(0);
    }
  };
#pragma unroll
  for (int k = 0; k < C::TN; ++k) copy_at(k);
  i32x8_t fb[C::TN], fa[2];
#pragma unroll
  for (int j = 0; j < C::TN; ++j) fb[j] = load_frag(smem + C::b_off(0) + (wn0 + 16 * j) * 128);
  fa[0] = load_frag(smem + C::a_off(0) + wm0 * 128);
  int ring = 0;
  int ring3 = 0;  // ring % 3 (DEEP: the B buffer of the current slab)

  float sbv_next = 0.f;
  if (tile_at(0) >= 0) {
    nt = sched_tile<C::BM, C::BN>(p, sched, tile_at(0));
    nt_id = tile_at(0);
    load_sbv(nt, sbv_next);
    if (DEEP && BLOCK) wait_vmcnt<0>();  // there the load is not the compiler's to wait for, and the first slab reads it
  }
  // The accumulators start at zero and the epilogue clears every strip right after it has converted it.
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
    const Tile cur = (!queued || tile_id == nt_id) ? nt : (tile_id == seen_id ? seen : sched_tile<C::BM, C::BN>(p, sched, tile_id));
    const int kt_n = __builtin_amdgcn_readfirstlane(slabs_of(cur));
    float sbv = sbv_next;
    // (queued launches look nothing up ahead here: the next id may not be drawn yet, and they need no weight scales)
    if (const int next_id = queued ? -1 : tile_at(tile_pos + 1); next_id >= 0) {
      nt = sched_tile<C::BM, C::BN>(p, sched, next_id);
      nt_id = next_id;
      load_sbv(nt, sbv_next);
    }

    // A wave whose block of the tile has no rows (groups of at most BM / WM rows) or no columns sits the tile
    // out, as in gemm_fast.hip: it keeps its copies and the barriers going and reads the fragments the next tile
    // starts with.
    if (IDLE && !KGROUP && (wm0 >= cur.rows || cur.n0 + wn0 >= p.N)) {
      for (int kt = 0; kt < kt_n; ++kt) {
#pragma unroll
        for (int k = C::TN; k < NC; ++k) {
          copy_at(k);
          __builtin_amdgcn_s_sleep(1);  // paced: the address unit's queue is shared with the working waves
        }
        const SlabCopy scn = begin_slab(ring & 1, ring3);
        wait_vmcnt<WAIT_N>();
        if (BLOCK) asm volatile("" : "+v"(sbv_next));
        __syncthreads();
        sc = scn;
#pragma unroll
        for (int k = 0; k < C::TN; ++k) {
          copy_at(k);
          __builtin_amdgcn_s_sleep(1);
        }
        ++ring;
        ring3 = ring3 == 2 ? 0 : ring3 + 1;
      }
      if (kt_n > 0) {
#pragma unroll
        for (int j = 0; j < C::TN; ++j) fb[j] = load_frag(smem + C::b_off(DEEP ? ring3 : (ring & 1)) + (wn0 + 16 * j) * 128);
        fa[0] = load_frag(smem + C::a_off(ring & 1) + wm0 * 128);
      }
      continue;
    }

    // block scaling: the products that are still to be folded in when a slab ends (those of its last kFoldLag
    // multiplies) are carried into the next slab
    f32x4_t part[4] = {{0.f, 0.f, 0.f, 0.f}, {0.f, 0.f, 0.f, 0.f}, {0.f, 0.f, 0.f, 0.f}, {0.f, 0.f, 0.f, 0.f}};
    float s_carry = 0.f;
    for (int kt = 0; kt < kt_n; ++kt) {
      const int ring3n = ring3 == 2 ? 0 : ring3 + 1;
      const char* sa = smem + C::a_off(ring & 1);                            // A slab of the current slab
      const char* sn = smem + C::a_off((ring + 1) & 1);                      // ... and of the next
      const char* sbn = smem + C::b_off(DEEP ? ring3n : ((ring + 1) & 1));   // B slab of the next slab
      // row scales of the slab: read here, multiplied with the weight scale only after the row block's first
      // multiply has been issued, so that the wait for the reads does not sit in front of the slab's first multiply
      float srow[C::TM];
      float sb_cur = 0.f;
      if (BLOCK) {
        sb_cur = __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, sbv), kt));
        const float* ss = (const float*)(smem + C::s_off(ring & 1)) + wm0 + l16;
#pragma unroll
        for (int i = 0; i < C::TM; ++i) srow[i] = ss[16 * i];
      }
      SlabCopy scn;
#pragma unroll
      for (int i = 0; i < C::TM; ++i) {
        __builtin_amdgcn_sched_barrier(0);
        if (i < C::TM - 1) {
          fa[(i + 1) & 1] = load_frag(sa + (wm0 + 16 * (i + 1)) * 128);
        } else {
          // this wave's share of the next slab has landed, and its reads of the current slab (the last A
          // fragment was requested a row block ago) are complete: after the barrier the buffer is overwritten
          wait_vmcnt_lgkmcnt0<WAIT_N>();
          if (BLOCK) asm volatile("" : "+v"(sbv_next));  // everything older than the newest B copies has landed: touching it costs no wait
          // queued: this tile's draw, where this wave has nothing in flight, in front of the barrier (gemm_fast.hip)
          if (KGROUP && queued && kt == 0 && threadIdx.x == 0) draw_from(tile_pos + 1);
          __syncthreads();
          sc = scn;
          fa[0] = load_frag(sn + wm0 * 128);
        }
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int jj = 0; jj < C::TN; ++jj) {
          // snake order over the column blocks, except that the last row block runs forward: its multiplies free
          // the B registers in the order in which the next slab's first row block needs them
          const int j = ((i & 1) && i != C::TM - 1) ? C::TN - 1 - jj : jj;
          const int n = i * C::TN + jj;
          if (BLOCK) {
            const f32x4_t zero = {0.f, 0.f, 0.f, 0.f};
            part[n & 3] = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(fb[j], fa[i & 1], zero, FB, FA, 0, 0, 0, 0);
          } else {
            acc[i][j] = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(fb[j], fa[i & 1], acc[i][j], FB, FA, 0, 0, 0, 0);
          }
          __builtin_amdgcn_sched_barrier(0);
          if (i == C::TM - 1) {
            copy_at(jj);
            fb[j] = load_frag(sbn + (wn0 + 16 * j) * 128);
          } else {
            if (n == C::TN * (C::TM - 2) + 1) scn = begin_slab(ring & 1, ring3);  // scalar work under a multiply
            // block-scaled: one copy per two multiplies.  One per multiply crowds the address unit's queue (the copies
            // of all waves come close together: 1.3 % slower), one per three or more delays the slab's last copies
            // (0.3-1.5 % slower).  Per-channel, with no folds between the multiplies, the copies come closer still: one
            // per four multiplies (1 % over one per two, 2 % over one per multiply; one per six is back at one per two)
            if (BLOCK) { if (n % 2 == 0) copy_at(C::TN + n / 2); }
            else if (n % 4 == 0) copy_at(C::TN + n / 4);
          }
          if (BLOCK && jj == 0) srow[i] *= sb_cur;
          if (BLOCK) {
            // fold in the product of the multiply three back (kFoldLag; for n < 3 that is one of the previous slab's
            // last three, all of its last row block, scaled with that slab's last row scale).  A lag of two measured
            // 0.5 % slower, a lag of one 1.7 %; four product buffers, indexed by n % 4, allow up to three.  The empty asm statements pin the order (plain arithmetic is
            // otherwise free to drift, which keeps many products alive at once and spills).
            constexpr int NB = C::TM * C::TN;
            static_assert(NB % 4 == 0, "product buffers are numbered per slab");
            const int pn = (n + NB - kFoldLag) % NB;
            const int pi = pn / C::TN, pjj = pn % C::TN;
            const int pj = ((pi & 1) && pi != C::TM - 1) ? C::TN - 1 - pjj : pjj;
            const float sc_prev = n < kFoldLag ? s_carry : srow[pi];
            const int pb = pn & 3;
            asm volatile("" : "+v"(part[pb]));
#pragma unroll
            for (int e = 0; e < 4; ++e) acc[pi][pj][e] += part[pb][e] * sc_prev;
            asm volatile("" : "+v"(acc[pi][pj]));
          }
          __builtin_amdgcn_sched_barrier(0);
        }
      }
      if (BLOCK) s_carry = srow[C::TM - 1];
      ++ring;
      ring3 = ring3n;
    }
    if (BLOCK) {
#pragma unroll
      for (int q = kFoldLag - 1; q >= 0; --q) {
        constexpr int NB = C::TM * C::TN;
        const int pn = NB - 1 - q;
        const int pj = pn % C::TN;  // the last row block runs forward
#pragma unroll
        for (int e = 0; e < 4; ++e) acc[C::TM - 1][pj][e] += part[pn & 3][e] * s_carry;
      }
    }

    // Epilogue (see gemm_fast.hip): a lane owns row l16 and columns 16 j + 4 lg + (0..3) of each 16-row block i.
    // One 16-row strip of the wave's columns at a time goes through the wave's LDS staging and leaves as 16-byte
    // stores that cover whole row segments; per-channel scaling happens on the fp32 values before packing.
    // The lane id passes through an opaque statement so that the address arithmetic below is redone per tile
    // instead of being hoisted: hoisted values would have to live (spilled) across the register-tight main loop,
    // and every reload waits for all outstanding stores.
    int el = lane;
    asm volatile("" : "+v"(el));
    const int e16 = el & 15, eg = el >> 4;
    char* const stage = smem + C::EPI_OFF + wave * C::EPI_WAVE_BYTES;
    const int64_t c_row0 = KGROUP ? ((int64_t)cur.g * p.m_total + cur.row0) : cur.row0;
    char* const c_tile = (char*)p.C + ((c_row0 + wm0) * (int64_t)p.N + cur.n0 + wn0) * 2;
    constexpr int CPS = 2 * C::TN;         // 16-byte chunks per staged row
    constexpr int PASSES = 16 * CPS / 64;  // wave-wide reads per strip
    static_assert(16 * CPS % 64 == 0, "a strip is read back by whole waves");
    // channel scales of this lane's columns, fetched up front; those of its rows strip by strip
    f32x4_t cs[C::TN];
    const float* sm = nullptr;
    if (EPI == EPI_CHANNEL) {
      sm = p.scale_m + (KGROUP ? (int64_t)cur.g * p.scale_m_sg : 0) + cur.row0;
      const float* sn = p.scale_n + (int64_t)cur.g * p.N;
#pragma unroll
      for (int j = 0; j < C::TN; ++j) {
        const int n = cur.n0 + wn0 + 16 * j + 4 * eg;  // N is a multiple of 8: 4 columns are in or out together
        const f32x4_t zero = {0.f, 0.f, 0.f, 0.f};
        cs[j] = n < p.N ? *(const f32x4_t*)(sn + n) : zero;
      }
    }
#pragma unroll
    for (int i = 0; i < C::TM; ++i) {
      float rs = 1.f;
      if (EPI == EPI_CHANNEL) {
        const int m = wm0 + 16 * i + e16;
        rs = m < cur.rows ? sm[m] : 0.f;
      }
#pragma unroll
      for (int j = 0; j < C::TN; ++j) {
        float v[4];
#pragma unroll
        for (int e = 0; e < 4; ++e) v[e] = acc[i][j][e];
        if (EPI == EPI_CHANNEL) {
#pragma unroll
          for (int e = 0; e < 4; ++e) v[e] = v[e] * rs * cs[j][e];
        }
        *(uint2*)(stage + e16 * C::EPI_PITCH + (16 * j + 4 * eg) * 2) = pack4<OUT>(v[0], v[1], v[2], v[3]);
      }
      clear_strip(i);
#pragma unroll
      for (int it = 0; it < PASSES; ++it) {
        const int idx = it * 64 + el, r = idx / CPS, ch = idx % CPS;
        const i32x4_t v = *(const i32x4_t*)(stage + r * C::EPI_PITCH + ch * 16);
        if (cur.n0 + wn0 + ch * 8 < p.N && wm0 + 16 * i + r < cur.rows)
          store_c((i32x4_t*)(c_tile + ((int64_t)(16 * i + r) * p.N + ch * 8) * 2), v, p.store_nt);
      }
    }
  }
  if (KGROUP && queued && threadIdx.x == 0) sched_queue_finish(p.queue);
  wait_vmcnt<0>();  // the trailing zero-length copies still write LDS: let them finish before the wave ends
}

template <class C, int FA, int FB, int EPI, int OUT, bool KGROUP>
__global__ __launch_bounds__(C::THREADS) void gemm_fp8_kernel(const GemmParams p) {
  extern __shared__ __attribute__((aligned(1024))) char smem[];
  auto& sched = *reinterpret_cast<SchedTableT<kFastMaxGroups>*>(smem + C::SCHED_OFF);
  sched_init<C::BM>(p, sched);
  if (KGROUP && !sched_kg_gate_open(p, sched)) return;
  gemm_fp8_body<C, FA, FB, EPI, OUT, KGROUP, C::SCHED_OFF, false>(p);
}

// Several bodies in one kernel, chosen per launch on the device from the group sizes (see gemm_fast_auto_kernel in
// gemm_fast.hip): narrow tiles when all of them fit one round of the persistent workgroups; otherwise wide tiles,
// with the sit-out path when at least one tile in eight is at most half full (groups whose size modulo the tile
// height lies in the lower half: decode-sized groups), without it otherwise.
// A fourth body, the weight-streaming configuration CS (128-row tiles, three B slab buffers, see gemm_fast.hip), runs
// when the narrow tiles do not fit one round and its rounds, at 0.7 of a wide tile's cost each, are no more than the
// wide configuration's (sched_short_tiles_pay), without the sit-out path (measured: no gain there); the table's tile
// prefix is switched to its tile height when that differs.
template <class CW, class CN, class CS, int FA, int FB, int EPI, int OUT>
__global__ __launch_bounds__(CW::THREADS) void gemm_fp8_auto_kernel(const GemmParams p) {
  static_assert(CW::BM == CN::BM && CW::THREADS == CN::THREADS, "one group table, one launch shape");
  static_assert(CN::SMEM_BYTES <= CW::SCHED_OFF, "the narrow configuration must not reach the shared group table");
  static_assert(CS::THREADS == CW::THREADS && CS::SCHED_OFF <= CW::SCHED_OFF && CS::SMEM_BYTES <= CW::SMEM_BYTES,
                "the weight-streaming configuration shares the launch shape and must not reach the group table");
  static_assert(CW::THREADS >= kFastMaxGroups && CS::BM * 2 == CW::BM, "one group per thread; sched_init's half-height prefix is CS's");
  extern __shared__ __attribute__((aligned(1024))) char smem[];
  auto& sched = *reinterpret_cast<SchedTableT<kFastMaxGroups>*>(smem + CW::SCHED_OFF);
  const int32_t half_tile0 = sched_init<CW::BM>(p, sched);
  int half_full = 0;
  if ((int)threadIdx.x < p.G) {
    const int r = sched.rows[threadIdx.x] & (CW::BM - 1);
    half_full = r >= 1 && r <= CW::BM / 2;
  }
  const int n_half_full = __syncthreads_count(half_full);
  const bool stream = sched_short_tiles_pay<CW::BN>(p, sched);
  const bool narrow = sched_num_tiles<CN::BM, CN::BN>(p, sched) <= (int64_t)gridDim.x;
  const bool sit_out = n_half_full * 8 >= sched.tile0[p.G];
  if (__builtin_expect(!narrow && !stream && !sit_out, 1))  // marked likely: the register allocator then favours this body's loops
    gemm_fp8_body<CW, FA, FB, EPI, OUT, false, CW::SCHED_OFF, false>(p);
  else if (narrow)
    gemm_fp8_body<CN, FA, FB, EPI, OUT, false, CW::SCHED_OFF, true>(p);
  else if (stream) {
    if (sched.pad_ != 0) {  // some group has more than one 128-row tile: the tile prefix for this tile height
      sched_use_half_height(p, sched, half_tile0);
    }
    gemm_fp8_body<CS, FA, FB, EPI, OUT, false, CW::SCHED_OFF, false>(p);
  }
  else
    gemm_fp8_body<CW, FA, FB, EPI, OUT, false, CW::SCHED_OFF, true>(p);
}

template <class Kern>
int launch_fp8_kernel(Kern kern, int smem_bytes, int threads, bool (&attr_set)[64], const GemmParams& p, hipStream_t s) {
  int dev = 0;
  (void)hipGetDevice(&dev);
  const bool listed = dev >= 0 && dev < 64;
  if (!listed || !attr_set[dev]) {
    if (hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize, smem_bytes) != hipSuccess)
      return check_launch("hipFuncSetAttribute(gemm_fp8)");
    if (listed) attr_set[dev] = true;
  }
  int grid = num_cus();
  if (p.grid_limit > 0 && p.grid_limit < grid) grid = p.grid_limit;
  hipLaunchKernelGGL(kern, dim3(grid), dim3(threads), smem_bytes, s, p);
  return check_launch("gemm_fp8");
}

typedef Fp8Cfg<256, 256, 2, 4> Fp8Wide;
typedef Fp8Cfg<256, 128, 2, 4> Fp8Narrow;
typedef Fp8Cfg<128, 256, 2, 4, 3> Fp8Stream;

std::atomic<int> g_fp8_variant{0};  // 0: chosen on the device (M-grouped), 1: narrow, 2: wide, 4: weight-streaming configuration

// M-grouped launches choose the tile width on the device; K-grouped ones (tile count known to the host, tile cost
// set by the group's token count) use the wide tiles.
template <int FA, int FB, int EPI, int OUT, bool KGROUP>
int launch_fp8_cfg(const GemmParams& p, hipStream_t s) {
  static bool attr_auto[64] = {false}, attr_wide[64] = {false}, attr_narrow[64] = {false}, attr_stream[64] = {false};
  const int variant = g_fp8_variant.load();
  if constexpr (!KGROUP) {
    if (variant == 0)
      return launch_fp8_kernel(gemm_fp8_auto_kernel<Fp8Wide, Fp8Narrow, Fp8Stream, FA, FB, EPI, OUT>, Fp8Wide::SMEM_BYTES, Fp8Wide::THREADS, attr_auto, p, s);
    if (variant == 4)
      return launch_fp8_kernel(gemm_fp8_kernel<Fp8Stream, FA, FB, EPI, OUT, false>, Fp8Stream::SMEM_BYTES, Fp8Stream::THREADS, attr_stream, p, s);
    if (variant == 1)
      return launch_fp8_kernel(gemm_fp8_kernel<Fp8Narrow, FA, FB, EPI, OUT, false>, Fp8Narrow::SMEM_BYTES, Fp8Narrow::THREADS, attr_narrow, p, s);
  }
  return launch_fp8_kernel(gemm_fp8_kernel<Fp8Wide, FA, FB, EPI, OUT, KGROUP>, Fp8Wide::SMEM_BYTES, Fp8Wide::THREADS, attr_wide, p, s);
}

template <int FA, int FB, bool KGROUP>
int launch_channel_out(const GemmParams& p, int out_dt, hipStream_t s) {
  if (out_dt == DT_BF16) return launch_fp8_cfg<FA, FB, EPI_CHANNEL, DT_BF16, KGROUP>(p, s);
  if (out_dt == DT_F16) return launch_fp8_cfg<FA, FB, EPI_CHANNEL, DT_F16, KGROUP>(p, s);
  return set_error("unsupported output dtype code %d", out_dt);
}

template <bool KGROUP>
int launch_channel_fmt(const GemmParams& p, int ta, int tb, int out_dt, hipStream_t s) {
  if (ta == DT_E4M3 && tb == DT_E4M3) return launch_channel_out<0, 0, KGROUP>(p, out_dt, s);
  if (ta == DT_E4M3 && tb == DT_E5M2) return launch_channel_out<0, 1, KGROUP>(p, out_dt, s);
  if (ta == DT_E5M2 && tb == DT_E4M3) return launch_channel_out<1, 0, KGROUP>(p, out_dt, s);
  if (ta == DT_E5M2 && tb == DT_E5M2) return launch_channel_out<1, 1, KGROUP>(p, out_dt, s);
  return set_error("unsupported fp8 formats (%d, %d)", ta, tb);
}

}  // namespace

void set_fp8_variant(int v) { g_fp8_variant = v; }

// K-contiguous fp8 operands; K-grouped: token counts that are multiples of 16 (checked on the device, see kg_gate).
bool fast_fp8_supported(const GemmParams& p, bool block_scaled) {
  if (p.G > kFastMaxGroups) return false;
  if ((p.N & 7) != 0) return false;
  const bool kgroup = p.mode == MODE_KG_COUNT;
  if (kgroup) {
    if (block_scaled) return false;
    return (p.k_total % 16) == 0 && p.k_total * 256 < (1ll << 30);
  }
  if (p.mode != MODE_MG && p.mode != MODE_MG_PAD) return false;
  if (p.K < 16 || (p.K & 15) != 0) return false;
  if (block_scaled && (p.K + BKB - 1) / BKB > 64) return false;  // a tile's weight scales sit in the 64 lanes of one register
  return (int64_t)p.K * 256 < (1ll << 30);
}

int launch_fast_fp8_channel(const GemmParams& p, int ta, int tb, int out_dt, hipStream_t s) {
  if (p.mode == MODE_KG_COUNT) return launch_channel_fmt<true>(p, ta, tb, out_dt, s);
  return launch_channel_fmt<false>(p, ta, tb, out_dt, s);
}

// sa must be laid out [ceil(K/128), m_total] (row-block major) for this kernel.
int launch_fast_fp8_block(const GemmParams& p, hipStream_t s) {
  return launch_fp8_cfg<0, 0, EPI_BLOCK, DT_BF16, false>(p, s);
}

}  // namespace tgg
