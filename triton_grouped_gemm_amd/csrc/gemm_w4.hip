// Four-wave bf16/fp16 grouped GEMM kernel for gfx950: the large-problem path of the M-grouped entry points.
//
// One workgroup per CU, four waves, one per SIMD; tile 256x256, K slab 64; every wave owns a 128x128 block of
// 16x16x32 MFMA tiles with its 256 accumulator registers in AGPRs.  Against the eight-wave kernel (gemm_fast.hip,
// 128x64 per wave) a K step needs a third fewer LDS fragment reads per multiply, and with a single wave per SIMD
// there is nobody to interleave with, so the instruction order *is* the schedule: the slab loop is written as a
// sequence of inline-assembly statements (multiplies, fragment reads, direct-to-LDS copies, waits), which the
// compiler keeps in source order and only allocates registers for.  Measured in isolation on random operands
// (all 256 CUs, cache-resident source): 1.29 us per 256x256x64 slab against 1.41 us for the eight-wave loop.
//
// Per slab r (two LDS slab buffers, r % 2), per wave:
//   K step 0   64 multiplies on fragment set 0; meanwhile the 16 fragments of K step 1 are read into set 1
//   wait for those reads and for this wave's copies of slab r+1, workgroup barrier
//   K step 1   64 multiplies on set 1; meanwhile the fragments of slab r+1 / K step 0 are read into set 0 and
//              this wave's 16 copies of slab r+2 go out into the buffer of slab r
// Fragment reads are issued every third multiply, so the last one is a quarter of a K step old when it is
// waited for; copies every fourth multiply (the address unit takes 16 cycles per copy and its queue is short).
// The slabs of all of a workgroup's tiles form one stream, as in gemm_fast.hip.
//
// The epilogue is deferred: a tile's results are converted, staged and stored between the multiplies of the next
// tile's first K step (see "deferred epilogue" below), whose multiplies start from a zero addend instead of the
// accumulators.  With one wave per SIMD an epilogue of its own leaves the matrix pipe idle for 12 us per tile
// (headline 3.88 ms); deferred, conversion and staging disappear under the multiplies (what remains, 0.2 ms per
// launch, is the issue of the stores themselves): headline 3.43 ms, K = 768 shape 2.78 -> 2.09 ms.  The eight-wave
// kernel stands at 3.36 / 2.01 ms, so this kernel stays an opt-in path.
//
// What the compiler does not know about assembly statements, and how it is handled here:
//   * a fragment read's result arrives later: every register a read targets passes through the wait statement
//     ("+v") before a multiply may use it;
//   * the multiplies write AGPRs: compiled code (the epilogue's conversions) reads a block's accumulators no sooner
//     than 48 multiplies after the multiply that wrote them, except where a flush follows a tile directly: there the
//     last row block's accumulators pass through a statement of idle cycles first.  Accumulators are never the
//     target of a load.
#include "fast_common.hpp"
#include "launch.hpp"

namespace tgg {

namespace {

enum : int { W4_NT = 0, W4_NN = 1 };
constexpr int BK4 = 64;

template <int DT> TGG_DEV void mfma_acc(f32x4_t& acc, const i32x4_t& w, const i32x4_t& x) {
  if (DT == DT_BF16) asm volatile("v_mfma_f32_16x16x32_bf16 %0, %1, %2, %0" : "+a"(acc) : "v"(w), "v"(x));
  else asm volatile("v_mfma_f32_16x16x32_f16 %0, %1, %2, %0" : "+a"(acc) : "v"(w), "v"(x));
}

// The same with a zero addend: the first K step of a tile starts its accumulators afresh
template <int DT> TGG_DEV void mfma_new(f32x4_t& acc, const i32x4_t& w, const i32x4_t& x) {
  if (DT == DT_BF16) asm volatile("v_mfma_f32_16x16x32_bf16 %0, %1, %2, 0" : "=a"(acc) : "v"(w), "v"(x));
  else asm volatile("v_mfma_f32_16x16x32_f16 %0, %1, %2, 0" : "=a"(acc) : "v"(w), "v"(x));
}

// 16-byte fragment of a K-contiguous operand
template <int OFF> TGG_DEV void lds_read_b128(i32x4_t& dst, uint32_t addr) {
  asm volatile("ds_read_b128 %0, %1 offset:%2" : "=v"(dst) : "v"(addr), "n"(OFF) : "memory");
}
// fragment of a token-row operand: two transposing 8-byte reads (K 0..3 and 4..7 of the lane's column)
template <int OFF0, int OFF1> TGG_DEV void lds_read_tr(i32x4_t& dst, uint32_t addr) {
  i32x2_t lo, hi;
  asm volatile("ds_read_b64_tr_b16 %0, %2 offset:%3\n\tds_read_b64_tr_b16 %1, %2 offset:%4"
               : "=&v"(lo), "=&v"(hi) : "v"(addr), "n"(OFF0), "n"(OFF1) : "memory");
  dst = __builtin_shufflevector(lo, hi, 0, 1, 2, 3);
}

#define TGG_TIE8(f) "+v"(f[0]), "+v"(f[1]), "+v"(f[2]), "+v"(f[3]), "+v"(f[4]), "+v"(f[5]), "+v"(f[6]), "+v"(f[7])

struct W4Cfg {
  static constexpr int BM = 256, BN = 256, NWAVES = 4, THREADS = 256;
  static constexpr int A_BYTES = BM * BK4 * 2, B_BYTES = BN * BK4 * 2, STAGE_BYTES = A_BYTES + B_BYTES;
  static constexpr int NI_A = A_BYTES / 1024, NI_B = B_BYTES / 1024;
  static constexpr int TM = 8, TN = 8;                       // 16x16 blocks per wave: 128 x 128
  static constexpr int EPI_PITCH = 4 * 32 + 16;              // staged piece: 16 rows x 64 outputs, row pitch in bytes
  static constexpr int EPI_PIECE = 16 * EPI_PITCH;
  static constexpr int EPI_WAVE_BYTES = 2 * EPI_PIECE;       // two pieces alternate
  static constexpr int SCHED_OFF = 2 * STAGE_BYTES;
  static constexpr int EPI_OFF = SCHED_OFF + (((int)sizeof(SchedTableT<kFastMaxGroups>) + 255) & ~255);
  static constexpr int SMEM_BYTES = EPI_OFF + NWAVES * EPI_WAVE_BYTES;
  static_assert(SMEM_BYTES <= 160 * 1024, "LDS budget");
};

template <int DT, int LAYOUT>
__global__ __launch_bounds__(W4Cfg::THREADS) void gemm_w4_kernel(const GemmParams p) {
  typedef W4Cfg C;
  constexpr bool B_KMAJOR = LAYOUT == W4_NT;
  typedef Operand<C::BM, true> OpA;
  typedef Operand<C::BN, B_KMAJOR> OpB;

  extern __shared__ __attribute__((aligned(1024))) char smem[];
  auto& sched = *reinterpret_cast<SchedTableT<kFastMaxGroups>*>(smem + C::SCHED_OFF);
  sched_init<C::BM>(p, sched);
  const int num_tiles = (int)sched_num_tiles<C::BM, C::BN>(p, sched);

  const uint32_t smem_addr = (uint32_t)(uintptr_t)(lds_ptr_t)smem;
  const int lane = lane_id();
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int wm0 = (wave >> 1) * 128, wn0 = (wave & 1) * 128;
  const int l16 = lane & 15, lg = lane >> 4;

  const int a_ld = p.K * 2;                                     // global row pitches in bytes
  const int b_ld = (B_KMAJOR ? p.K : p.N) * 2;
  // per-lane source offsets of this wave's copies: copy k of an operand is instruction wave + 4 k of the slab, and
  // the swizzle pattern of an instruction repeats with period NPAT
  int a_voff[2], b_voff[2], a_voff_tail[2], b_voff_tail[2];
  const int tail_chunks = (p.K % BK4) / 8;  // K tail: chunks at or beyond K fetch nothing in a tile's last slab
#pragma unroll
  for (int q = 0; q < 2; ++q) {
    a_voff[q] = OpA::lane_voff(lane, (wave + 4 * q) % OpA::NPAT, a_ld);
    b_voff[q] = OpB::lane_voff(lane, (wave + 4 * q) % OpB::NPAT, b_ld);
    a_voff_tail[q] = OpA::lane_chunk(lane, (wave + 4 * q) % OpA::NPAT) >= tail_chunks ? kNoFetch : a_voff[q];
    b_voff_tail[q] = (B_KMAJOR && OpB::lane_chunk(lane, (wave + 4 * q) % OpB::NPAT) >= tail_chunks) ? kNoFetch : b_voff[q];
  }
  static_assert(OpA::NPAT <= 8 && OpB::NPAT <= 8 && 8 % OpA::NPAT == 0 && 8 % OpB::NPAT == 0, "two patterns per wave");

  // LDS addresses of the fragment reads relative to a slab buffer (see gemm_fast.hip for the layouts)
  uint32_t a_rd[2], b_rd[B_KMAJOR ? 2 : C::TN];
#pragma unroll
  for (int ks = 0; ks < 2; ++ks) a_rd[ks] = smem_addr + (wm0 + l16) * 128 + (((4 * ks + lg) ^ ((l16 / 2) % 8)) << 4);
  if (B_KMAJOR) {
#pragma unroll
    for (int ks = 0; ks < 2; ++ks)
      b_rd[ks] = smem_addr + C::A_BYTES + (wn0 + l16) * 128 + (((4 * ks + lg) ^ ((l16 / 2) % 8)) << 4);
  } else {
#pragma unroll
    for (int j = 0; j < C::TN; ++j) {
      const int e = l16 >> 2, c = l16 & 3;
      const int chunk = ((wn0 + 16 * j) / 8 + (c >> 1)) ^ (e * 4) ^ ((lg & 1) * 2);
      b_rd[B_KMAJOR ? 0 : j] = smem_addr + C::A_BYTES + (lg * 8 + e) * (C::BN * 2) + chunk * 16 + (c & 1) * 8;
    }
  }

  // ---- the copy stream (as in gemm_fast.hip) ---------------------------------------------------------------------
  struct TileIo {
    uint64_t a_base, b_base;
    int a_rem, b_rem, b_off;
    int kt_n, issued;
  };
  const int kt_all = (p.K + BK4 - 1) / BK4;
  const int64_t b_step = B_KMAJOR ? BK4 * 2 : (int64_t)BK4 * b_ld;
  auto make_io = [&](const Tile& t) {
    TileIo io;
    io.a_base = uniform64((uint64_t)p.A + (uint64_t)(t.row0 * a_ld));
    io.a_rem = __builtin_amdgcn_readfirstlane(t.rows * a_ld);  // only the tile's valid rows are fetched
    io.b_off = 0;
    if (B_KMAJOR) {
      const int n_left = p.N - t.n0;
      io.b_base = uniform64((uint64_t)p.B + (uint64_t)(((int64_t)t.g * p.N + t.n0) * b_ld));
      io.b_rem = __builtin_amdgcn_readfirstlane((n_left < C::BN ? n_left : C::BN) * b_ld);
    } else {
      io.b_base = uniform64((uint64_t)p.B + (uint64_t)((int64_t)t.g * p.K * b_ld + (int64_t)t.n0 * 2));
      io.b_rem = p.K;
      io.b_off = __builtin_amdgcn_readfirstlane(t.n0 * 2);
    }
    io.kt_n = kt_all;
    io.issued = 0;
    return io;
  };
  const TileWalk walk64 = sched_walk(num_tiles, p.tile_split != 0);
  struct { int first, end, stride; } walk = {(int)walk64.first, (int)walk64.end, (int)walk64.stride};
  TileIo feed;
  int feed_id;
  Tile seen;
  int seen_id = -1, seen_g = -1;
  auto feed_seek = [&](int id) {
    feed.kt_n = 0;
    feed.issued = 0;
    feed.a_base = feed.b_base = (uint64_t)p.A;
    feed.a_rem = feed.b_rem = feed.b_off = 0;
    if (id < walk.end) {
      seen = sched_tile<C::BM, C::BN>(p, sched, id, seen_g);
      seen_id = id;
      seen_g = seen.g;
      feed = make_io(seen);
    }
    feed_id = id;
  };
  struct SlabCopy {
    i32x4_t ra, rb;
    uint32_t base;
    bool tail;
  };
  constexpr int CA = C::NI_A / C::NWAVES, CB = C::NI_B / C::NWAVES, NC = CA + CB;
  static_assert(NC == 16, "one copy every fourth multiply of a K step");
  auto begin_slab = [&](int buf) {
    SlabCopy sc;
    const bool live = feed.issued < feed.kt_n;
    const int b_len = B_KMAJOR ? feed.b_rem : min(feed.b_rem, BK4) * b_ld - feed.b_off;
    sc.ra = make_rsrc32(feed.a_base, live ? feed.a_rem : 0);
    sc.rb = make_rsrc32(feed.b_base, live ? b_len : 0);
    sc.base = smem_addr + buf * C::STAGE_BYTES;
    sc.tail = tail_chunks != 0 && feed.issued + 1 == feed.kt_n;
    feed.a_base += BK4 * 2;
    feed.a_rem -= BK4 * 2;
    feed.b_base += b_step;
    feed.b_rem -= B_KMAJOR ? BK4 * 2 : BK4;
    feed.issued += 1;
    if (live && feed.issued >= feed.kt_n) feed_seek(feed_id + walk.stride);
    return sc;
  };
  auto copy_k = [&](const SlabCopy& sc, int k) {  // k is a compile-time constant at every call site
    if (k < CA) {
      const int idx = wave + k * C::NWAVES;
      copy_b128_to_lds(sc.ra, sc.base + idx * 1024, (sc.tail ? a_voff_tail[k & 1] : a_voff[k & 1]) + idx * OpA::RPI * a_ld);
    } else {
      const int kb = k - CA, idx = wave + kb * C::NWAVES;
      copy_b128_to_lds(sc.rb, sc.base + C::A_BYTES + idx * 1024,
                       (sc.tail ? b_voff_tail[kb & 1] : b_voff[kb & 1]) + idx * OpB::RPI * b_ld);
    }
  };

  // ---- fragments and accumulators --------------------------------------------------------------------------------
  i32x4_t fa[2][8], fb[2][8];
  f32x4_t acc[8][8];
#pragma unroll
  for (int i = 0; i < 8; ++i)
#pragma unroll
    for (int j = 0; j < 8; ++j) acc[i][j] = f32x4_t{0.f, 0.f, 0.f, 0.f};

  // read number q (0..15) of the fragments of K step KS of the slab at byte offset `buf_off`: B fragments first
  // (the next step needs all of them at once), then A fragments in the order of use
  auto read_frag = [&](auto KSc, auto Qc, i32x4_t (&sa)[8], i32x4_t (&sb)[8], uint32_t buf_off) {
    constexpr int KS = decltype(KSc)::value, Q = decltype(Qc)::value;
    if (Q < 8) {
      if (B_KMAJOR) lds_read_b128<Q * 2048>(sb[Q], b_rd[B_KMAJOR ? KS : 0] + buf_off);
      else lds_read_tr<KS * 32 * (C::BN * 2), KS * 32 * (C::BN * 2) + 4 * (C::BN * 2)>(sb[Q], b_rd[B_KMAJOR ? 0 : Q] + buf_off);
    } else {
      lds_read_b128<(Q - 8) * 2048>(sa[Q - 8], a_rd[KS] + buf_off);
    }
  };
  // One K step: 64 multiplies on set CUR (when MUL); the 16 fragments of K step NKS of the slab at nb_off go to the
  // other set; when COPY, this wave's 16 copies of `sc` go out.
  // Ends with the wait for those reads (and, when COPY is false, i.e. in front of the barrier, for this wave's copies
  // of the next slab): the registers the reads target pass through the wait statement, inside the same straight-line
  // code, before anything else may touch them.
  // ---- deferred epilogue ---------------------------------------------------------------------------------------------
  // A tile's results are stored during the first K step of the workgroup's next tile: with one wave per SIMD nothing
  // else would keep the matrix pipe busy while a wave converts and stores its 128x128 block.  A lane owns row l16 and
  // columns 16 j + 4 lg + (0..3) of each 16-row block i.  Strip i (one 16-row block, 128 columns) goes through the
  // wave's LDS staging as two pieces of 64 columns and leaves as 16-byte stores covering 128-byte row segments.
  // During the multiplies of row block i the blocks of strip i+1 are converted and staged one per multiply (their
  // accumulators are the next to be overwritten: the first K step multiplies with a zero addend) and strip i,
  // staged a row block earlier, is read back and stored.  The stores go through a buffer descriptor over the wave's
  // block that ends with its last valid row; lanes whose columns lie beyond N get an out-of-range offset: no branches.
  // Nothing pending = a descriptor of length zero.
  i32x4_t pend_rs = make_rsrc32(0, 0);
  int pend_cols = 0;
  bool pending = false;
  char* const stage = smem + C::EPI_OFF + wave * C::EPI_WAVE_BYTES;
  // per-lane staging addresses and output offset, recomputed where a first K step or a flush begins
  struct EpiLane { char* wr; const char* rd; int off; int ch8; };
  auto epi_lane = [&]() {
    int el = lane;
    asm volatile("" : "+v"(el));
    EpiLane e;
    e.wr = stage + (el & 15) * C::EPI_PITCH + (el >> 4) * 8;
    e.rd = stage + (el >> 3) * C::EPI_PITCH + (el & 7) * 16;
    e.off = ((el >> 3) * p.N + (el & 7) * 8) * 2;
    e.ch8 = (el & 7) * 8;
    return e;
  };
  // block (i, j) -> staging piece j / 4; not before this point in the instruction stream
  auto epi_cvt = [&](const EpiLane& e, int i, int j) {
    asm volatile("" : "+a"(acc[i][j]));
    *(uint2*)(e.wr + (j >> 2) * C::EPI_PIECE + (j & 3) * 32) = pack4<DT>(acc[i][j][0], acc[i][j][1], acc[i][j][2], acc[i][j][3]);
    asm volatile("" ::: "memory");
  };
  auto epi_read = [&](const EpiLane& e, int h, i32x4_t (&v)[2]) {
#pragma unroll
    for (int it = 0; it < 2; ++it) v[it] = *(const i32x4_t*)(e.rd + h * C::EPI_PIECE + it * 8 * C::EPI_PITCH);
    asm volatile("" ::: "memory");
  };
  auto epi_store = [&](const EpiLane& e, int i, int h, int it, const i32x4_t& v) {
    const int off = (64 * h + e.ch8 < pend_cols) ? e.off + ((16 * i + 8 * it) * p.N + 64 * h) * 2 : kNoFetch;
    i32x4_t rs;
#pragma unroll
    for (int q = 0; q < 4; ++q) rs[q] = __builtin_amdgcn_readfirstlane(pend_rs[q]);
    // the wait states in front cover a descriptor written by a vector instruction just before (the compiler does not
    // space what sits inside this statement), those behind it keep the data registers intact until the store has them
    asm volatile("s_nop 4\n\tbuffer_store_dwordx4 %0, %1, %2, 0 offen nt\n\ts_nop 1" : : "v"(v), "v"(off), "s"(rs) : "memory");
  };
  // everything that is pending, without multiplies to hide it under
  auto epi_flush = [&]() {
    if (pending) {
      // the last row block's multiplies may have just been issued: give them time before compiled code reads the registers
      asm volatile("s_nop 15\n\ts_nop 7" : "+a"(acc[7][0]), "+a"(acc[7][1]), "+a"(acc[7][2]), "+a"(acc[7][3]),
                   "+a"(acc[7][4]), "+a"(acc[7][5]), "+a"(acc[7][6]), "+a"(acc[7][7]));
      const EpiLane e = epi_lane();
#pragma unroll
      for (int i = 0; i < 8; ++i) {
#pragma unroll
        for (int j = 0; j < 8; ++j) epi_cvt(e, i, j);
#pragma unroll
        for (int h = 0; h < 2; ++h) {
          i32x4_t v[2];
          epi_read(e, h, v);
          epi_store(e, i, h, 0, v[0]);
          epi_store(e, i, h, 1, v[1]);
        }
      }
    }
    pending = false;
    pend_rs[2] = 0;
  };

  // EPI: the first K step of a tile -- multiplies start from zero, and the pending epilogue runs between them.
  auto kstep = [&](auto CURc, auto NKSc, auto MULc, auto COPYc, uint32_t nb_off, const SlabCopy& sc, auto EPIc) {
    constexpr int CUR = decltype(CURc)::value, NKS = decltype(NKSc)::value;
    constexpr bool MUL = decltype(MULc)::value, COPY = decltype(COPYc)::value, EPI = decltype(EPIc)::value;
    static_assert(!EPI || MUL, "the deferred epilogue rides on a multiplying K step");
    EpiLane e = {nullptr, nullptr, 0, 0};
    i32x4_t v0[2], v1[2];
    if (EPI) {
      e = epi_lane();
#pragma unroll
      for (int j = 0; j < 8; ++j) epi_cvt(e, 0, j);  // strip 0 has no multiplies in front of it to hide under
    }
#pragma unroll
    for (int i = 0; i < 8; ++i)
#pragma unroll
      for (int jj = 0; jj < 8; ++jj) {
        const int j = (i & 1) ? 7 - jj : jj;  // snake order: one operand register changes per multiply
        if (EPI) {
          if (jj == 0) epi_read(e, 0, v0);            // strip i, staged during the previous row block
          if (jj == 1) epi_read(e, 1, v1);
          if (i < 7) epi_cvt(e, i + 1, jj);           // its piece's read-back has been issued (jj = 0: piece 0, jj = 4: piece 1)
          if (jj == 3) epi_store(e, i, 0, 0, v0[0]);
          if (jj == 4) epi_store(e, i, 0, 1, v0[1]);
          if (jj == 5) epi_store(e, i, 1, 0, v1[0]);
          if (jj == 6) epi_store(e, i, 1, 1, v1[1]);
          mfma_new<DT>(acc[i][j], fb[CUR][j], fa[CUR][i]);
        } else if (MUL) {
          mfma_acc<DT>(acc[i][j], fb[CUR][j], fa[CUR][i]);
        }
        const int n = i * 8 + jj;
#define TGG_W4_RD(q) if (n + 1 == 3 * (q + 1)) read_frag(std::integral_constant<int, NKS>(), std::integral_constant<int, q>(), fa[CUR ^ 1], fb[CUR ^ 1], nb_off);
        TGG_W4_RD(0) TGG_W4_RD(1) TGG_W4_RD(2) TGG_W4_RD(3) TGG_W4_RD(4) TGG_W4_RD(5) TGG_W4_RD(6) TGG_W4_RD(7)
        TGG_W4_RD(8) TGG_W4_RD(9) TGG_W4_RD(10) TGG_W4_RD(11) TGG_W4_RD(12) TGG_W4_RD(13) TGG_W4_RD(14) TGG_W4_RD(15)
#undef TGG_W4_RD
        if (COPY && (n + 1) % 4 == 0) {
          copy_k(sc, (n + 1) / 4 - 1);
          if (!MUL) __builtin_amdgcn_s_sleep(1);  // a wave without multiplies must not crowd the address unit's queue
        }
      }
    if (COPY) asm volatile("s_waitcnt lgkmcnt(0)" : TGG_TIE8(fa[CUR ^ 1]), TGG_TIE8(fb[CUR ^ 1]) : : "memory");
    else asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)" : TGG_TIE8(fa[CUR ^ 1]), TGG_TIE8(fb[CUR ^ 1]) : : "memory");
  };
  typedef std::integral_constant<int, 0> I0;
  typedef std::integral_constant<int, 1> I1;
  typedef std::integral_constant<bool, true> Yes;
  typedef std::integral_constant<bool, false> No;

  // ---- prologue: slab 0 lands, its first fragments are read, slab 1 is requested -------------------------------------
  feed_seek(walk.first);
  {
    const SlabCopy s0 = begin_slab(0);
#pragma unroll
    for (int k = 0; k < NC; ++k) copy_k(s0, k);
  }
  wait_vmcnt<0>();
  __syncthreads();
  {
    const SlabCopy s1 = begin_slab(1);
#pragma unroll
    for (int k = 0; k < NC; ++k) copy_k(s1, k);
  }
  {
    SlabCopy none;
    kstep(I1(), I0(), No(), No(), 0u, none, No());  // reads K step 0 of buffer 0 into set 0, multiplies nothing, waits for everything
  }
  int ring = 0;

  for (int tile_id = walk.first; tile_id < walk.end; tile_id += walk.stride) {
    const Tile cur = tile_id == seen_id ? seen : sched_tile<C::BM, C::BN>(p, sched, tile_id);
    // a wave whose block of the tile has no rows or no columns multiplies nothing and stores nothing
    const bool active = wm0 < cur.rows && cur.n0 + wn0 < p.N;
    if (!active) epi_flush();  // no multiplies in this tile to hide the pending stores under
    // one slab; FIRST: the tile's first, whose first K step starts the accumulators afresh and carries the epilogue
    auto slab = [&](auto FIRST) {
      const uint32_t cur_off = (ring & 1) * C::STAGE_BYTES, nxt_off = C::STAGE_BYTES - cur_off;
      const SlabCopy sc = begin_slab(ring & 1);  // descriptors of the slab after the next one, into the current slab's buffer
      if (active) kstep(I0(), I1(), Yes(), No(), cur_off, sc, FIRST);
      else kstep(I0(), I1(), No(), No(), cur_off, sc, No());
      // set 1 is complete, this wave has read all it needs of the current slab, its copies of the next slab have landed
      asm volatile("s_barrier" ::: "memory");
      if (active) kstep(I1(), I0(), Yes(), Yes(), nxt_off, sc, No());
      else kstep(I1(), I0(), No(), Yes(), nxt_off, sc, No());
      ++ring;
    };
    slab(Yes());
    for (int kt = 1; kt < kt_all; ++kt) slab(No());
    if (!active) continue;
    // what the next tile's first K step (or a flush) will store
    const int rows_left = cur.rows - wm0;
    pend_rs = make_rsrc32((uint64_t)p.C + (uint64_t)(((cur.row0 + wm0) * (int64_t)p.N + cur.n0 + wn0) * 2),
                          (rows_left < 128 ? rows_left : 128) * p.N * 2);
    pend_cols = __builtin_amdgcn_readfirstlane(p.N - cur.n0 - wn0);
    pending = true;
  }
  epi_flush();
  wait_vmcnt<0>();  // trailing zero-length copies still write LDS
}

template <int DT, int LAYOUT>
int launch_w4(const GemmParams& p, hipStream_t s) {
  static bool attr_set[64] = {false};
  int dev = 0;
  (void)hipGetDevice(&dev);
  const bool listed = dev >= 0 && dev < 64;
  auto kern = gemm_w4_kernel<DT, LAYOUT>;
  if (!listed || !attr_set[dev]) {
    if (hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize, W4Cfg::SMEM_BYTES) != hipSuccess)
      return check_launch("hipFuncSetAttribute(gemm_w4)");
    if (listed) attr_set[dev] = true;
  }
  int grid = num_cus();
  if (p.grid_limit > 0 && p.grid_limit < grid) grid = p.grid_limit;
  hipLaunchKernelGGL(kern, dim3(grid), dim3(W4Cfg::THREADS), W4Cfg::SMEM_BYTES, s, p);
  return check_launch("gemm_w4");
}

}  // namespace

// The four-wave kernel takes M-grouped launches (rows contiguous or padded) whose tile count is large whatever the
// group sizes turn out to be: at least ceil(m_total / 256) row tiles.  Smaller launches stay with the eight-wave
// kernels, which choose narrower tiles on the device.
bool w4_supported(const GemmParams& p, int dt, int layout, bool any_size) {
  if (dt != DT_BF16 && dt != DT_F16) return false;
  if (layout != W4_NT) return false;
  if (p.mode != MODE_MG && p.mode != MODE_MG_PAD) return false;
  if (p.q_fmt != 0 || p.G > kFastMaxGroups) return false;
  if ((p.N & 7) != 0 || p.K < 8 || (p.K & 7) != 0) return false;
  if ((int64_t)p.K * 2 * 256 >= (1ll << 30)) return false;
  if (any_size) return true;
  int grid = num_cus();
  if (p.grid_limit > 0 && p.grid_limit < grid) grid = p.grid_limit;
  const int64_t row_tiles = (p.m_total + 255) / 256;
  const int64_t narrow_tiles = row_tiles * ((p.N + 127) / 128);
  return narrow_tiles > 4 * (int64_t)grid;
}

int launch_w4_16bit(const GemmParams& p, int dt, int layout, hipStream_t s) {
  if (dt == DT_BF16) return launch_w4<DT_BF16, W4_NT>(p, s);
  return launch_w4<DT_F16, W4_NT>(p, s);
}

}  // namespace tgg
