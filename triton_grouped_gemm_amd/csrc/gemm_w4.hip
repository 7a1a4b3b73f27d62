// Four-wave bf16/fp16 grouped GEMM kernel for gfx950: the large-problem path of the M-grouped and masked entry points
// (B as [G, N, K], or as [G, K, N] with N a multiple of 256).
//
// One workgroup per CU, four waves, one per SIMD; tile 256x256, K slab 64; every wave owns a 128x128 block of
// 16x16x32 MFMA tiles with its 256 accumulator registers in AGPRs.  Against the eight-wave kernel (gemm_fast.hip,
// 128x64 per wave) a K step needs a third fewer LDS fragment reads per multiply.  With a single wave per SIMD there
// is nobody to interleave with, so the instruction order *is* the schedule: the slab loop is a sequence of
// inline-assembly statements (multiplies, fragment reads, copies, waits), which the compiler keeps in source order and
// only allocates registers for.  What the order has to respect (measured with a stream of multiplies and one kind
// of instruction between them): a wave issues in order and a multiply keeps the matrix pipe busy for 16 cycles, so
// one or two other instructions between two multiplies cost nothing, three or four cost 4-10 cycles of pipe time,
// and a 16-byte-per-lane LDS write costs 13 cycles on its own (33 next to fragment reads).  Hence: never more than
// two instructions in a gap of the slab loop proper, m0 written a multiply ahead of the copy that needs it, every per-copy address in a
// register or an immediate, and the per-slab bookkeeping down to an offset and three selects per cursor.
//
// Per slab r (two LDS slab buffers, r % 2; two register sets for A chunks), per wave:
//   K step 0   64 multiplies on fragment set 0; meanwhile the 16 fragments of K step 1 are read into set 1, the A
//              chunks of slab r+1 go from their register set to LDS and the A chunks of slab r+3 are requested
//              into that set
//   wait for the fragment reads and for this wave's B copies of slab r+1, workgroup barrier
//   K step 1   64 multiplies on set 1; meanwhile the fragments of slab r+1 / K step 0 are read into set 0 and
//              this wave's B copies of slab r+2 go straight to LDS, into the buffer of slab r
// Within a K step the sixteen fragment reads follow the first sixteen multiplies, one each; the LDS writes with their
// reloads, or the copies, follow from the seventeenth multiply on, one every fourth or fifth multiply (fragment
// reads and 16-byte LDS writes slow each other down when they alternate).
// A is the operand that streams from memory (B panels are shared through L2), so it is requested two slabs
// earlier than an LDS buffer is free for it: worth 3 % over copying it straight to LDS a slab ahead, although
// the LDS writes cost more than that copy would.  The slabs of all of a workgroup's tiles form one stream; each
// of the two cursors carries the buffer descriptor of its tile's window and an offset along K.
//
// The epilogue rides on multiplies: the upper half of a wave's block is converted and stored between the multiplies
// of the tile's last K step, the lower half between those of the next tile's first K step, whose multiplies start
// from a zero addend instead of the accumulators (see "epilogue" below).  With B as [G, N, K] the results never pass
// through LDS: the rows of a B slab sit in LDS in an order that makes each lane's results of the eight column blocks
// eight neighbouring outputs of a row.  Measured on the headline shape: staging a tile's results in LDS costs 9 % of
// a launch in LDS bandwidth however it is spread over those two K steps (fragment reads already take half of it);
// exchanging halves between lane groups instead gives 16 rows x 64 bytes per store, whose lanes four by four lie in
// different rows, and costs 6 % more than staging; the permuted slab rows give 4 rows x 256 bytes per store and
// cost nothing.  What remains of the epilogue is the write traffic itself (6 % of a launch against stores that
// write nothing).
//
// Headline shape (G = 128, M = 655360, N = 1536, K = 2048), same box: 3.03 ms against 3.30 ms for the eight-wave
// kernel; K = 768 shape 1.77 against 1.97 ms; masked decode (G = 128, up to 512 rows per group, N = 4096, K = 1536)
// 0.51 against 0.56 ms.  Large M-grouped launches with K a multiple of 128 take this kernel (w4_supported); masked
// launches of that size enqueue it together with the eight-wave kernel and the counts decide on the device which of
// the two runs (GemmParams::wide_gate); everything else goes to the eight-wave kernels.
//
// What the compiler does not know about assembly statements, and how it is handled here:
//   * a fragment read's result arrives later: every register a read targets passes through the wait statement
//     ("+v") before a multiply may use it;
//   * the A chunks are in flight across loop iterations and paths that join: their registers (v[192:255]) are named
//     in the instruction text and listed as clobbered, the compiler never holds a value in them
//     (tests/test_isa_hazards.py scans the kept assembly for any other use);
//   * the multiplies write AGPRs: compiled code (the epilogue's conversions) reads a block's accumulators no sooner
//     than three multiplies after the multiply that wrote them (a multiply takes 16 cycles to issue and delivers
//     within two more), except where a flush follows a tile directly: there the last row block's accumulators pass
//     through a statement of idle cycles first.  Accumulators are never the target of a load.
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
  static constexpr int EPI_PITCH = 4 * 32 + 16;              // epilogue staging (B as [G, K, N] only); a piece: 16 rows x 64 outputs, row pitch in bytes
  static constexpr int EPI_PIECE = 16 * EPI_PITCH;
  static constexpr int EPI_WAVE_BYTES = 2 * EPI_PIECE;       // two pieces alternate
  static constexpr int SCHED_OFF = 2 * STAGE_BYTES;
  static constexpr int EPI_OFF = SCHED_OFF + (((int)sizeof(SchedTableT<kFastMaxGroups>) + 255) & ~255);
  static constexpr int SMEM_BYTES = EPI_OFF + NWAVES * EPI_WAVE_BYTES;
  static_assert(SMEM_BYTES <= 160 * 1024, "LDS budget");
};

// A is the operand that takes the long way through registers ("staged", s), B is copied straight to LDS ("direct",
// d).  Staging B instead makes no difference even where the weights are what streams from memory (masked decode:
// 0.526 ms either way).
// SIT_OUT: a wave whose block of a tile has no rows or no columns multiplies nothing in that tile (it keeps its share
// of the copy stream and the barriers going).  Worth 2 % where a quarter of the tiles have at most 128 rows (masked
// decode); where nearly every tile is full the branch per K step costs the others 1 %, and such a wave multiplies
// the zeros its windows deliver.
template <int DT, int LAYOUT, bool SIT_OUT>
__global__ __launch_bounds__(W4Cfg::THREADS) void gemm_w4_kernel(const GemmParams p) {
  typedef W4Cfg C;
  constexpr int S_OFF = 0, D_OFF = C::A_BYTES;  // the operands' places in a slab buffer
  constexpr bool B_KMAJOR = LAYOUT == W4_NT;  // NN: B is [G, K, N], its slab 64 token rows of 512 bytes (N a multiple of 256)
  typedef Operand<C::BM, true> Op;            // the A slab, and B's when K-contiguous: 256 rows of 128 bytes
  typedef Operand<C::BN, B_KMAJOR> OpB;

  extern __shared__ __attribute__((aligned(1024))) char smem[];
  auto& sched = *reinterpret_cast<SchedTableT<kFastMaxGroups>*>(smem + C::SCHED_OFF);
  sched_init<C::BM>(p, sched);
  // a launch that only pays where the eight-wave kernels would choose 256x256 tiles as well (GemmParams::wide_gate):
  // the same predicate on the same table decides there that the eight-wave launch behind this one has nothing to do
  if (p.wide_gate == 1 && !sched_wide_tiles_chosen<C::BM, C::BN>(p, sched)) return;
  const int num_tiles = (int)sched_num_tiles<C::BM, C::BN>(p, sched);

  const uint32_t smem_addr = (uint32_t)(uintptr_t)(lds_ptr_t)smem;
  const int lane = lane_id();
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int wm0 = (wave >> 1) * 128, wn0 = (wave & 1) * 128;
  const int l16 = lane & 15, lg = lane >> 4;

  const int ld = p.K * 2;  // row pitch of A and of B in bytes; K is a multiple of 128 (w4_supported)
  // Copy k (0..7) of an operand's slab by this wave is copy instruction wave + 4 k of the slab: rows 8 (wave + 4 k) ...
  // + 7.  Its per-lane source offset within the tile's window is fixed for the launch; the slab's offset along K
  // travels in the instruction's scalar offset, which the range check of the window (its valid rows) leaves out.
  int vo[8];
#pragma unroll
  for (int k = 0; k < 8; ++k) vo[k] = Op::lane_voff(lane, wave % Op::NPAT, ld) + (wave + 4 * k) * Op::RPI * ld;
  static_assert(Op::NPAT == 2, "the swizzle pattern of copy wave + 4 k is that of copy wave");
  // NN: B's copies have offsets of their own (two token rows of 512 bytes per copy, row pitch 2 N)
  const int ld_b = (B_KMAJOR ? p.K : p.N) * 2;
  // NT: B's rows land in LDS permuted: LDS row 128 h + 16 j + c of the slab (column block j of a wave's half h, lane
  // column c of the multiply) holds column 128 h + 8 c + j of the tile, so that a lane's results of the eight column
  // blocks are eight neighbouring outputs of a row and leave as one 16-byte store without passing through LDS.
  int vo_b[8];
#pragma unroll
  for (int k = 0; k < 8; ++k) {
    if (B_KMAJOR) {
      const int r_local = lane / Op::CPR;  // LDS row 8 (wave + 4 k) + r_local: h = k / 4, j = 2 (k % 4) + wave / 2, c = 8 (wave % 2) + r_local
      const int col = 128 * (k >> 2) + 8 * (8 * (wave & 1) + r_local) + 2 * (k & 3) + (wave >> 1);
      vo_b[k] = Op::lane_voff(lane, wave % Op::NPAT, ld) + (col - r_local) * ld;
    } else {
      vo_b[k] = OpB::lane_voff(lane, (wave + 4 * k) % OpB::NPAT, ld_b) + (wave + 4 * k) * OpB::RPI * ld_b;
    }
  }

  // LDS addresses of the fragment reads relative to a slab buffer (see gemm_fast.hip for the layout)
  uint32_t a_rd[2], b_rd[B_KMAJOR ? 2 : 8];
#pragma unroll
  for (int ks = 0; ks < 2; ++ks) a_rd[ks] = smem_addr + (wm0 + l16) * 128 + (((4 * ks + lg) ^ ((l16 / 2) % 8)) << 4);
  if (B_KMAJOR) {
#pragma unroll
    for (int ks = 0; ks < 2; ++ks) b_rd[ks] = smem_addr + C::A_BYTES + (wn0 + l16) * 128 + (((4 * ks + lg) ^ ((l16 / 2) % 8)) << 4);
  } else {
#pragma unroll
    for (int j = 0; j < 8; ++j) {  // per column block: token row 8 lg + e, 16-byte chunk of the lane's columns, swizzled
      const int e = l16 >> 2, c = l16 & 3;
      const int chunk = ((wn0 + 16 * j) / 8 + (c >> 1)) ^ (e * 4) ^ ((lg & 1) * 2);
      b_rd[B_KMAJOR ? 0 : j] = smem_addr + C::A_BYTES + (lg * 8 + e) * (C::BN * 2) + chunk * 16 + (c & 1) * 8;
    }
  }

  // ---- the copy stream --------------------------------------------------------------------------------------------
  // The slabs of all of this workgroup's tiles form one stream.  While slab r is multiplied, the B copies of slab
  // r + 2 go straight to LDS (into the buffer of slab r, free after the barrier in the middle of the slab) and the A
  // chunks of slab r + 3 are loaded into registers, from where the chunks of slab r + 1, loaded two slabs earlier,
  // have just been written to LDS: A is the operand that comes from memory, B panels are shared through L2.
  // Each of the two cursors holds the window (buffer descriptor) of the tile it is in and its offset along K.
  struct Win { i32x4_t rs, rd; };  // staged operand, directly copied operand
  auto window = [&](const Tile& t, bool live) __attribute__((always_inline))  {
    Win w;
    const int n_left = p.N - t.n0;
    w.rs = make_rsrc32((uint64_t)p.A + (uint64_t)(t.row0 * ld), live ? t.rows * ld : 0);  // only the tile's valid rows
    if (B_KMAJOR) w.rd = make_rsrc32((uint64_t)p.B + (uint64_t)(((int64_t)t.g * p.N + t.n0) * ld), live ? (n_left < C::BN ? n_left : C::BN) * ld : 0);
    // NN: the tile's 256 columns of the group's K rows; N is a multiple of 256 (w4_supported), so every 512-byte row
    // segment lies inside its row, and the scalar offset of a slab (which the range check leaves out) stays below K rows
    else w.rd = make_rsrc32((uint64_t)p.B + (uint64_t)(((int64_t)t.g * p.K * p.N + t.n0) * 2), live ? p.K * ld_b : 0);
    return w;
  };
  const TileWalk walk64 = sched_walk(num_tiles, p.tile_split != 0);
  struct { int first, end, stride; } walk = {(int)walk64.first, (int)walk64.end, (int)walk64.stride};
  const int row_bytes = __builtin_amdgcn_readfirstlane(ld);
  int hint_g = -1;
  auto tile_at = [&](int id, Tile& t) __attribute__((always_inline))  {  // false: the walk has ended
    if (id >= walk.end) { t.g = 0; t.row0 = 0; t.rows = 0; t.n0 = 0; t.k0 = t.k1 = 0; return false; }
    const Tile v = sched_tile<C::BM, C::BN>(p, sched, id, hint_g);
    // the same in every lane; in scalar registers, so that what depends on it branches as a wave
    t.g = __builtin_amdgcn_readfirstlane(v.g);
    t.row0 = (int64_t)uniform64((uint64_t)v.row0);
    t.rows = __builtin_amdgcn_readfirstlane(v.rows);
    t.n0 = __builtin_amdgcn_readfirstlane(v.n0);
    t.k0 = t.k1 = 0;
    hint_g = t.g;
    return true;
  };

  // The staged A chunks live in v[192:255] (two sets of eight), named in the instruction text: a value that is in
  // flight across loop iterations must not be known to the compiler, which would move it between registers (before
  // it has arrived) wherever two paths join.  The compiler's own allocation ends below v192 (checked on the kept
  // assembly by the tests).
#define TGG_W4_GA(c, f) \
  if (c == 0) { f("224", "227") } else if (c == 1) { f("228", "231") } else if (c == 2) { f("232", "235") } else if (c == 3) { f("236", "239") } \
  else if (c == 4) { f("240", "243") } else if (c == 5) { f("244", "247") } else if (c == 6) { f("248", "251") } else if (c == 7) { f("252", "255") } \
  else if (c == 8) { f("192", "195") } else if (c == 9) { f("196", "199") } else if (c == 10) { f("200", "203") } else if (c == 11) { f("204", "207") } \
  else if (c == 12) { f("208", "211") } else if (c == 13) { f("212", "215") } else if (c == 14) { f("216", "219") } else { f("220", "223") }
#define TGG_W4_GA_CLOBBER "v192", "v193", "v194", "v195", "v196", "v197", "v198", "v199", "v200", "v201", "v202", "v203", "v204", "v205", "v206", "v207", \
  "v208", "v209", "v210", "v211", "v212", "v213", "v214", "v215", "v216", "v217", "v218", "v219", "v220", "v221", "v222", "v223", "v224", "v225", "v226", "v227", \
  "v228", "v229", "v230", "v231", "v232", "v233", "v234", "v235", "v236", "v237", "v238", "v239", "v240", "v241", "v242", "v243", "v244", "v245", "v246", "v247", \
  "v248", "v249", "v250", "v251", "v252", "v253", "v254", "v255"
  const uint32_t s_wr = smem_addr + S_OFF + wave * 1024 + lane * 16;  // LDS address of this lane's 16 bytes of A copy 0 (buffer 0)
  // A chunk k of the slab at offset koff of window ra -> register set SET
  auto load_s = [&](auto Kc, auto SETc, const i32x4_t& ra, int koff) __attribute__((always_inline))  {
    constexpr int k = decltype(Kc)::value, kq = k + 8 * decltype(SETc)::value;
    const int v = vo[k];
#define TGG_W4_F(lo, hi) asm volatile("buffer_load_dwordx4 v[" lo ":" hi "], %0, %1, %2 offen" : : "v"(v), "s"(ra), "s"(koff) : "memory", TGG_W4_GA_CLOBBER);
    TGG_W4_GA(kq, TGG_W4_F)
#undef TGG_W4_F
  };
  // register set SET, chunk k -> LDS (wr_addr: s_wr + the buffer's offset)
  auto write_s = [&](auto Kc, auto SETc, uint32_t wr_addr) __attribute__((always_inline))  {
    constexpr int k = decltype(Kc)::value, kq = k + 8 * decltype(SETc)::value;
#define TGG_W4_F(lo, hi) asm volatile("ds_write_b128 %0, v[" lo ":" hi "] offset:%1" : : "v"(wr_addr), "n"(k * 4096) : "memory", TGG_W4_GA_CLOBBER);
    TGG_W4_GA(kq, TGG_W4_F)
#undef TGG_W4_F
  };
  // B copy k of the slab at offset koff of window rb, straight to LDS, in two statements a multiply apart: the LDS
  // address goes to m0 first (a copy to LDS needs a wait state after a write of m0; the multiply in between is one)
  auto copy_d_m0 = [&](auto Kc, uint32_t buf_addr) __attribute__((always_inline))  {
    constexpr int k = decltype(Kc)::value;
    asm volatile("s_add_u32 m0, %0, %1" : : "s"(buf_addr), "n"(D_OFF + 4 * k * 1024) : "memory", "m0", "scc");
  };
  auto copy_d = [&](auto Kc, const i32x4_t& rb, int koff, bool spaced) __attribute__((always_inline))  {
    constexpr int k = decltype(Kc)::value;
    const int v = vo_b[k];
    if (spaced) asm volatile("buffer_load_dwordx4 %0, %1, %2 offen lds" : : "v"(v), "s"(rb), "s"(koff) : "memory");
    else asm volatile("s_nop 0\n\tbuffer_load_dwordx4 %0, %1, %2 offen lds" : : "v"(v), "s"(rb), "s"(koff) : "memory");
  };
  // a slab's A copy k straight to LDS (prologue only)
  auto copy_direct = [&](auto Kc, auto ISBc, const i32x4_t& ra, int koff, uint32_t buf_addr) __attribute__((always_inline))  {
    constexpr int k = decltype(Kc)::value;
    const int v = decltype(ISBc)::value ? vo_b[k] : vo[k];
    asm volatile("s_add_u32 m0, %0, %1\n\ts_nop 0\n\tbuffer_load_dwordx4 %2, %3, %4 offen lds"
                 : : "s"(buf_addr), "n"(4 * k * 1024), "v"(v), "s"(ra), "s"(koff) : "memory", "m0", "scc");
  };
  const uint32_t wave_buf = smem_addr + wave * 1024;  // copy `wave` of buffer 0's A slab

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
      else lds_read_tr<KS * 32 * (C::BN * 2), KS * 32 * (C::BN * 2) + 4 * (C::BN * 2)>(sb[Q], b_rd[B_KMAJOR ? 0 : (Q < 8 ? Q : 0)] + buf_off);
    } else {
      lds_read_b128<(Q - 8) * 2048>(sa[Q - 8], a_rd[KS] + buf_off);
    }
  };
  // ---- epilogue ------------------------------------------------------------------------------------------------------
  // With one wave per SIMD nothing else would keep the matrix pipe busy while a wave converts and stores its 128x128
  // block, so the work sits in the gaps between multiplies: strips 0-3 (a strip: one 16-row block, 128 columns) during
  // the tile's last K step, each after its last multiply, strips 4-7 during the first K step of the workgroup's next
  // tile, each before the multiply that starts it afresh (that K step multiplies with a zero addend); a wave without
  // a next tile to multiply stores strips 4-7 in a flush.  Half a block's conversion per gap on average keeps the
  // gaps within what a multiply hides.
  // B as [G, N, K]: the multiply takes A's fragment as its first operand, so a lane holds rows 16 i + 4 lg + r
  // (r = 0..3) of one column per block, and the permuted slab rows (vo_b) make that column 8 l16 + j for block j:
  // the lane's eight blocks of a strip are 16 contiguous bytes of an output row, 16 lanes cover 256 bytes of it, and
  // a store instruction writes 4 rows x 256 bytes.
  // B as [G, K, N] (fragments come from transposing reads, which tie a lane's column to its number): B's fragment is
  // the first operand, a lane owns row l16 and columns 16 j + 4 lg + (0..3) of block (i, j); a strip goes through the
  // wave's LDS staging as two pieces of 64 columns and leaves as 16-byte stores covering 128-byte row segments.
  // The stores go through a buffer descriptor over the wave's block that ends with its last valid row; lanes whose
  // columns lie beyond N get an out-of-range offset: no branches.
  // Nothing pending = a descriptor of length zero.
  i32x4_t pend_rs = make_rsrc32(0, 0);
  int pend_cols = 0;
  bool pending = false;
  char* const stage = smem + C::EPI_OFF + wave * C::EPI_WAVE_BYTES;
  // per-lane staging addresses and output offset, recomputed where a first K step or a flush begins
  struct EpiLane { char* wr; const char* rd; int off[2]; };  // off[h]: output offset of the lane's 16 bytes in column half h of strip 0, out of range where those columns lie beyond N
  auto epi_lane = [&]() __attribute__((always_inline))  {
    int el = lane;
    asm volatile("" : "+v"(el));
    EpiLane e;
    e.wr = stage + (el & 15) * C::EPI_PITCH + (el >> 4) * 8;
    e.rd = stage + (el >> 3) * C::EPI_PITCH + (el & 7) * 16;
    const int off = ((el >> 3) * p.N + (el & 7) * 8) * 2, ch8 = (el & 7) * 8;
#pragma unroll
    for (int h = 0; h < 2; ++h) e.off[h] = (64 * h + ch8 < pend_cols) ? off + 128 * h : kNoFetch;
    return e;
  };
  // block (i, j) -> staging piece j / 4; not before this point in the instruction stream
  auto epi_cvt = [&](const EpiLane& e, int i, int j) __attribute__((always_inline))  {
    asm volatile("" : "+a"(acc[i][j]));
    *(uint2*)(e.wr + (j >> 2) * C::EPI_PIECE + (j & 3) * 32) = pack4<DT>(acc[i][j][0], acc[i][j][1], acc[i][j][2], acc[i][j][3]);
    asm volatile("" ::: "memory");
  };
  auto epi_read = [&](const EpiLane& e, int h, i32x4_t (&v)[2]) {
#pragma unroll
    for (int it = 0; it < 2; ++it) v[it] = *(const i32x4_t*)(e.rd + h * C::EPI_PIECE + it * 8 * C::EPI_PITCH);
    asm volatile("" ::: "memory");
  };
  auto epi_store = [&](const EpiLane& e, int i, int h, int it, const i32x4_t& v, bool between_multiplies) __attribute__((always_inline))  {
    // (an out-of-range marker stays out of range with the rows' offset added: both are far below 2^31)
    const int off = e.off[h] + (16 * i + 8 * it) * p.N * 2;
    // Two wait states must pass before a 16-byte store's data registers may be overwritten, and the compiler, which
    // considers them free after this statement, reuses them at once: between multiplies the multiply that follows is
    // one wait state, the flush has none.  No wait states in front: the descriptor sits in scalar registers since the
    // end of the tile.  Both hazards are checked on the kept assembly (tests/test_isa_hazards.py).
    if (between_multiplies) asm volatile("buffer_store_dwordx4 %0, %1, %2, 0 offen nt\n\ts_nop 0" : : "v"(v), "v"(off), "s"(pend_rs) : "memory");
    else asm volatile("buffer_store_dwordx4 %0, %1, %2, 0 offen nt\n\ts_nop 1" : : "v"(v), "v"(off), "s"(pend_rs) : "memory");
  };
  // NT: no staging.  A lane holds rows 16 i + 4 lg + r (r = 0..3) of column 8 l16 + j of the wave's block in
  // accumulator block (i, j), component r: the eight blocks of a strip give eight neighbouring outputs of a row.
  auto epi_lane_t = [&]() __attribute__((always_inline))  {
    int el = lane;
    asm volatile("" : "+v"(el));
    const int col = (el & 15) * 8;
    return col < pend_cols ? ((el >> 4) * 4 * p.N + col) * 2 : kNoFetch;
  };
  // outputs 4 h .. 4 h + 3 of the lane's eight in row r of strip i, converted; not before this point in the instruction stream
  auto epi_half_t = [&](int i, int r, int h) __attribute__((always_inline))  {
    asm volatile("" : "+a"(acc[i][4 * h]), "+a"(acc[i][4 * h + 1]), "+a"(acc[i][4 * h + 2]), "+a"(acc[i][4 * h + 3]));
    uint2 x;
    x.x = pack2<DT>(acc[i][4 * h][r], acc[i][4 * h + 1][r]);
    x.y = pack2<DT>(acc[i][4 * h + 2][r], acc[i][4 * h + 3][r]);
    asm volatile("" : "+v"(x.x), "+v"(x.y));
    return x;
  };
  auto epi_store_t = [&](int lane_off, int i, int r, const uint2& x, const uint2& y, bool between_multiplies) __attribute__((always_inline))  {
    i32x4_t v;
    v[0] = (int)x.x; v[1] = (int)x.y; v[2] = (int)y.x; v[3] = (int)y.y;
    const int off = lane_off + (16 * i + r) * p.N * 2;
    if (between_multiplies) asm volatile("buffer_store_dwordx4 %0, %1, %2, 0 offen nt\n\ts_nop 0" : : "v"(v), "v"(off), "s"(pend_rs) : "memory");
    else asm volatile("buffer_store_dwordx4 %0, %1, %2, 0 offen nt\n\ts_nop 1" : : "v"(v), "v"(off), "s"(pend_rs) : "memory");
  };
  // everything that is pending, without multiplies to hide it under
  auto epi_flush = [&]() __attribute__((always_inline))  {
    if (pending) {
      // the last row block's multiplies may have just been issued: give them time before compiled code reads the registers
      asm volatile("s_nop 15\n\ts_nop 7" : "+a"(acc[7][0]), "+a"(acc[7][1]), "+a"(acc[7][2]), "+a"(acc[7][3]),
                   "+a"(acc[7][4]), "+a"(acc[7][5]), "+a"(acc[7][6]), "+a"(acc[7][7]));
      if (B_KMAJOR) {
        const int lane_off = epi_lane_t();
#pragma unroll
        for (int i = 4; i < 8; ++i)
#pragma unroll
          for (int r = 0; r < 4; ++r) {
            const uint2 x = epi_half_t(i, r, 0), y = epi_half_t(i, r, 1);
            epi_store_t(lane_off, i, r, x, y, false);
          }
      }
      const EpiLane e = epi_lane();
#pragma unroll
      for (int i = B_KMAJOR ? 8 : 4; i < 8; ++i) {  // the first four strips left during the tile's last K step
#pragma unroll
        for (int j = 0; j < 8; ++j) epi_cvt(e, i, j);
#pragma unroll
        for (int h = 0; h < 2; ++h) {
          i32x4_t v[2];
          epi_read(e, h, v);
          epi_store(e, i, h, 0, v[0], false);
          epi_store(e, i, h, 1, v[1], false);
        }
      }
    }
    pending = false;
    pend_rs[2] = 0;
  };


  typedef std::integral_constant<int, 0> I0;
  typedef std::integral_constant<int, 1> I1;
  typedef std::integral_constant<int, 2> I2;
  typedef std::integral_constant<bool, true> Yes;
  typedef std::integral_constant<bool, false> No;

  // the two cursors of the copy stream and the tile after the one being multiplied
  i32x4_t rs_c, rd_c;
  int koff_s, koff_d;
  Win nxt;
  Tile nxt_tile;
  const int k_bytes = row_bytes;  // a tile's extent along K in bytes: where a cursor moves on to the next tile
  auto advance_s = [&]() __attribute__((always_inline))  {
    const bool wrap = koff_s + 128 == k_bytes;
    koff_s = wrap ? 0 : koff_s + 128;
#pragma unroll
    for (int q = 0; q < 3; ++q) rs_c[q] = wrap ? nxt.rs[q] : rs_c[q];
  };
  const int d_step = B_KMAJOR ? 128 : __builtin_amdgcn_readfirstlane(64 * ld_b);         // B's slab offset per slab ...
  const int d_bytes = B_KMAJOR ? k_bytes : __builtin_amdgcn_readfirstlane(p.K * ld_b);   // ... and where it reaches the next tile
  auto advance_d = [&]() __attribute__((always_inline))  {
    const bool wrap = koff_d + d_step == d_bytes;
    koff_d = wrap ? 0 : koff_d + d_step;
#pragma unroll
    for (int q = 0; q < 3; ++q) rd_c[q] = wrap ? nxt.rd[q] : rd_c[q];
  };

  // One K step: 64 multiplies on fragment set CUR (when MUL); the 16 fragments of K step NKS of the slab at nb_off go
  // to the other set, one read after each of the first sixteen multiplies; the LDS writes and the loads and copies follow
  // behind them (reads and staged writes apart in time: 2.5 % over interleaving them through the whole K step; the
  // loads must not slip much later, a quarter of a slab less lead costs 6 %).  Outside the two K steps that carry
  // the epilogue at most two other instructions sit between two multiplies: a wave issues in order, and what exceeds
  // the sixteen cycles of a multiply leaves the matrix pipe idle.
  // ROLE 0: prologue (reads only, waits for everything).
  // ROLE 1: a slab's first K step.  The A chunks of the next slab go from register set SET to LDS (wr_addr) and the
  //         chunks of the slab three ahead are requested into the same set; ends with the wait for the B copies of
  //         the next slab (eight younger loads, and the 16 stores of a tile's first K step, may stay in flight; loads
  //         and stores complete in order, so the A chunks written here -- requested two slabs ago -- have arrived
  //         since the previous such wait).
  // ROLE 2: second K step: the B copies of the slab two ahead, into the buffer at cp_addr.
  // EPI 1: the first K step of a tile -- multiplies start from zero, strips 4-7 of the tile before are stored between
  //        them.  EPI 2: the last K step of a tile -- strips 0-3 are stored between its multiplies.
  auto kstep = [&](auto CURc, auto NKSc, auto MULc, auto ROLEc, uint32_t nb_off, auto EPIc, uint32_t wr_addr, auto SETc, uint32_t cp_addr) __attribute__((always_inline))  {
    constexpr int CUR = decltype(CURc)::value, NKS = decltype(NKSc)::value, ROLE = decltype(ROLEc)::value;
    constexpr bool MUL = decltype(MULc)::value;
    constexpr int EPI = decltype(EPIc)::value;
    static_assert(!EPI || MUL, "the epilogue rides on a multiplying K step");
    EpiLane e = {nullptr, nullptr, {0, 0}};
    i32x4_t vv[2][2];
    if (EPI && !B_KMAJOR) e = epi_lane();
    int lane_off = 0;
    uint2 ex = {0, 0};
    if (EPI && B_KMAJOR) lane_off = epi_lane_t();
    // NT: unit u = 4 (strip - first strip) + r in the gaps in front of multiplies T0 + 3 u and T0 + 3 u + 1: a strip of
    // the tile's last K step is complete three multiplies before its first unit, a strip of the first K step is
    // started afresh after its last unit
    constexpr int EPI_T0 = EPI == 2 ? 11 : 0;
    // EPI 2 (a tile's last K step) converts and stores strips 0-3 of the tile, EPI 1 (the next tile's first) strips
    // 4-7: block bb of the half in the gap in front of multiply G0 + 7 bb / 4, at least four multiplies after the
    // multiply that completed it and before the one that starts it afresh; a piece (four blocks) is read back in the
    // gap of its last block and stored two and four gaps later.
    constexpr int EPI_S0 = EPI == 2 ? 0 : 4, EPI_G0 = EPI == 2 ? 4 : 0;
#pragma unroll
    for (int i = 0; i < 8; ++i)
#pragma unroll
      for (int jj = 0; jj < 8; ++jj) {
        const int j = (i & 1) ? 7 - jj : jj;  // snake order: one operand register changes per multiply
        if (EPI && B_KMAJOR) {
          const int gap = i * 8 + jj;
#pragma unroll
          for (int u = 0; u < 16; ++u) {
            if (EPI_T0 + 3 * u == gap) ex = epi_half_t(EPI_S0 + u / 4, u % 4, 0);
            if (EPI_T0 + 3 * u + 1 == gap) { const uint2 ey = epi_half_t(EPI_S0 + u / 4, u % 4, 1); epi_store_t(lane_off, EPI_S0 + u / 4, u % 4, ex, ey, true); }
          }
        }
        if (EPI && !B_KMAJOR) {
          const int gap = i * 8 + jj;
#pragma unroll
          for (int bb = 0; bb < 32; ++bb) {
            const int g = EPI_G0 + 7 * bb / 4, si = EPI_S0 + bb / 8, sj = (si & 1) ? 7 - bb % 8 : bb % 8;
            if (g == gap) epi_cvt(e, si, sj);
            if ((bb & 3) == 3 && g == gap) epi_read(e, sj >> 2, vv[(bb >> 2) & 1]);
          }
#pragma unroll
          for (int bb = 3; bb < 32; bb += 4) {
            const int g = EPI_G0 + 7 * bb / 4, si = EPI_S0 + bb / 8, sj = (si & 1) ? 7 - bb % 8 : bb % 8;
            if (g + 2 == gap) epi_store(e, si, sj >> 2, 0, vv[(bb >> 2) & 1][0], true);
            if (g + 4 == gap) epi_store(e, si, sj >> 2, 1, vv[(bb >> 2) & 1][1], true);
          }
        }
        if (EPI == 1) {
          if (B_KMAJOR) mfma_new<DT>(acc[i][j], fa[CUR][i], fb[CUR][j]);
          else mfma_new<DT>(acc[i][j], fb[CUR][j], fa[CUR][i]);
        } else if (MUL) {
          if (B_KMAJOR) mfma_acc<DT>(acc[i][j], fa[CUR][i], fb[CUR][j]);
          else mfma_acc<DT>(acc[i][j], fb[CUR][j], fa[CUR][i]);
        }
        const int n = i * 8 + jj;
#define TGG_W4_RD(q) if (n == q) read_frag(std::integral_constant<int, NKS>(), std::integral_constant<int, q>(), fa[CUR ^ 1], fb[CUR ^ 1], nb_off);
        TGG_W4_RD(0) TGG_W4_RD(1) TGG_W4_RD(2) TGG_W4_RD(3) TGG_W4_RD(4) TGG_W4_RD(5) TGG_W4_RD(6) TGG_W4_RD(7)
        TGG_W4_RD(8) TGG_W4_RD(9) TGG_W4_RD(10) TGG_W4_RD(11) TGG_W4_RD(12) TGG_W4_RD(13) TGG_W4_RD(14) TGG_W4_RD(15)
#undef TGG_W4_RD
        if (ROLE == 1) {
#define TGG_W4_ST(c) if (n == 16 + 4 * c) write_s(std::integral_constant<int, c>(), SETc, wr_addr); \
                     if (n == 18 + 4 * c) { load_s(std::integral_constant<int, c>(), SETc, rs_c, koff_s); if (!MUL) __builtin_amdgcn_s_sleep(1); }
          TGG_W4_ST(0) TGG_W4_ST(1) TGG_W4_ST(2) TGG_W4_ST(3) TGG_W4_ST(4) TGG_W4_ST(5) TGG_W4_ST(6) TGG_W4_ST(7)
#undef TGG_W4_ST
          if (n == 52) advance_s();
        }
        if (ROLE == 2) {
#define TGG_W4_CP(c) if (n == 16 + 5 * c) copy_d_m0(std::integral_constant<int, c>(), cp_addr); \
                     if (n == 17 + 5 * c) { copy_d(std::integral_constant<int, c>(), rd_c, koff_d, MUL); if (!MUL) __builtin_amdgcn_s_sleep(1); }
          TGG_W4_CP(0) TGG_W4_CP(1) TGG_W4_CP(2) TGG_W4_CP(3) TGG_W4_CP(4) TGG_W4_CP(5) TGG_W4_CP(6) TGG_W4_CP(7)
#undef TGG_W4_CP
          if (n == 56) advance_d();
        }
      }
    if (ROLE == 2) asm volatile("s_waitcnt lgkmcnt(0)" : TGG_TIE8(fa[CUR ^ 1]), TGG_TIE8(fb[CUR ^ 1]) : : "memory");
    else if (ROLE == 1) asm volatile("s_waitcnt vmcnt(%16) lgkmcnt(0)" : TGG_TIE8(fa[CUR ^ 1]), TGG_TIE8(fb[CUR ^ 1]) : "n"(EPI ? 24 : 8) : "memory");
    else asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)" : TGG_TIE8(fa[CUR ^ 1]), TGG_TIE8(fb[CUR ^ 1]) : : "memory");
  };

  // ---- prologue: slab 0 lands in buffer 0, slabs 1 and 2 are requested, the first fragments are read -----------------
  Tile cur;
  tile_at(walk.first, cur);
  {
    const Win w0 = window(cur, walk.first < walk.end);
    const bool more = tile_at(walk.first + walk.stride, nxt_tile);
    nxt = window(nxt_tile, more);
    rs_c = w0.rs;
    rd_c = w0.rd;
  }
#define TGG_W4_EACH(f) f(0) f(1) f(2) f(3) f(4) f(5) f(6) f(7)
#define TGG_W4_P0(c) copy_direct(std::integral_constant<int, c>(), No(), rs_c, 0, wave_buf + S_OFF); \
                     copy_direct(std::integral_constant<int, c>(), Yes(), rd_c, 0, wave_buf + D_OFF);
  TGG_W4_EACH(TGG_W4_P0)
#undef TGG_W4_P0
  wait_vmcnt<0>();
  __syncthreads();
#define TGG_W4_P1(c) load_s(std::integral_constant<int, c>(), I1(), rs_c, 128);
  TGG_W4_EACH(TGG_W4_P1)
#undef TGG_W4_P1
#define TGG_W4_P2(c) copy_direct(std::integral_constant<int, c>(), Yes(), rd_c, d_step, wave_buf + C::STAGE_BYTES + D_OFF);
  TGG_W4_EACH(TGG_W4_P2)
#undef TGG_W4_P2
#define TGG_W4_P3(c) load_s(std::integral_constant<int, c>(), I0(), rs_c, 256);
  TGG_W4_EACH(TGG_W4_P3)
#undef TGG_W4_P3
  koff_s = 3 * 128;  // at least four slabs per tile (w4_supported): both cursors are still in the first tile
  koff_d = 2 * d_step;
  kstep(I1(), I0(), No(), I0(), 0u, I0(), 0u, I0(), 0u);  // reads K step 0 of buffer 0 into set 0, multiplies nothing, waits for everything
  const int kt_all = p.K / BK4;

  for (int tile_id = walk.first; tile_id < walk.end; tile_id += walk.stride) {
    const bool active = wm0 < cur.rows && cur.n0 + wn0 < p.N;  // this wave's block of the tile has rows and columns
    const bool mul = !SIT_OUT || active;
    if (!mul) epi_flush();  // no multiplies in this tile to hide the pending stores under
    // one slab; FIRST: the tile's first, whose first K step starts the accumulators afresh and carries the epilogue;
    // PAR: parity of the slab = its LDS buffer; the A chunks of the next slab wait in register set 1 - PAR
    auto slab = [&](auto EPc, auto PARc) __attribute__((always_inline)) {
      typedef std::integral_constant<int, decltype(EPc)::value == 1 ? 1 : 0> Ep0;  // the tile's first slab: its first K step carries strips 4-7 of the tile before
      typedef std::integral_constant<int, decltype(EPc)::value == 2 ? 2 : 0> Ep1;  // the tile's last slab: its second K step carries strips 0-3
      constexpr int PAR = decltype(PARc)::value;
      typedef std::integral_constant<int, 1 - PAR> SetN;
      constexpr uint32_t cur_off = PAR * C::STAGE_BYTES, nxt_off = C::STAGE_BYTES - cur_off;
      if (mul) kstep(I0(), I1(), Yes(), I1(), cur_off, Ep0(), s_wr + nxt_off, SetN(), 0u);
      else kstep(I0(), I1(), No(), I1(), cur_off, I0(), s_wr + nxt_off, SetN(), 0u);
      // set 1 is complete, this wave has read all it needs of the current slab, its copies of the next slab have landed
      asm volatile("s_barrier" ::: "memory");
      if (mul) kstep(I1(), I0(), Yes(), I2(), nxt_off, Ep1(), 0u, I0(), wave_buf + cur_off);
      else kstep(I1(), I0(), No(), I2(), nxt_off, I0(), 0u, I0(), wave_buf + cur_off);
    };
    slab(I1(), I0());  // an even number of slabs per tile, at least four: every tile starts in buffer 0
    slab(I0(), I1());
    for (int kt = 4; kt < kt_all; kt += 2) {
      slab(I0(), I0());
      slab(I0(), I1());
    }
    // what the tile's last K step, the next tile's first K step and a flush store: nothing for a wave whose block of
    // the tile has no rows or no columns
    const int rows_left = cur.rows - wm0;
    pend_rs = make_rsrc32((uint64_t)p.C + (uint64_t)(((cur.row0 + wm0) * (int64_t)p.N + cur.n0 + wn0) * 2),
                          active ? (rows_left < 128 ? rows_left : 128) * p.N * 2 : 0);
    pend_cols = __builtin_amdgcn_readfirstlane(active ? p.N - cur.n0 - wn0 : 0);
    pending = mul;  // a wave that sat the tile out has flushed and leaves nothing behind
    slab(I0(), I0());
    slab(I2(), I1());
    // both cursors are in the next tile by now: it becomes the current one, and the one after it is looked up
    cur = nxt_tile;
    const bool more = tile_at(tile_id + 2 * walk.stride, nxt_tile);
    nxt = window(nxt_tile, more);
  }
  epi_flush();
  wait_vmcnt<0>();  // trailing zero-length copies still write LDS
#undef TGG_W4_EACH
#undef TGG_W4_GA
#undef TGG_W4_GA_CLOBBER
}

template <int DT, int LAYOUT, bool SIT_OUT>
int launch_w4(const GemmParams& p, hipStream_t s) {
  static bool attr_set[64] = {false};
  int dev = 0;
  (void)hipGetDevice(&dev);
  const bool listed = dev >= 0 && dev < 64;
  auto kern = gemm_w4_kernel<DT, LAYOUT, SIT_OUT>;
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

// Whether 256-row tiles pay depends on the group sizes, which only the device knows.  With 512 rows and more per group on
// average they do; a masked launch (counts anywhere up to its row stride) or an M-grouped one with smaller groups is
// enqueued together with the eight-wave kernel, and the two decide from the sizes which of them runs.
bool w4_decided_on_device(const GemmParams& p) {
  return p.mode == MODE_MASKED || p.m_total < 512 * (int64_t)p.G;
}

// The four-wave kernel takes M-grouped launches (rows contiguous or padded) whose tile count is large whatever the
// group sizes turn out to be: at least ceil(m_total / 256) row tiles.  Smaller launches stay with the eight-wave
// kernels, which choose narrower tiles on the device.
bool w4_supported(const GemmParams& p, int dt, int layout, bool any_size) {
  if (dt != DT_BF16 && dt != DT_F16) return false;
  if (layout != W4_NT && layout != W4_NN) return false;
  // NN: every 512-byte row segment of a tile must lie inside its row of B, and a group's B within 2 GiB
  if (layout == W4_NN && ((p.N & 255) != 0 || (int64_t)p.K * p.N * 2 >= (1ll << 31))) return false;
  if (p.mode != MODE_MG && p.mode != MODE_MG_PAD && p.mode != MODE_MASKED) return false;
  // launches whose groups may be small are decided on the device (w4_decided_on_device), by a predicate that needs
  // one thread of this kernel per group
  if (w4_decided_on_device(p) && p.G > W4Cfg::THREADS) return false;
  if (p.q_fmt != 0 || p.G > kFastMaxGroups) return false;
  if ((p.N & 7) != 0 || p.K < 8 || (p.K & 7) != 0) return false;
  if ((int64_t)p.K * 2 * 256 >= (1ll << 30)) return false;
  if ((int64_t)p.N * 2 * 128 >= (1ll << 30)) return false;  // a wave's block of the output within the epilogue's 32-bit offsets, out-of-range marker included
  if (p.K % 128 != 0 || p.K < 256) return false;  // an even number of 64-deep slabs per tile, four at least
  if (any_size) return true;
  int grid = num_cus();
  if (p.grid_limit > 0 && p.grid_limit < grid) grid = p.grid_limit;
  const int64_t row_tiles = (p.m_total + 255) / 256;
  const int64_t narrow_tiles = row_tiles * ((p.N + 127) / 128);
  return narrow_tiles > 4 * (int64_t)grid;
}

int launch_w4_16bit(const GemmParams& p, int dt, int layout, hipStream_t s) {
  const bool sit_out = p.mode == MODE_MASKED;
  if (layout == W4_NT) {
    if (dt == DT_BF16) return sit_out ? launch_w4<DT_BF16, W4_NT, true>(p, s) : launch_w4<DT_BF16, W4_NT, false>(p, s);
    return sit_out ? launch_w4<DT_F16, W4_NT, true>(p, s) : launch_w4<DT_F16, W4_NT, false>(p, s);
  }
  if (dt == DT_BF16) return sit_out ? launch_w4<DT_BF16, W4_NN, true>(p, s) : launch_w4<DT_BF16, W4_NN, false>(p, s);
  return sit_out ? launch_w4<DT_F16, W4_NN, true>(p, s) : launch_w4<DT_F16, W4_NN, false>(p, s);
}

}  // namespace tgg
