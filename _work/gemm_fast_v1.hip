// Tuned bf16/fp16 grouped GEMM for gfx950, K-contiguous operands ("NT": A [rows, K], B [G, N, K]).
//
// Persistent workgroups walk the grouped tile space (sched.hpp).  Per tile:
//   * A and B slabs of BK columns stream HBM/L2 -> LDS with buffer_load_dwordx4 ... lds
//     (no VGPR staging); rows past the end of the operand read as zero through the buffer
//     descriptor's bounds check, so ragged groups need no special path;
//   * NSTAGE slabs are in flight; one barrier per slab;
//   * LDS rows are XOR-swizzled at 16-byte granularity (applied on the global side of the
//     direct-to-LDS copy, whose LDS side is lane-linear) so that ds_read_b128 fragment reads
//     are bank-conflict free;
//   * each wave owns a (BM/WM) x (BN/WN) block of 32x32x16 MFMA tiles, issued with the
//     weights as srcA and the activations as srcB so a lane ends up with 4 consecutive
//     output columns of one row.
#include "common.hpp"
#include "sched.hpp"
#include "launch.hpp"

namespace tgg {

namespace {

typedef __attribute__((address_space(3))) void* lds_ptr_t;

template <int DT> struct Mma16;
template <> struct Mma16<DT_BF16> {
  static TGG_DEV f32x16_t run(i32x4_t w, i32x4_t x, f32x16_t c) {
    return __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8_t, w), __builtin_bit_cast(bf16x8_t, x), c, 0, 0, 0);
  }
};
template <> struct Mma16<DT_F16> {
  static TGG_DEV f32x16_t run(i32x4_t w, i32x4_t x, f32x16_t c) {
    return __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(f16x8_t, w), __builtin_bit_cast(f16x8_t, x), c, 0, 0, 0);
  }
};

// s_waitcnt vmcnt(n) only (gfx9 encoding: vmcnt[3:0] | expcnt[6:4] | lgkmcnt[11:8] | vmcnt_hi[15:14]).
template <int N> TGG_DEV void wait_vmcnt() {
  static_assert(N >= 0 && N < 64, "vmcnt range");
  __builtin_amdgcn_s_waitcnt((N & 15) | ((N >> 4) << 14) | (7 << 4) | (15 << 8));
}

// One wave-wide 16-byte-per-lane copy global -> LDS.  The LDS destination is m0 + lane * 16, the
// global source is the descriptor base + voff (bounds-checked: out-of-range lanes write zeros).
// Written as inline assembly on purpose: the compiler does not model the copy, so it cannot
// serialise the software pipeline with conservative waits; completion is tracked by hand with
// wait_vmcnt<>() and the workgroup barrier.
TGG_DEV void copy_b128_to_lds(i32x4_t rsrc, uint32_t lds_addr, int voff) {
  asm volatile("s_mov_b32 m0, %0\n\tbuffer_load_dwordx4 %1, %2, 0 offen lds" : : "s"(lds_addr), "v"(voff), "s"(rsrc) : "memory");
}

// Same, 4 bytes per lane (LDS destination m0 + lane * 4).
TGG_DEV void copy_b32_to_lds(i32x4_t rsrc, uint32_t lds_addr, int voff) {
  asm volatile("s_mov_b32 m0, %0\n\tbuffer_load_dword %1, %2, 0 offen lds" : : "s"(lds_addr), "v"(voff), "s"(rsrc) : "memory");
}

TGG_DEV i32x4_t make_rsrc(const void* base, uint32_t num_bytes) {
  const uint64_t a = (uint64_t)base;
  i32x4_t r;  // wave-uniform by construction; readfirstlane pins it to scalar registers
  r[0] = __builtin_amdgcn_readfirstlane((int)(uint32_t)a);
  r[1] = __builtin_amdgcn_readfirstlane((int)(uint32_t)(a >> 32) & 0xffff);  // stride 0, no swizzle
  r[2] = __builtin_amdgcn_readfirstlane((int)num_bytes);
  r[3] = 0x00020000;                                                          // raw 32-bit data format
  return r;
}

constexpr int kFastMaxGroups = 256;

// PFD: how many slabs beyond the one being copied the L2 warm-up reads run (0 = no warm-up).
template <int BM_, int BN_, int BK_, int NSTAGE_, int WM_, int WN_, int PFD_ = 2>
struct FastCfg {
  static constexpr int BM = BM_, BN = BN_, BK = BK_, NSTAGE = NSTAGE_, WM = WM_, WN = WN_, PFD = PFD_;
  static constexpr int NWAVES = WM * WN;
  static constexpr int THREADS = NWAVES * 64;
  static constexpr int RB = BK * 2;            // bytes per LDS row
  static constexpr int CPR = RB / 16;          // 16-byte chunks per row
  static constexpr int RPB = 256 / RB;         // rows per 256 bytes (one pass over all banks)
  static constexpr int RPI = 1024 / RB;        // rows written by one wave-wide direct-to-LDS load
  static constexpr int NI_A = BM / RPI, NI_B = BN / RPI;   // load instructions per slab
  static constexpr int NI = NI_A + NI_B;
  static constexpr int NCOPY = PFD > 0 ? NWAVES / 2 : NWAVES;  // waves that issue the slab copies
  static constexpr int NTOUCH = NWAVES - NCOPY;                // waves that issue L2 warm-up reads instead
  static constexpr int LPW = NI / NCOPY;       // copies per copying wave per slab
  static constexpr int A_BYTES = BM * RB, B_BYTES = BN * RB;
  static constexpr int STAGE_BYTES = A_BYTES + B_BYTES;
  static constexpr int TM = BM / WM / 32, TN = BN / WN / 32;
  static constexpr int NPAT = (RPB * CPR) / RPI > 1 ? (RPB * CPR) / RPI : 1;  // distinct swizzle patterns over load instrs
  static constexpr int EPI_PITCH = (BN / WN) * 2 + 16;   // staged output row pitch in bytes
  static constexpr int EPI_WAVE_BYTES = 32 * EPI_PITCH;
  static constexpr int PFW = PFD > 0 ? ((BM + BN) / 64 + NTOUCH - 1) / NTOUCH : 0;  // warm-up reads per touching wave per slab
  static constexpr int SINK_OFFSET = NSTAGE * STAGE_BYTES + (int)sizeof(SchedTableT<kFastMaxGroups>);
  static constexpr int SMEM_BYTES = SINK_OFFSET + NWAVES * 256;
  static_assert(BM % 64 == 0 && BN % 64 == 0, "warm-up split");
  static_assert(PFD == 0 || BK == 64, "warm-up reads assume one 128-byte line per slab row");
  static_assert(NWAVES * EPI_WAVE_BYTES <= STAGE_BYTES, "epilogue staging must fit in one slab buffer");
  static_assert(NI_A % NCOPY == 0 && NI_B % NCOPY == 0, "copies must divide evenly over the copying waves");
  static_assert(LPW * (NSTAGE - 1) < 64, "vmcnt range");
};

// DBG is a development aid for isolating pipeline stages: bit 0 drops the slab copies, bit 1 the
// fragment reads, bit 2 the MFMAs (results are then meaningless).
template <class C, int DT, int DBG = 0>
__global__ __launch_bounds__(C::THREADS) void gemm_fast_nt_kernel(const GemmParams p) {
  extern __shared__ __attribute__((aligned(1024))) char smem[];
  auto& sched = *reinterpret_cast<SchedTableT<kFastMaxGroups>*>(smem + C::NSTAGE * C::STAGE_BYTES);
  sched_init<C::BM>(p, sched);
  const int64_t num_tiles = sched_num_tiles<C::BM, C::BN>(p, sched);

  const uint32_t smem_addr = (uint32_t)(uintptr_t)(lds_ptr_t)smem;
  const int lane = lane_id();
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int wm0 = (wave / C::WN) * (C::BM / C::WM);
  const int wn0 = (wave % C::WN) * (C::BN / C::WN);
  const int l32 = lane & 31, lh = lane >> 5;
  const int K = p.K;
  const int kt_n = K / C::BK;
  const int row_bytes = K * 2;

  // Per-lane byte offset of a direct-to-LDS load relative to (first row of the instruction, k = 0):
  // lane -> (row l / CPR, LDS slot l % CPR); the slot holds logical chunk slot ^ f(row).
  int ld_voff[C::NPAT];
#pragma unroll
  for (int pt = 0; pt < C::NPAT; ++pt) {
    const int r = pt * C::RPI + lane / C::CPR;
    const int f = (r / C::RPB) % C::CPR;
    ld_voff[pt] = (lane / C::CPR) * row_bytes + (((lane % C::CPR) ^ f) << 4);
  }
  static_assert(C::NCOPY % C::NPAT == 0, "static load split");
  // With warm-up enabled the waves split roles for memory traffic (all of them compute): the lower
  // half issues every slab copy, the upper half only issues warm-up reads.  vmcnt retires in
  // order, so a wave that mixed both would have its copies' completion held up by the slow,
  // far-ahead warm-up reads; a touching wave never waits on vmcnt at all.
  const bool copier = wave < C::NCOPY;
  const int my_voff = ld_voff[wave % C::NPAT];  // every copy of this wave uses the same swizzle pattern
  // Per-lane LDS byte offsets of the fragment reads, relative to the operand's slab base.
  const int fsw = (l32 / C::RPB) % C::CPR;
  int rd_off[C::BK / 16];
#pragma unroll
  for (int ks = 0; ks < C::BK / 16; ++ks) rd_off[ks] = l32 * C::RB + (((2 * ks + lh) ^ fsw) << 4);

  // Buffer descriptors of a tile's A rows and B rows (pinned to scalar registers).
  struct Desc { i32x4_t a, b; };
  auto make_desc = [&](const Tile& t) {
    const int64_t a_rows_left = p.m_total - t.row0;
    const int a_rows = a_rows_left < C::BM ? (int)a_rows_left : C::BM;
    const int b_rows = (p.N - t.n0) < C::BN ? (p.N - t.n0) : C::BN;
    Desc d;
    d.a = make_rsrc((const char*)p.A + t.row0 * (int64_t)row_bytes, (uint32_t)(a_rows * row_bytes));
    d.b = make_rsrc((const char*)p.B + ((int64_t)t.g * p.N + t.n0) * (int64_t)row_bytes, (uint32_t)(b_rows * row_bytes));
    return d;
  };
  // Offsets at or past this marker are outside every descriptor: such a copy fetches nothing (zeros
  // land in LDS that nobody reads) but still occupies its slot in the vmcnt bookkeeping.
  constexpr int kNoFetch = 0x40000000;
  auto issue_slab = [&](const Desc& d, int kt, int buf) {
    const uint32_t base = smem_addr + buf * C::STAGE_BYTES;
    const int koff = kt < kt_n ? kt * (C::BK * 2) : kNoFetch;
    if ((DBG & 1) || !copier) return;
#pragma unroll
    for (int j = 0; j < C::NI_A / C::NCOPY; ++j) {
      const int idx = wave + j * C::NCOPY;  // wave-uniform
      copy_b128_to_lds(d.a, base + idx * 1024, my_voff + idx * C::RPI * row_bytes + koff);
    }
#pragma unroll
    for (int j = 0; j < C::NI_B / C::NCOPY; ++j) {
      const int idx = wave + j * C::NCOPY;
      copy_b128_to_lds(d.b, base + C::A_BYTES + idx * 1024, my_voff + idx * C::RPI * row_bytes + koff);
    }
  };
  // L2 warm-up of a slab that will be copied a few iterations from now: one 4-byte read per
  // 128-byte line (every row of the slab is one line), dropped into a scratch corner of LDS.  The
  // slab copies then hit in L2 instead of waiting on HBM / Infinity Cache inside the barrier.
  const uint32_t sink_addr = smem_addr + C::SINK_OFFSET + wave * 256;
  auto touch_slab = [&](const Desc& d, int kt) {
    if (C::PFD == 0 || (DBG & 1) || copier) return;
    if (kt >= kt_n) return;
    const int koff = kt * (C::BK * 2);
#pragma unroll
    for (int j = 0; j < C::PFW; ++j) {
      const int blk = (wave - C::NCOPY) + j * C::NTOUCH;  // 64-row block of the (A rows, then B rows) list
      const bool is_a = blk * 64 < C::BM;            // wave-uniform
      const int row = blk * 64 - (is_a ? 0 : C::BM) + lane;
      if (blk * 64 < C::BM + C::BN) copy_b32_to_lds(is_a ? d.a : d.b, sink_addr, row * row_bytes + koff);
    }
  };
  // Slab `s` counted from the start of the current tile; past its end it names a slab of the next tile.
  auto touch_ahead = [&](const Desc& cur_d, const Desc& next_d, bool have_next, int s) {
    if (s < kt_n) touch_slab(cur_d, s);
    else if (have_next) touch_slab(next_d, s - kt_n);
  };

  // Epilogue staging: a private region per wave inside slab buffer NSTAGE-1 (free between tiles),
  // 32 rows x (BN/WN) columns of 16-bit outputs, rows padded by 16 bytes.
  char* const stage_c = smem + (C::NSTAGE - 1) * C::STAGE_BYTES + wave * C::EPI_WAVE_BYTES;

  int64_t tile_id = sched_first_tile(p.tile_order);
  Tile t;
  Desc dsc = {{0, 0, 0, 0}, {0, 0, 0, 0}};
  if (tile_id < num_tiles) {
    t = sched_tile<C::BM, C::BN>(p, sched, tile_id);
    dsc = make_desc(t);
#pragma unroll
    for (int s = 0; s < C::NSTAGE - 1; ++s) {
      issue_slab(dsc, s, s);
      touch_slab(dsc, s + C::PFD);
    }
  }
  while (tile_id < num_tiles) {
    // look one tile ahead: its descriptors are needed for warm-up reads near the end of this tile
    const int64_t next_id = tile_id + gridDim.x;
    const bool have_next = next_id < num_tiles;
    Tile nt = t;
    Desc ndsc = dsc;
    if (have_next) {
      nt = sched_tile<C::BM, C::BN>(p, sched, next_id);
      ndsc = make_desc(nt);
    }

    f32x16_t acc[C::TM][C::TN];
#pragma unroll
    for (int i = 0; i < C::TM; ++i)
#pragma unroll
      for (int j = 0; j < C::TN; ++j)
#pragma unroll
        for (int e = 0; e < 16; ++e) acc[i][j][e] = 0.f;

    for (int kt = 0; kt < kt_n; ++kt) {
      if (copier) wait_vmcnt<C::LPW * (C::NSTAGE - 2)>();  // this wave's share of slab kt has landed
      __syncthreads();  // everyone's share of slab kt has landed; everyone is done with slab kt-1
      issue_slab(dsc, kt + C::NSTAGE - 1, (kt + C::NSTAGE - 1) % C::NSTAGE);
      touch_ahead(dsc, ndsc, have_next, kt + C::NSTAGE - 1 + C::PFD);
      const char* sa = smem + (kt % C::NSTAGE) * C::STAGE_BYTES + wm0 * C::RB;
      const char* sb = smem + (kt % C::NSTAGE) * C::STAGE_BYTES + C::A_BYTES + wn0 * C::RB;
#pragma unroll
      for (int ks = 0; ks < C::BK / 16; ++ks) {
        i32x4_t fa[C::TM], fb[C::TN];
#pragma unroll
        for (int i = 0; i < C::TM; ++i) {
          if (DBG & 2) { fa[i][0] = kt + i; fa[i][1] = ks; fa[i][2] = lane; fa[i][3] = i; }
          else fa[i] = *(const i32x4_t*)(sa + rd_off[ks] + i * 32 * C::RB);
        }
#pragma unroll
        for (int j = 0; j < C::TN; ++j) {
          if (DBG & 2) { fb[j][0] = kt; fb[j][1] = ks + j; fb[j][2] = lane; fb[j][3] = j; }
          else fb[j] = *(const i32x4_t*)(sb + rd_off[ks] + j * 32 * C::RB);
        }
#pragma unroll
        for (int i = 0; i < C::TM; ++i)
#pragma unroll
          for (int j = 0; j < C::TN; ++j) {
            if (DBG & 4) { acc[i][j][0] += __builtin_bit_cast(float, fa[i][0] ^ fb[j][1]); acc[i][j][5] += __builtin_bit_cast(float, fa[i][3] ^ fb[j][2]); }
            else acc[i][j] = Mma16<DT>::run(fb[j], fa[i], acc[i][j]);
          }
      }
    }
    if (copier) wait_vmcnt<0>();
    __syncthreads();  // every fragment read of this tile is done: all slab buffers are free

    // Start the next tile's first slabs before draining this tile's results (they were warmed by the
    // touches of this tile's last iterations).
    const Tile cur = t;
    if (have_next) {
      t = nt;
      dsc = ndsc;
#pragma unroll
      for (int s = 0; s < C::NSTAGE - 1; ++s) issue_slab(dsc, s, s);
    }
    tile_id = next_id;

    // Epilogue.  A lane owns row l32 and columns 32 j + 8 q + 4 lh + (0..3) of each 32-row block i:
    // transpose through the wave's LDS staging so that global stores are 16 bytes per lane and
    // whole 128-byte (or longer) row segments per instruction.
    constexpr int WCOLS = C::BN / C::WN;          // columns owned by this wave
    constexpr int CPRW = WCOLS / 8;               // 16-byte chunks per staged row
    constexpr int RPIW = 64 / CPRW;               // rows covered by one wave-wide read
    char* const c_tile = (char*)p.C + ((cur.row0 + wm0) * (int64_t)p.N + cur.n0 + wn0) * 2;
    const int st_row = lane / CPRW, st_chunk = lane % CPRW;
    const bool col_ok = cur.n0 + wn0 + st_chunk * 8 < p.N;
#pragma unroll
    for (int i = 0; i < C::TM; ++i) {
#pragma unroll
      for (int j = 0; j < C::TN; ++j)
#pragma unroll
        for (int q = 0; q < 4; ++q)
          *(uint2*)(stage_c + l32 * C::EPI_PITCH + (32 * j + 8 * q + 4 * lh) * 2) =
              pack4<DT>(acc[i][j][4 * q], acc[i][j][4 * q + 1], acc[i][j][4 * q + 2], acc[i][j][4 * q + 3]);
#pragma unroll
      for (int it = 0; it < 32 / RPIW; ++it) {
        const int r = it * RPIW + st_row;
        const i32x4_t v = *(const i32x4_t*)(stage_c + r * C::EPI_PITCH + st_chunk * 16);
        if (col_ok && wm0 + 32 * i + r < cur.rows)
          *(i32x4_t*)(c_tile + ((int64_t)(32 * i + r) * p.N + st_chunk * 8) * 2) = v;
      }
    }
  }
}

int g_tile_order = 0;

template <class C, int DT, int DBG = 0>
int launch_cfg(const GemmParams& p, hipStream_t s) {
  static bool attr_set[64] = {false};
  int dev = 0;
  (void)hipGetDevice(&dev);
  auto kern = gemm_fast_nt_kernel<C, DT, DBG>;
  if (dev >= 0 && dev < 64 && !attr_set[dev]) {
    if (hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize, C::SMEM_BYTES) != hipSuccess)
      return check_launch("hipFuncSetAttribute(gemm_fast)");
    attr_set[dev] = true;
  }
  int grid = num_cus();
  if (p.grid_limit > 0 && p.grid_limit < grid) grid = p.grid_limit;
  GemmParams q = p;
  q.tile_order = g_tile_order;
  hipLaunchKernelGGL(kern, dim3(grid), dim3(C::THREADS), C::SMEM_BYTES, s, q);
  return check_launch("gemm_fast");
}

int g_variant = 0;

template <int DT>
int launch_variant(const GemmParams& p, hipStream_t s) {
  switch (g_variant) {
    default:
    case 0: return launch_cfg<FastCfg<256, 256, 64, 2, 2, 4>, DT>(p, s);
    case 1: return launch_cfg<FastCfg<256, 256, 64, 2, 2, 2>, DT>(p, s);
    case 2: return launch_cfg<FastCfg<256, 128, 64, 3, 4, 2>, DT>(p, s);
    case 3: return launch_cfg<FastCfg<256, 128, 64, 3, 2, 2>, DT>(p, s);
    case 4: return launch_cfg<FastCfg<256, 128, 64, 3, 2, 4>, DT>(p, s);
    case 5: return launch_cfg<FastCfg<128, 256, 64, 3, 2, 2>, DT>(p, s);
    case 6: return launch_cfg<FastCfg<256, 128, 64, 2, 2, 4>, DT>(p, s);
    case 7: return launch_cfg<FastCfg<128, 128, 64, 4, 2, 2>, DT>(p, s);
    case 8: return launch_cfg<FastCfg<256, 256, 64, 2, 2, 4, 0>, DT>(p, s);
    case 9: return launch_cfg<FastCfg<256, 256, 64, 2, 2, 4, 3>, DT>(p, s);
    case 16: return launch_cfg<FastCfg<256, 256, 64, 2, 2, 4, 1>, DT>(p, s);
    case 17: return launch_cfg<FastCfg<256, 256, 64, 2, 2, 4, 4>, DT>(p, s);
    case 10: return launch_cfg<FastCfg<256, 256, 64, 2, 2, 4>, DT, 1>(p, s);
    case 11: return launch_cfg<FastCfg<256, 256, 64, 2, 2, 4>, DT, 2>(p, s);
    case 12: return launch_cfg<FastCfg<256, 256, 64, 2, 2, 4>, DT, 4>(p, s);
    case 13: return launch_cfg<FastCfg<256, 256, 64, 2, 2, 4>, DT, 3>(p, s);
    case 14: return launch_cfg<FastCfg<256, 256, 64, 2, 2, 4>, DT, 6>(p, s);
    case 15: return launch_cfg<FastCfg<256, 256, 64, 2, 2, 4>, DT, 5>(p, s);
    case 20: return launch_cfg<FastCfg<256, 256, 64, 2, 2, 2>, DT, 1>(p, s);
    case 21: return launch_cfg<FastCfg<256, 256, 64, 2, 2, 2>, DT, 2>(p, s);
    case 23: return launch_cfg<FastCfg<256, 256, 64, 2, 2, 2>, DT, 3>(p, s);
  }
}

}  // namespace

void set_fast_variant(int v) { g_variant = v; }
void set_tile_order(int v) { g_tile_order = v; }

bool fast_supported(const GemmParams& p, int dt, int layout) {
  if (layout != 0) return false;
  if (dt != DT_BF16 && dt != DT_F16) return false;
  if (p.mode != MODE_MG && p.mode != MODE_MG_PAD && p.mode != MODE_MASKED) return false;
  if (p.G > kFastMaxGroups) return false;
  if (p.K < 64 || (p.K % 64) != 0) return false;
  if ((int64_t)p.K * 2 * 256 >= (1ll << 30)) return false;  // slab offsets stay far below the out-of-range marker
  return true;
}

int launch_fast_16bit(const GemmParams& p, int dt, int layout, hipStream_t s) {
  (void)layout;
  if (dt == DT_BF16) return launch_variant<DT_BF16>(p, s);
  return launch_variant<DT_F16>(p, s);
}

}  // namespace tgg
