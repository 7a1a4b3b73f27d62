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

template <int BM_, int BN_, int BK_, int NSTAGE_, int WM_, int WN_>
struct FastCfg {
  static constexpr int BM = BM_, BN = BN_, BK = BK_, NSTAGE = NSTAGE_, WM = WM_, WN = WN_;
  static constexpr int NWAVES = WM * WN;
  static constexpr int THREADS = NWAVES * 64;
  static constexpr int RB = BK * 2;            // bytes per LDS row
  static constexpr int CPR = RB / 16;          // 16-byte chunks per row
  static constexpr int RPB = 256 / RB;         // rows per 256 bytes (one pass over all banks)
  static constexpr int RPI = 1024 / RB;        // rows written by one wave-wide direct-to-LDS load
  static constexpr int NI_A = BM / RPI, NI_B = BN / RPI;   // load instructions per slab
  static constexpr int NI = NI_A + NI_B;
  static constexpr int LPW = NI / NWAVES;      // loads per wave per slab
  static constexpr int A_BYTES = BM * RB, B_BYTES = BN * RB;
  static constexpr int STAGE_BYTES = A_BYTES + B_BYTES;
  static constexpr int TM = BM / WM / 32, TN = BN / WN / 32;
  static constexpr int NPAT = (RPB * CPR) / RPI > 1 ? (RPB * CPR) / RPI : 1;  // distinct swizzle patterns over load instrs
  static constexpr int SMEM_BYTES = NSTAGE * STAGE_BYTES + (int)sizeof(SchedTableT<kFastMaxGroups>);
  static_assert(NI_A % NWAVES == 0 && NI_B % NWAVES == 0, "loads must divide evenly over waves");
  static_assert(LPW * (NSTAGE - 1) < 64, "vmcnt range");
};

template <class C, int DT>
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
  static_assert(C::NWAVES % C::NPAT == 0 && C::NI_A % C::NWAVES == 0 && C::NI_B % C::NWAVES == 0, "static load split");
  const int my_voff = ld_voff[wave % C::NPAT];  // every load of this wave uses the same swizzle pattern
  // Per-lane LDS byte offsets of the fragment reads, relative to the operand's slab base.
  const int fsw = (l32 / C::RPB) % C::CPR;
  int rd_off[C::BK / 16];
#pragma unroll
  for (int ks = 0; ks < C::BK / 16; ++ks) rd_off[ks] = l32 * C::RB + (((2 * ks + lh) ^ fsw) << 4);

  for (int64_t tile_id = sched_first_tile(); tile_id < num_tiles; tile_id += gridDim.x) {
    const Tile t = sched_tile<C::BM, C::BN>(p, sched, tile_id);
    const int64_t a_rows_left = p.m_total - t.row0;
    const int a_rows = a_rows_left < C::BM ? (int)a_rows_left : C::BM;
    const int b_rows = (p.N - t.n0) < C::BN ? (p.N - t.n0) : C::BN;
    const i32x4_t rsrc_a = make_rsrc((const char*)p.A + t.row0 * (int64_t)row_bytes, (uint32_t)(a_rows * row_bytes));
    const i32x4_t rsrc_b = make_rsrc((const char*)p.B + ((int64_t)t.g * p.N + t.n0) * (int64_t)row_bytes,
                                     (uint32_t)(b_rows * row_bytes));

    auto issue_slab = [&](int kt, int buf) {
      const uint32_t base = smem_addr + buf * C::STAGE_BYTES;
      // past the last slab the offset is pushed out of the descriptor's range: nothing is fetched,
      // zeros land in a buffer nobody reads, and the vmcnt bookkeeping stays uniform
      const int koff = kt < kt_n ? kt * (C::BK * 2) : 0x40000000;
#pragma unroll
      for (int j = 0; j < C::NI_A / C::NWAVES; ++j) {
        const int idx = wave + j * C::NWAVES;  // wave-uniform
        copy_b128_to_lds(rsrc_a, base + idx * 1024, my_voff + idx * C::RPI * row_bytes + koff);
      }
#pragma unroll
      for (int j = 0; j < C::NI_B / C::NWAVES; ++j) {
        const int idx = wave + j * C::NWAVES;
        copy_b128_to_lds(rsrc_b, base + C::A_BYTES + idx * 1024, my_voff + idx * C::RPI * row_bytes + koff);
      }
    };

    f32x16_t acc[C::TM][C::TN];
#pragma unroll
    for (int i = 0; i < C::TM; ++i)
#pragma unroll
      for (int j = 0; j < C::TN; ++j)
#pragma unroll
        for (int e = 0; e < 16; ++e) acc[i][j][e] = 0.f;

#pragma unroll
    for (int s = 0; s < C::NSTAGE - 1; ++s) issue_slab(s, s);

    for (int kt = 0; kt < kt_n; ++kt) {
      wait_vmcnt<C::LPW * (C::NSTAGE - 2)>();  // this wave's share of slab kt has landed
      __syncthreads();                          // everyone's share has; everyone is done with slab kt-1
      issue_slab(kt + C::NSTAGE - 1, (kt + C::NSTAGE - 1) % C::NSTAGE);
      const char* sa = smem + (kt % C::NSTAGE) * C::STAGE_BYTES + wm0 * C::RB;
      const char* sb = smem + (kt % C::NSTAGE) * C::STAGE_BYTES + C::A_BYTES + wn0 * C::RB;
#pragma unroll
      for (int ks = 0; ks < C::BK / 16; ++ks) {
        i32x4_t fa[C::TM], fb[C::TN];
#pragma unroll
        for (int i = 0; i < C::TM; ++i) fa[i] = *(const i32x4_t*)(sa + rd_off[ks] + i * 32 * C::RB);
#pragma unroll
        for (int j = 0; j < C::TN; ++j) fb[j] = *(const i32x4_t*)(sb + rd_off[ks] + j * 32 * C::RB);
#pragma unroll
        for (int i = 0; i < C::TM; ++i)
#pragma unroll
          for (int j = 0; j < C::TN; ++j) acc[i][j] = Mma16<DT>::run(fb[j], fa[i], acc[i][j]);
      }
    }
    wait_vmcnt<0>();
    __syncthreads();  // all fragment reads of this tile are done before the next tile's loads land

    // epilogue: lane owns row m = wm0 + 32 i + l32 and columns wn0 + 32 j + 8 q + 4 lh + (0..3)
    char* c_row = (char*)p.C + ((t.row0 + wm0 + l32) * (int64_t)p.N + t.n0 + wn0 + 4 * lh) * 2;
#pragma unroll
    for (int i = 0; i < C::TM; ++i) {
      __builtin_amdgcn_sched_barrier(0);
      if (wm0 + 32 * i + l32 < t.rows) {
#pragma unroll
        for (int j = 0; j < C::TN; ++j)
#pragma unroll
          for (int q = 0; q < 4; ++q) {
            const int n = t.n0 + wn0 + 32 * j + 8 * q + 4 * lh;
            if (n < p.N)
              *(uint2*)(c_row + ((int64_t)(32 * i) * p.N + 32 * j + 8 * q) * 2) =
                  pack4<DT>(acc[i][j][4 * q], acc[i][j][4 * q + 1], acc[i][j][4 * q + 2], acc[i][j][4 * q + 3]);
          }
      }
    }
  }
}

template <class C, int DT>
int launch_cfg(const GemmParams& p, hipStream_t s) {
  static bool attr_set[64] = {false};
  int dev = 0;
  (void)hipGetDevice(&dev);
  auto kern = gemm_fast_nt_kernel<C, DT>;
  if (dev >= 0 && dev < 64 && !attr_set[dev]) {
    if (hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize, C::SMEM_BYTES) != hipSuccess)
      return check_launch("hipFuncSetAttribute(gemm_fast)");
    attr_set[dev] = true;
  }
  int grid = num_cus();
  if (p.grid_limit > 0 && p.grid_limit < grid) grid = p.grid_limit;
  hipLaunchKernelGGL(kern, dim3(grid), dim3(C::THREADS), C::SMEM_BYTES, s, p);
  return check_launch("gemm_fast");
}

int g_variant = 0;

template <int DT>
int launch_variant(const GemmParams& p, hipStream_t s) {
  switch (g_variant) {
    default:
    case 0: return launch_cfg<FastCfg<256, 256, 32, 4, 2, 2>, DT>(p, s);
    case 1: return launch_cfg<FastCfg<256, 256, 64, 2, 2, 2>, DT>(p, s);
    case 2: return launch_cfg<FastCfg<256, 256, 32, 4, 2, 4>, DT>(p, s);
    case 3: return launch_cfg<FastCfg<256, 256, 64, 2, 2, 4>, DT>(p, s);
    case 4: return launch_cfg<FastCfg<256, 128, 32, 4, 2, 2>, DT>(p, s);
    case 5: return launch_cfg<FastCfg<256, 128, 64, 3, 2, 2>, DT>(p, s);
    case 6: return launch_cfg<FastCfg<128, 128, 64, 4, 2, 2>, DT>(p, s);
    case 7: return launch_cfg<FastCfg<256, 256, 32, 3, 2, 2>, DT>(p, s);
  }
}

}  // namespace

void set_fast_variant(int v) { g_variant = v; }

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
