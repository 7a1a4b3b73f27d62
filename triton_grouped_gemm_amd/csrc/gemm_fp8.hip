// Tuned FP8 (OCP e4m3fn / e5m2) grouped GEMM kernels for gfx950, K-contiguous operands.
//
// Same skeleton as the 16-bit kernels (persistent grouped tiles, direct-to-LDS slabs, swizzled
// LDS, staged epilogue); a slab is 128 bytes = 128 K values of every row, i.e. exactly one
// 128-wide scale block.  The contraction runs on v_mfma_f32_32x32x64_f8f6f4.
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

namespace tgg {

namespace {

enum : int { EPI_CHANNEL = 1, EPI_BLOCK = 2 };
constexpr int BKB = 128;  // K depth of a slab in fp8 values (= bytes)

// One copy of 4 bytes per lane global -> LDS (destination m0 + lane * 4).
TGG_DEV void copy_b32_to_lds(i32x4_t rsrc, uint32_t lds_addr, int voff) {
  asm volatile("s_mov_b32 m0, %0\n\tbuffer_load_dword %1, %2, 0 offen lds" : : "s"(lds_addr), "v"(voff), "s"(rsrc) : "memory");
}

TGG_DEV i32x4_t raw_rsrc(uint64_t a, int64_t bytes) {
  bytes = bytes < 0 ? 0 : (bytes > 0x7fffffff ? 0x7fffffff : bytes);
  i32x4_t r;
  r[0] = __builtin_amdgcn_readfirstlane((int)(uint32_t)a);
  r[1] = __builtin_amdgcn_readfirstlane((int)(uint32_t)(a >> 32) & 0xffff);
  r[2] = __builtin_amdgcn_readfirstlane((int)bytes);
  r[3] = 0x00020000;
  return r;
}

template <int BM_, int BN_, int NSTAGE_, int WM_, int WN_>
struct Fp8Cfg {
  static constexpr int BM = BM_, BN = BN_, NSTAGE = NSTAGE_, WM = WM_, WN = WN_;
  static constexpr int NWAVES = WM * WN;
  static constexpr int THREADS = NWAVES * 64;
  static constexpr int A_BYTES = BM * 128, B_BYTES = BN * 128;
  static constexpr int SA_BYTES = BM * 4 + 256;  // activation scales of the slab's rows + a sink for spare waves' copies
  static constexpr int STAGE_BYTES = A_BYTES + B_BYTES + SA_BYTES;
  static constexpr int NI_A = A_BYTES / 1024, NI_B = B_BYTES / 1024;
  static constexpr int TM = BM / WM / 32, TN = BN / WN / 32;
  static constexpr int EPI_PITCH = (BN / WN) * 2 + 16;
  static constexpr int EPI_WAVE_BYTES = 32 * EPI_PITCH;
  static constexpr int SMEM_BYTES = NSTAGE * STAGE_BYTES + (int)sizeof(SchedTableT<kFastMaxGroups>);
  static_assert(NI_A % NWAVES == 0 && NI_B % NWAVES == 0, "copies must divide evenly over waves");
  static_assert(NWAVES % 2 == 0 && BM / 64 <= NWAVES, "scale copies: one per wave");
  static_assert((BN / WN) <= 128, "a wave's columns must share one 128-wide weight scale block");
  static_assert(NWAVES * EPI_WAVE_BYTES <= A_BYTES + B_BYTES, "epilogue staging must fit in one slab buffer");
};

// FA / FB: 0 = e4m3fn, 1 = e5m2 (the cbsz / blgp format codes of the f8f6f4 MFMA).
template <class C, int FA, int FB, int EPI, int OUT, bool KGROUP>
__global__ __launch_bounds__(C::THREADS) void gemm_fp8_kernel(const GemmParams p) {
  typedef Operand<C::BM, true> OpA;
  typedef Operand<C::BN, true> OpB;
  constexpr int LPW = (C::NI_A + C::NI_B) / C::NWAVES + (EPI == EPI_BLOCK ? 1 : 0);  // copies per wave per slab
  static_assert(LPW * (C::NSTAGE - 1) < 64, "vmcnt range");

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

  const int64_t ld = KGROUP ? p.k_total : (int64_t)p.K;  // bytes between consecutive rows of A and of B
  const int a_voff = OpA::lane_voff(lane, wave % OpA::NPAT, (int)ld);
  const int b_voff = OpB::lane_voff(lane, wave % OpB::NPAT, (int)ld);
  const int kblocks = (p.K + 127) >> 7;
  const int nblocks = (p.N + 127) >> 7;

  // LDS offsets of a lane's 32 bytes of fragment (64-deep MFMA step ks): chunks 4 ks + 2 lh + {0, 1}
  const int fsw = (l32 / 2) % 8;
  int rd[2][2];
#pragma unroll
  for (int ks = 0; ks < 2; ++ks)
#pragma unroll
    for (int h = 0; h < 2; ++h) rd[ks][h] = l32 * 128 + (((4 * ks + 2 * lh + h) ^ fsw) << 4);

  struct TileIo { Stream a, b; uint64_t sa_base; int sa_bytes; int kt_n; };
  auto make_io = [&](const Tile& t) {
    TileIo io;
    const int64_t k0 = KGROUP ? t.k0 : 0;
    io.kt_n = KGROUP ? (int)((t.k1 - t.k0 + BKB - 1) / BKB) : p.K / BKB;
    const int64_t rows_left = p.m_total - t.row0;
    const int a_rows = (int)(rows_left < C::BM ? rows_left : C::BM);
    const int n_left = p.N - t.n0;
    io.a.base = (uint64_t)p.A + (uint64_t)(t.row0 * ld + k0);
    io.a.bytes = (int64_t)a_rows * ld - k0;
    io.a.step = BKB;
    io.b.base = (uint64_t)p.B + (uint64_t)((KGROUP ? (int64_t)t.n0 : ((int64_t)t.g * p.N + t.n0)) * ld + k0);
    io.b.bytes = (int64_t)(n_left < C::BN ? n_left : C::BN) * ld - k0;
    io.b.step = BKB;
    io.sa_base = 0;
    io.sa_bytes = 0;
    if (EPI == EPI_BLOCK) {
      io.sa_base = (uint64_t)(p.sa + t.row0);   // [kblocks, m_total]: row kb starts m_total floats further
      io.sa_bytes = a_rows * 4;
    }
    return io;
  };
  // Weight scales of this wave's column block for every slab of a tile: lane kb holds block kb.
  // This is an ordinary vector load, so the compiler waits for *all* outstanding vector memory
  // traffic at its first use; it is therefore fetched one tile ahead and first touched right after
  // the end-of-tile drain, where nothing is in flight anyway.
  auto load_sbv = [&](const Tile& t) {
    const int64_t idx = ((int64_t)t.g * nblocks + ((t.n0 + wn0) >> 7)) * kblocks;
    return (EPI == EPI_BLOCK && lane < kblocks) ? p.sb[idx + lane] : 0.f;
  };
  constexpr int kNoFetch = 0x40000000;
  auto issue_slab = [&](const TileIo& io, int kt, int buf) {
    const uint32_t base = smem_addr + buf * C::STAGE_BYTES;
    const int ktc = kt < io.kt_n ? kt : 0;
    const int dead = kt < io.kt_n ? 0 : kNoFetch;
    const i32x4_t ra = stream_rsrc(io.a, ktc), rb = stream_rsrc(io.b, ktc);
#pragma unroll
    for (int j = 0; j < C::NI_A / C::NWAVES; ++j) {
      const int idx = wave + j * C::NWAVES;
      copy_b128_to_lds(ra, base + idx * 1024, a_voff + idx * OpA::RPI * (int)ld + dead);
    }
#pragma unroll
    for (int j = 0; j < C::NI_B / C::NWAVES; ++j) {
      const int idx = wave + j * C::NWAVES;
      copy_b128_to_lds(rb, base + C::A_BYTES + idx * 1024, b_voff + idx * OpB::RPI * (int)ld + dead);
    }
    if (EPI == EPI_BLOCK) {
      // activation scales of this slab's rows: wave w fetches rows 64 w .. 64 w + 63 (spare waves issue
      // an out-of-range copy so that every wave has the same number of copies in flight)
      const i32x4_t rs = raw_rsrc(io.sa_base + (uint64_t)ktc * (uint64_t)p.m_total * 4, io.sa_bytes);
      const int off = wave * 64 < C::BM ? (wave * 64 + lane) * 4 + dead : kNoFetch;
      copy_b32_to_lds(rs, base + C::A_BYTES + C::B_BYTES + (wave * 64 < C::BM ? wave * 256 : C::BM * 4), off);
    }
  };

  char* const stage_c = smem + (C::NSTAGE - 1) * C::STAGE_BYTES + wave * C::EPI_WAVE_BYTES;

  const TileWalk walk = sched_walk(num_tiles, !KGROUP && p.tile_split);
  int64_t tile_id = walk.first;
  Tile t;
  TileIo io;
  float sbv = 0.f;
  if (tile_id < walk.end) {
    t = sched_tile<C::BM, C::BN>(p, sched, tile_id);
    io = make_io(t);
    sbv = load_sbv(t);
    asm volatile("" : "+v"(sbv));
#pragma unroll
    for (int s = 0; s < C::NSTAGE - 1; ++s) issue_slab(io, s, s);
  }
  while (tile_id < walk.end) {
    const int64_t next_id = tile_id + walk.stride;
    Tile nt = t;
    float sbv_next = 0.f;
    if (next_id < walk.end) {
      nt = sched_tile<C::BM, C::BN>(p, sched, next_id);
      sbv_next = load_sbv(nt);
    }
    f32x16_t acc[C::TM][C::TN];
#pragma unroll
    for (int i = 0; i < C::TM; ++i)
#pragma unroll
      for (int j = 0; j < C::TN; ++j)
#pragma unroll
        for (int e = 0; e < 16; ++e) acc[i][j][e] = 0.f;

    const int kt_n = io.kt_n;
    for (int kt = 0; kt < kt_n; ++kt) {
      wait_vmcnt<LPW * (C::NSTAGE - 2)>();
      __syncthreads();
      issue_slab(io, kt + C::NSTAGE - 1, (kt + C::NSTAGE - 1) % C::NSTAGE);
      const float sb_cur = EPI == EPI_BLOCK ? __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, sbv), kt)) : 1.f;
      const char* sa = smem + (kt % C::NSTAGE) * C::STAGE_BYTES + wm0 * 128;
      const char* sb = smem + (kt % C::NSTAGE) * C::STAGE_BYTES + C::A_BYTES + wn0 * 128;
      const float* ss = (const float*)(smem + (kt % C::NSTAGE) * C::STAGE_BYTES + C::A_BYTES + C::B_BYTES) + wm0 + l32;

      i32x8_t fb[2][C::TN];
#pragma unroll
      for (int ks = 0; ks < 2; ++ks)
#pragma unroll
        for (int j = 0; j < C::TN; ++j) {
          const i32x4_t lo = *(const i32x4_t*)(sb + rd[ks][0] + j * 32 * 128);
          const i32x4_t hi = *(const i32x4_t*)(sb + rd[ks][1] + j * 32 * 128);
          fb[ks][j] = __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
        }
#pragma unroll
      for (int i = 0; i < C::TM; ++i) {
        i32x8_t fa[2];
#pragma unroll
        for (int ks = 0; ks < 2; ++ks) {
          const i32x4_t lo = *(const i32x4_t*)(sa + rd[ks][0] + i * 32 * 128);
          const i32x4_t hi = *(const i32x4_t*)(sa + rd[ks][1] + i * 32 * 128);
          fa[ks] = __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
        }
        float s = 0.f;
        if (EPI == EPI_BLOCK) s = ss[32 * i] * sb_cur;
#pragma unroll
        for (int j = 0; j < C::TN; ++j) {
          if (EPI == EPI_BLOCK) {
            f32x16_t part = {0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0};
            part = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(fb[0][j], fa[0], part, FB, FA, 0, 0, 0, 0);
            part = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(fb[1][j], fa[1], part, FB, FA, 0, 0, 0, 0);
#pragma unroll
            for (int e = 0; e < 16; ++e) acc[i][j][e] += part[e] * s;
          } else {
            acc[i][j] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(fb[0][j], fa[0], acc[i][j], FB, FA, 0, 0, 0, 0);
            acc[i][j] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(fb[1][j], fa[1], acc[i][j], FB, FA, 0, 0, 0, 0);
          }
        }
      }
    }
    wait_vmcnt<0>();
    asm volatile("" : "+v"(sbv_next));
    sbv = sbv_next;
    __syncthreads();

    const Tile cur = t;
    if (next_id < walk.end) {
      t = nt;
      io = make_io(t);
#pragma unroll
      for (int s = 0; s < C::NSTAGE - 1; ++s) issue_slab(io, s, s);
    }
    tile_id = next_id;

    // Epilogue (see gemm_fast.hip): per-channel scaling happens on the fp32 values before packing.
    constexpr int WCOLS = C::BN / C::WN, CPRW = WCOLS / 8, RPIW = 64 / CPRW;
    const int64_t c_row0 = KGROUP ? ((int64_t)cur.g * p.m_total + cur.row0) : cur.row0;
    char* const c_tile = (char*)p.C + ((c_row0 + wm0) * (int64_t)p.N + cur.n0 + wn0) * 2;
    const int st_row = lane / CPRW, st_chunk = lane % CPRW;
    const bool col_ok = cur.n0 + wn0 + st_chunk * 8 < p.N;
#pragma unroll
    for (int i = 0; i < C::TM; ++i) {
      float rs = 1.f;
      if (EPI == EPI_CHANNEL) {
        const int m = wm0 + 32 * i + l32;
        rs = m < cur.rows ? p.scale_m[(KGROUP ? (int64_t)cur.g * p.scale_m_sg : 0) + cur.row0 + m] : 0.f;
      }
#pragma unroll
      for (int j = 0; j < C::TN; ++j)
#pragma unroll
        for (int q = 0; q < 4; ++q) {
          float v[4];
#pragma unroll
          for (int e = 0; e < 4; ++e) v[e] = acc[i][j][4 * q + e];
          if (EPI == EPI_CHANNEL) {
            const int n = cur.n0 + wn0 + 32 * j + 8 * q + 4 * lh;
#pragma unroll
            for (int e = 0; e < 4; ++e) v[e] = (n + e < p.N) ? v[e] * rs * p.scale_n[(int64_t)cur.g * p.N + n + e] : 0.f;
          }
          *(uint2*)(stage_c + l32 * C::EPI_PITCH + (32 * j + 8 * q + 4 * lh) * 2) = pack4<OUT>(v[0], v[1], v[2], v[3]);
        }
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

template <class C, int FA, int FB, int EPI, int OUT, bool KGROUP>
int launch_fp8_cfg(const GemmParams& p, hipStream_t s) {
  static bool attr_set[64] = {false};
  int dev = 0;
  (void)hipGetDevice(&dev);
  auto kern = gemm_fp8_kernel<C, FA, FB, EPI, OUT, KGROUP>;
  if (dev >= 0 && dev < 64 && !attr_set[dev]) {
    if (hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize, C::SMEM_BYTES) != hipSuccess)
      return check_launch("hipFuncSetAttribute(gemm_fp8)");
    attr_set[dev] = true;
  }
  int grid = num_cus();
  if (p.grid_limit > 0 && p.grid_limit < grid) grid = p.grid_limit;
  hipLaunchKernelGGL(kern, dim3(grid), dim3(C::THREADS), C::SMEM_BYTES, s, p);
  return check_launch("gemm_fp8");
}

typedef Fp8Cfg<256, 256, 2, 2, 4> Fp8Default;

template <int FA, int FB, bool KGROUP>
int launch_channel_out(const GemmParams& p, int out_dt, hipStream_t s) {
  if (out_dt == DT_BF16) return launch_fp8_cfg<Fp8Default, FA, FB, EPI_CHANNEL, DT_BF16, KGROUP>(p, s);
  if (out_dt == DT_F16) return launch_fp8_cfg<Fp8Default, FA, FB, EPI_CHANNEL, DT_F16, KGROUP>(p, s);
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

// K-contiguous fp8 operands with every reduction range a multiple of the 128-deep slab.
bool fast_fp8_supported(const GemmParams& p, bool block_scaled) {
  if (p.G > kFastMaxGroups) return false;
  if ((p.N & 7) != 0) return false;
  const bool kgroup = p.mode == MODE_KG_COUNT;
  if (kgroup) {
    if (block_scaled) return false;
    return (p.k_total % BKB) == 0 && p.k_total * 256 < (1ll << 30);
  }
  if (p.mode != MODE_MG && p.mode != MODE_MG_PAD) return false;
  if (p.K < BKB || (p.K % BKB) != 0) return false;
  return (int64_t)p.K * 256 < (1ll << 30);
}

int launch_fast_fp8_channel(const GemmParams& p, int ta, int tb, int out_dt, hipStream_t s) {
  if (p.mode == MODE_KG_COUNT) return launch_channel_fmt<true>(p, ta, tb, out_dt, s);
  return launch_channel_fmt<false>(p, ta, tb, out_dt, s);
}

// sa must be laid out [ceil(K/128), m_total] (row-block major) for this kernel.
int launch_fast_fp8_block(const GemmParams& p, hipStream_t s) {
  return launch_fp8_cfg<Fp8Default, 0, 0, EPI_BLOCK, DT_BF16, false>(p, s);
}

}  // namespace tgg
