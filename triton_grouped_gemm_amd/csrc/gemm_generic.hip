// Shape-agnostic grouped GEMM for gfx950: any group sizes, K tails, both operand
// majors, bf16/fp16/fp8 inputs, plain / per-channel / 128-block scaled epilogues.
//
// 128x128x32 tile, 256 threads (2x2 waves, each 64x64 = 2x2 MFMA 32x32x16),
// operands staged global -> VGPR -> LDS (K-contiguous rows, 16 B row padding),
// register prefetch of the next K slab, double-buffered LDS, one barrier per slab.
// The MFMA is issued with the operands swapped (weights as srcA, activations as
// srcB) so every lane ends up owning 4 consecutive output columns of one row.
//
// This is the kernel every entry point can fall back on; the tuned kernels in
// gemm_fast.hip take over for the aligned shapes.
#include "common.hpp"
#include "sched.hpp"
#include "generic_addr.hpp"
#include "launch.hpp"

namespace tgg {

namespace {

constexpr int GBM = kGenericBM, GBN = kGenericBN, GBK = kGenericBK, GTHREADS = 256;

template <int DT> struct ElemSize { static constexpr int v = (DT <= DT_F16) ? 2 : 1; };

// One MFMA operand: 8 consecutive K elements of one row.
template <int DT> struct Frag;
template <> struct Frag<DT_BF16> { typedef i32x4_t type; };
template <> struct Frag<DT_F16> { typedef i32x4_t type; };
template <> struct Frag<DT_E4M3> { typedef long type; };
template <> struct Frag<DT_E5M2> { typedef long type; };

// acc[n][m] += sum_k w[n][k] * x[m][k]
template <int TW, int TX> struct Mma;
template <> struct Mma<DT_BF16, DT_BF16> {
  static TGG_DEV f32x16_t run(i32x4_t w, i32x4_t x, f32x16_t c) {
    return __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8_t, w), __builtin_bit_cast(bf16x8_t, x), c, 0, 0, 0);
  }
};
template <> struct Mma<DT_F16, DT_F16> {
  static TGG_DEV f32x16_t run(i32x4_t w, i32x4_t x, f32x16_t c) {
    return __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(f16x8_t, w), __builtin_bit_cast(f16x8_t, x), c, 0, 0, 0);
  }
};
template <> struct Mma<DT_E4M3, DT_E4M3> {
  static TGG_DEV f32x16_t run(long w, long x, f32x16_t c) { return __builtin_amdgcn_mfma_f32_32x32x16_fp8_fp8(w, x, c, 0, 0, 0); }
};
template <> struct Mma<DT_E4M3, DT_E5M2> {
  static TGG_DEV f32x16_t run(long w, long x, f32x16_t c) { return __builtin_amdgcn_mfma_f32_32x32x16_fp8_bf8(w, x, c, 0, 0, 0); }
};
template <> struct Mma<DT_E5M2, DT_E4M3> {
  static TGG_DEV f32x16_t run(long w, long x, f32x16_t c) { return __builtin_amdgcn_mfma_f32_32x32x16_bf8_fp8(w, x, c, 0, 0, 0); }
};
template <> struct Mma<DT_E5M2, DT_E5M2> {
  static TGG_DEV f32x16_t run(long w, long x, f32x16_t c) { return __builtin_amdgcn_mfma_f32_32x32x16_bf8_bf8(w, x, c, 0, 0, 0); }
};

// First nbytes (< 16) bytes of a 16-byte vector, the rest zero.
TGG_DEV i32x4_t load_partial(const char* src, int nbytes) {
  i32x4_t r = {0, 0, 0, 0};
#pragma unroll
  for (int b = 0; b < 16; ++b)
    if (b < nbytes) r[b >> 2] |= (int)((uint32_t)(uint8_t)src[b] << ((b & 3) * 8));
  return r;
}

// Global -> register staging of one 128 x 32 operand slab.
// KMAJOR: rows are K-contiguous (row stride s_row, unit K stride).
// !KMAJOR: K rows are MN-contiguous (K stride s_k, unit MN stride); 16-bit only.
template <int DT, bool KMAJOR> struct Stager {
  static constexpr int ES = ElemSize<DT>::v;
  static constexpr int VEC = 16 / ES;                      // elements per 16-byte vector
  static constexpr int NVEC = (128 * GBK) / VEC / GTHREADS; // vectors per thread
  static constexpr int PITCH = GBK * ES + 16;              // LDS row pitch in bytes
  i32x4_t v[NVEC];

  // base: element (row 0 of the tile, k = 0 of the whole operand); lim_mn: rows of the tile that may be read
  TGG_DEV void load(const char* base, int64_t s_row, int64_t s_k, int lim_mn, int64_t k, int64_t k_end) {
#pragma unroll
    for (int i = 0; i < NVEC; ++i) {
      const int idx = threadIdx.x + i * GTHREADS;
      i32x4_t val = {0, 0, 0, 0};
      if (KMAJOR) {
        constexpr int VPR = GBK / VEC;
        const int row = idx / VPR;
        const int64_t kk = k + (idx % VPR) * VEC;
        if (row < lim_mn && kk < k_end) {
          const char* src = base + generic_elem_kmajor(row, s_row, kk) * ES;
          if (kk + VEC <= k_end) val = *(const i32x4_t*)src;
          else val = load_partial(src, (int)(k_end - kk) * ES);
        }
      } else {
        constexpr int VPR = 128 / VEC;
        const int krow = idx / VPR;
        const int mn = (idx % VPR) * VEC;
        const int64_t kk = k + krow;
        if (kk < k_end && mn < lim_mn) {
          const char* src = base + generic_elem_mnmajor(kk, s_k, mn) * ES;
          if (mn + VEC <= lim_mn) val = *(const i32x4_t*)src;
          else val = load_partial(src, (lim_mn - mn) * ES);
        }
      }
      v[i] = val;
    }
  }

  TGG_DEV void store(char* lds) const {
#pragma unroll
    for (int i = 0; i < NVEC; ++i) {
      const int idx = threadIdx.x + i * GTHREADS;
      if (KMAJOR) {
        constexpr int VPR = GBK / VEC;
        *(i32x4_t*)(lds + (idx / VPR) * PITCH + (idx % VPR) * 16) = v[i];
      } else {
        constexpr int VPR = 128 / VEC;
        const int krow = idx / VPR;
        const int mn = (idx % VPR) * VEC;
#pragma unroll
        for (int j = 0; j < 8; ++j)
          *(uint16_t*)(lds + (mn + j) * PITCH + krow * 2) = (uint16_t)((uint32_t)v[i][j >> 1] >> ((j & 1) * 16));
      }
    }
  }
};

template <int DT> TGG_DEV typename Frag<DT>::type read_frag(const char* lds, int row, int koff) {
  constexpr int ES = ElemSize<DT>::v;
  constexpr int PITCH = GBK * ES + 16;
  return *(const typename Frag<DT>::type*)(lds + row * PITCH + koff * ES);
}

enum : int { EPI_PLAIN = 0, EPI_CHANNEL = 1, EPI_BLOCK = 2 };

struct GenericSmem {
  SchedTable sched;
  __attribute__((aligned(16))) char a[2][128 * (GBK * 2 + 16)];
  __attribute__((aligned(16))) char b[2][128 * (GBK * 2 + 16)];
};

template <int TA, int TB, bool A_KMAJOR, bool B_KMAJOR, int EPI, int OUT>
__global__ __launch_bounds__(GTHREADS) void gemm_generic_kernel(const GemmParams p) {
  __shared__ GenericSmem sm;
  constexpr int ESA = ElemSize<TA>::v, ESB = ElemSize<TB>::v;
  sched_init<GBM>(p, sm.sched);
  if (!sched_kg_gate_open(p, sm.sched)) return;
  const int64_t num_tiles = sched_num_tiles<GBM, GBN>(p, sm.sched);
  const bool kmode = (p.mode == MODE_KG || p.mode == MODE_KG_COUNT);

  const int lane = lane_id();
  const int wave = threadIdx.x >> 6;
  const int wm = (wave >> 1) * 64, wn = (wave & 1) * 64;
  const int l32 = lane & 31, lh = lane >> 5;

  const TileWalk walk = sched_walk(num_tiles, !kmode);
  for (int64_t tile_id = walk.first; tile_id < walk.end; tile_id += walk.stride) {
    const Tile t = sched_tile<GBM, GBN>(p, sm.sched, tile_id);
    // operand bases for this tile at k = 0 (generic_addr.hpp)
    const GenericTileIo io = generic_tile_io<A_KMAJOR>(p, t);
    const char* a_base = (const char*)p.A + io.a_elem * ESA;
    const int a_lim = io.a_lim;
    const char* b_base = (const char*)p.B + io.b_elem * ESB;
    const int b_lim = io.b_lim;

    f32x16_t acc[2][2];
    f32x16_t part[2][2];
#pragma unroll
    for (int i = 0; i < 2; ++i)
#pragma unroll
      for (int j = 0; j < 2; ++j)
#pragma unroll
        for (int e = 0; e < 16; ++e) { acc[i][j][e] = 0.f; part[i][j][e] = 0.f; }

    Stager<TA, A_KMAJOR> sa_;
    Stager<TB, B_KMAJOR> sb_;
    const int64_t klen = t.k1 - t.k0;
    const int kt_n = (int)((klen + GBK - 1) / GBK);
    if (kt_n > 0) {
      sa_.load(a_base, p.a_sm, p.a_sk, a_lim, t.k0, t.k1);
      sb_.load(b_base, p.b_sn, p.b_sk, b_lim, t.k0, t.k1);
      sa_.store(sm.a[0]);
      sb_.store(sm.b[0]);
    }
    __syncthreads();
    for (int kt = 0; kt < kt_n; ++kt) {
      const int cur = kt & 1;
      if (kt + 1 < kt_n) {
        sa_.load(a_base, p.a_sm, p.a_sk, a_lim, t.k0 + (int64_t)(kt + 1) * GBK, t.k1);
        sb_.load(b_base, p.b_sn, p.b_sk, b_lim, t.k0 + (int64_t)(kt + 1) * GBK, t.k1);
      }
#pragma unroll
      for (int ks = 0; ks < GBK / 16; ++ks) {
        typename Frag<TA>::type fa[2];
        typename Frag<TB>::type fb[2];
#pragma unroll
        for (int i = 0; i < 2; ++i) fa[i] = read_frag<TA>(sm.a[cur], wm + i * 32 + l32, ks * 16 + lh * 8);
#pragma unroll
        for (int j = 0; j < 2; ++j) fb[j] = read_frag<TB>(sm.b[cur], wn + j * 32 + l32, ks * 16 + lh * 8);
#pragma unroll
        for (int i = 0; i < 2; ++i)
#pragma unroll
          for (int j = 0; j < 2; ++j) {
            if (EPI == EPI_BLOCK) part[i][j] = Mma<TB, TA>::run(fb[j], fa[i], part[i][j]);
            else acc[i][j] = Mma<TB, TA>::run(fb[j], fa[i], acc[i][j]);
          }
      }
      if (EPI == EPI_BLOCK) {
        // every 128 of K (or at the end) fold the partial sums in with their block scales
        const int64_t kpos = (int64_t)(kt + 1) * GBK;
        if ((kpos & 127) == 0 || kt + 1 == kt_n) {
          const int kb = generic_scale_block_of_slab(kt);
          const float sbv = p.sb[generic_sb_index(p, t, kb)];
#pragma unroll
          for (int i = 0; i < 2; ++i) {
            const int m = wm + i * 32 + l32;
            const float s = (m < t.rows) ? p.sa[generic_sa_index(p, t, m, kb)] * sbv : 0.f;
#pragma unroll
            for (int j = 0; j < 2; ++j)
#pragma unroll
              for (int e = 0; e < 16; ++e) {
                acc[i][j][e] += part[i][j][e] * s;
                part[i][j][e] = 0.f;
              }
          }
        }
      }
      if (kt + 1 < kt_n) {
        sa_.store(sm.a[cur ^ 1]);
        sb_.store(sm.b[cur ^ 1]);
      }
      __syncthreads();
    }

    // epilogue: lane owns row m, columns n = wn + j*32 + 8q + 4*lh + (0..3)
    char* c_base = (char*)p.C + io.c_elem * 2;
    const bool vec_ok = (p.N & 3) == 0;
#pragma unroll
    for (int i = 0; i < 2; ++i) {
      const int m = wm + i * 32 + l32;
      if (m >= t.rows) continue;
      float rs = 1.f;
      if (EPI == EPI_CHANNEL) rs = p.scale_m[generic_scale_m_index(p, t, m)];
#pragma unroll
      for (int j = 0; j < 2; ++j)
#pragma unroll
        for (int q = 0; q < 4; ++q) {
          const int n = t.n0 + wn + j * 32 + q * 8 + lh * 4;
          if (n >= p.N) continue;
          float v[4];
#pragma unroll
          for (int e = 0; e < 4; ++e) {
            v[e] = acc[i][j][q * 4 + e];
            if (EPI == EPI_CHANNEL) v[e] = (n + e < p.N) ? v[e] * rs * p.scale_n[generic_scale_n_index(p, t, n + e)] : 0.f;
          }
          char* dst = c_base + ((int64_t)m * p.N + n) * 2;
          if (vec_ok) {
            *(uint2*)dst = pack4<OUT>(v[0], v[1], v[2], v[3]);
          } else {
#pragma unroll
            for (int e = 0; e < 4; ++e)
              if (n + e < p.N) *(uint16_t*)(dst + e * 2) = Out16<OUT>::cvt(v[e]);
          }
        }
    }
  }
}

template <int TA, int TB, bool AK, bool BK_, int EPI, int OUT>
int launch_one(const GemmParams& p, hipStream_t stream) {
  int grid = num_cus();
  if (p.grid_limit > 0 && p.grid_limit < grid) grid = p.grid_limit;
  hipLaunchKernelGGL((gemm_generic_kernel<TA, TB, AK, BK_, EPI, OUT>), dim3(grid), dim3(GTHREADS), 0, stream, p);
  return check_launch("gemm_generic");
}

template <int TA, int TB, int EPI>
int launch_fp8_out(const GemmParams& p, int out_dt, hipStream_t s) {
  if (out_dt == DT_BF16) return launch_one<TA, TB, true, true, EPI, DT_BF16>(p, s);
  if (out_dt == DT_F16) return launch_one<TA, TB, true, true, EPI, DT_F16>(p, s);
  return set_error("unsupported output dtype code %d", out_dt);
}

}  // namespace

// layout: 0 = NT (A and B K-contiguous), 1 = NN (B is [K, N]), 2 = TN (A is [K, M], B is [K, N])
int launch_generic_16bit(const GemmParams& p, int dt, int layout, hipStream_t s) {
  if (dt == DT_BF16) {
    if (layout == 0) return launch_one<DT_BF16, DT_BF16, true, true, EPI_PLAIN, DT_BF16>(p, s);
    if (layout == 1) return launch_one<DT_BF16, DT_BF16, true, false, EPI_PLAIN, DT_BF16>(p, s);
    if (layout == 2) return launch_one<DT_BF16, DT_BF16, false, false, EPI_PLAIN, DT_BF16>(p, s);
  } else if (dt == DT_F16) {
    if (layout == 0) return launch_one<DT_F16, DT_F16, true, true, EPI_PLAIN, DT_F16>(p, s);
    if (layout == 1) return launch_one<DT_F16, DT_F16, true, false, EPI_PLAIN, DT_F16>(p, s);
    if (layout == 2) return launch_one<DT_F16, DT_F16, false, false, EPI_PLAIN, DT_F16>(p, s);
  }
  return set_error("unsupported dtype/layout (%d, %d)", dt, layout);
}

int launch_generic_fp8_channel(const GemmParams& p, int ta, int tb, int out_dt, hipStream_t s) {
  if (ta == DT_E4M3 && tb == DT_E4M3) return launch_fp8_out<DT_E4M3, DT_E4M3, EPI_CHANNEL>(p, out_dt, s);
  if (ta == DT_E4M3 && tb == DT_E5M2) return launch_fp8_out<DT_E4M3, DT_E5M2, EPI_CHANNEL>(p, out_dt, s);
  if (ta == DT_E5M2 && tb == DT_E4M3) return launch_fp8_out<DT_E5M2, DT_E4M3, EPI_CHANNEL>(p, out_dt, s);
  if (ta == DT_E5M2 && tb == DT_E5M2) return launch_fp8_out<DT_E5M2, DT_E5M2, EPI_CHANNEL>(p, out_dt, s);
  return set_error("unsupported fp8 formats (%d, %d)", ta, tb);
}

int launch_generic_fp8_block(const GemmParams& p, hipStream_t s) {
  return launch_one<DT_E4M3, DT_E4M3, true, true, EPI_BLOCK, DT_BF16>(p, s);
}

}  // namespace tgg
