// FP8 quantizers for gfx950: streaming, HBM-bound kernels.
//
//  * trans_quant128: per 128x128 block of a grouped bf16 matrix, quantise with one
//    fp32 scale, transpose, and place at the group's 128-padded column offset.
//  * token_cast128:  1x128 groups along K (activation recipe).
//  * block_cast128:  128x128 blocks, no transpose (weight recipe).
//
// Bit-exactness contract: scale and quotient/product are single IEEE fp32
// operations on the exact fp32 value of the bf16 input; fp32 -> fp8 is
// round-to-nearest-even after an explicit clamp (hardware v_cvt_pk_{fp8,bf8}_f32).
#include "common.hpp"
#include "sched.hpp"
#include "launch.hpp"

namespace tgg {

namespace {

TGG_DEV float bf16_bits_to_f32(uint32_t h) { return __builtin_bit_cast(float, h << 16); }

template <int FMT> TGG_DEV uint32_t cvt_pk(float a, float b, uint32_t old, bool hi) {
  if (FMT == DT_E4M3) return hi ? __builtin_amdgcn_cvt_pk_fp8_f32(a, b, old, true) : __builtin_amdgcn_cvt_pk_fp8_f32(a, b, old, false);
  return hi ? __builtin_amdgcn_cvt_pk_bf8_f32(a, b, old, true) : __builtin_amdgcn_cvt_pk_bf8_f32(a, b, old, false);
}

template <int FMT> TGG_DEV uint32_t cvt4(float a, float b, float c, float d) {
  uint32_t w = cvt_pk<FMT>(a, b, 0u, false);
  return cvt_pk<FMT>(c, d, w, true);
}

template <int FMT> struct FmtMax;
template <> struct FmtMax<DT_E4M3> { static constexpr float v = 448.0f; };
template <> struct FmtMax<DT_E5M2> { static constexpr float v = 57344.0f; };

TGG_DEV float clampf(float x, float lo, float hi) { return fminf(fmaxf(x, lo), hi); }

TGG_DEV float wave_max(float v) {
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) v = fmaxf(v, __shfl_xor(v, off, 64));
  return v;
}

// abs-max of 8 bf16 packed in a 16-byte vector
TGG_DEV float amax8(i32x4_t v) {
  float m = 0.f;
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const uint32_t w = (uint32_t)v[i];
    m = fmaxf(m, fabsf(bf16_bits_to_f32(w & 0xffffu)));
    m = fmaxf(m, fabsf(bf16_bits_to_f32(w >> 16)));
  }
  return m;
}

template <int MAXG> struct TransSmem {
  SchedTableT<MAXG> sched;
  __attribute__((aligned(16))) uint8_t t[128 * 128];
  float wmax[4];
};

// One 128x128 block per iteration, 256 threads.
// Read: thread (rr = tid/16, cv = tid%16) owns rows rr*8 .. rr*8+7, columns cv*8 .. cv*8+7.
// LDS holds the transposed codes: byte (c, r) at c*128 + ((r/16) ^ ((c/8)%8))*16 + r%16.
// MAXG sizes the group table in LDS: the small one lets twice as many workgroups share a CU.
template <int FMT, int MAXG>
__global__ __launch_bounds__(256) void trans_quant128_kernel(const uint16_t* __restrict__ x, uint8_t* __restrict__ codes,
                                                            float* __restrict__ scales, GemmParams p, int64_t m_expand) {
  __shared__ TransSmem<MAXG> sm;
  sched_init<128>(p, sm.sched);
  const int N = p.N;
  const int tiles_n = N >> 7;
  const int m_tiles_real = sm.sched.tile0[p.G];
  const int m_tiles_all = (int)(m_expand >> 7);
  const int64_t total = (int64_t)m_tiles_all * tiles_n;
  const int tid = threadIdx.x;
  const int rr = tid >> 4, cv = tid & 15;
  constexpr float fmax_ = FmtMax<FMT>::v;

  for (int64_t tile = blockIdx.x; tile < total; tile += gridDim.x) {
    const int pm = (int)(tile / tiles_n);
    const int bn = (int)(tile % tiles_n);
    uint8_t* out_base = codes + ((int64_t)bn * 128) * m_expand + (int64_t)pm * 128;
    if (pm >= m_tiles_real) {  // tail beyond the padded groups: zero codes, zero scale
      const i32x4_t z = {0, 0, 0, 0};
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const int c = (tid >> 3) + 32 * i, u = tid & 7;
        *(i32x4_t*)(out_base + (int64_t)c * m_expand + u * 16) = z;
      }
      if (tid == 0) scales[(int64_t)bn * m_tiles_all + pm] = 0.f;
      continue;
    }
    // The row tile is looked up directly in the group table: the GEMM tile-id order (column chunks) plays no part here.
    const RowTile t = sched_row_tile<128>(sm.sched, p.G, pm);
    i32x4_t v[8];
    float amax = 0.f;
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      const int r = rr * 8 + i;
      i32x4_t val = {0, 0, 0, 0};
      if (r < t.rows) val = *(const i32x4_t*)(x + (t.row0 + r) * (int64_t)N + bn * 128 + cv * 8);
      v[i] = val;
      amax = fmaxf(amax, amax8(val));
    }
    amax = wave_max(amax);
    __syncthreads();  // previous iteration's LDS reads are done
    if ((tid & 63) == 0) sm.wmax[tid >> 6] = amax;
    __syncthreads();
    amax = fmaxf(fmaxf(sm.wmax[0], sm.wmax[1]), fmaxf(sm.wmax[2], sm.wmax[3]));
    const float scale = clampf(amax / fmax_, 1e-12f, 3e38f);
    // column j of this thread's 8x8 patch -> 8 consecutive r bytes
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      float q[8];
#pragma unroll
      for (int i = 0; i < 8; ++i) {
        const uint32_t w = (uint32_t)v[i][j >> 1];
        const float f = bf16_bits_to_f32((j & 1) ? (w >> 16) : (w & 0xffffu));
        q[i] = clampf(f / scale, -fmax_, fmax_);
      }
      uint2 pk;
      pk.x = cvt4<FMT>(q[0], q[1], q[2], q[3]);
      pk.y = cvt4<FMT>(q[4], q[5], q[6], q[7]);
      const int c = cv * 8 + j;
      const int slot = (rr >> 1) ^ (cv & 7);
      *(uint2*)(sm.t + c * 128 + slot * 16 + (rr & 1) * 8) = pk;
    }
    __syncthreads();
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int c = (tid >> 3) + 32 * i, u = tid & 7;
      const i32x4_t o = *(const i32x4_t*)(sm.t + c * 128 + ((u ^ ((c >> 3) & 7)) * 16));
      *(i32x4_t*)(out_base + (int64_t)c * m_expand + u * 16) = o;
    }
    if (tid == 0) scales[(int64_t)bn * m_tiles_all + pm] = scale;
  }
}

// 16 lanes per 1x128 group; each lane 8 elements.  A workgroup's 16 lane groups take 16 neighbouring groups
// along the axis the scales are contiguous in, so that the 16 scale stores of a step fill one 64-byte segment:
//   scales [rows, kblocks]  (mn_major = 0): 16 consecutive K blocks of one row
//   scales [kblocks, rows]  (mn_major = 1): the same K block of 16 consecutive rows
// Two steps are in flight per thread.
template <int FMT>
__global__ __launch_bounds__(256) void token_cast128_kernel(const uint16_t* __restrict__ x, uint8_t* __restrict__ codes,
                                                           float* __restrict__ scales, int64_t rows, int kblocks, int mn_major) {
  constexpr float fmax_ = FmtMax<FMT>::v;
  const int64_t groups = rows * kblocks;
  const int sub = threadIdx.x & 15, grp = threadIdx.x >> 4;
  // step s of the launch covers 16 groups; steps are numbered so that consecutive steps touch neighbouring memory
  const int64_t row_blocks = (rows + 15) / 16;
  const int64_t steps = mn_major ? row_blocks * kblocks : (groups + 15) / 16;
  auto group_of = [&](int64_t step, int64_t& g, int64_t& sidx) -> bool {
    if (mn_major) {
      const int64_t rb = step / kblocks;
      const int kb = (int)(step - rb * kblocks);
      const int64_t r = rb * 16 + grp;
      g = r * kblocks + kb;
      sidx = (int64_t)kb * rows + r;
      return r < rows;
    }
    g = step * 16 + grp;
    sidx = g;
    return g < groups;
  };
  auto quantise = [&](const i32x4_t v, int64_t g, int64_t sidx, bool ok) {
    float amax = amax8(v);
#pragma unroll
    for (int off = 8; off > 0; off >>= 1) amax = fmaxf(amax, __shfl_xor(amax, off, 64));
    amax = fmaxf(amax, 1e-4f);
    const float mult = (1.0f / amax) * fmax_;  // torch evaluates `448.0 / amax` as reciprocal * 448
    float f[8];
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const uint32_t w = (uint32_t)v[i];
      f[2 * i] = bf16_bits_to_f32(w & 0xffffu) * mult;
      f[2 * i + 1] = bf16_bits_to_f32(w >> 16) * mult;
    }
    uint2 pk;
    pk.x = cvt4<FMT>(f[0], f[1], f[2], f[3]);
    pk.y = cvt4<FMT>(f[4], f[5], f[6], f[7]);
    if (ok) {
      *(uint2*)(codes + g * 128 + sub * 8) = pk;
      if (sub == 0) scales[sidx] = amax / fmax_;
    }
  };
  const i32x4_t zero = {0, 0, 0, 0};
  for (int64_t s0 = (int64_t)blockIdx.x * 2; s0 < steps; s0 += (int64_t)gridDim.x * 2) {
    int64_t g0, g1, i0, i1;
    const bool ok0 = group_of(s0, g0, i0);
    const bool ok1 = s0 + 1 < steps && group_of(s0 + 1, g1, i1);
    const i32x4_t v0 = ok0 ? *(const i32x4_t*)(x + g0 * 128 + sub * 8) : zero;
    const i32x4_t v1 = ok1 ? *(const i32x4_t*)(x + g1 * 128 + sub * 8) : zero;
    quantise(v0, g0, i0, ok0);
    quantise(v1, g1, i1, ok1);
  }
}

// 128x128 blocks of a [batch, R, C] tensor (blocks never straddle batch entries).
template <int FMT>
__global__ __launch_bounds__(256) void block_cast128_kernel(const uint16_t* __restrict__ x, uint8_t* __restrict__ codes,
                                                           float* __restrict__ scales, int batch, int R, int C) {
  __shared__ float wmax[4];
  constexpr float fmax_ = FmtMax<FMT>::v;
  const int tr = (R + 127) >> 7, tc = (C + 127) >> 7;
  const int64_t total = (int64_t)batch * tr * tc;
  const int tid = threadIdx.x;
  const int rr = tid >> 4, cv = tid & 15;
  const bool vec_ok = (C & 7) == 0;
  for (int64_t tile = blockIdx.x; tile < total; tile += gridDim.x) {
    const int b = (int)(tile / (tr * tc));
    const int rem = (int)(tile % (tr * tc));
    const int r0 = (rem / tc) * 128, c0 = (rem % tc) * 128;
    const uint16_t* src = x + (int64_t)b * R * C;
    uint8_t* dst = codes + (int64_t)b * R * C;
    i32x4_t v[8];
    float amax = 0.f;
    const int c = c0 + cv * 8;
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      const int r = r0 + rr + 16 * i;
      i32x4_t val = {0, 0, 0, 0};
      if (r < R && c < C) {
        const uint16_t* s = src + (int64_t)r * C + c;
        if (vec_ok) {
          val = *(const i32x4_t*)s;
        } else {
#pragma unroll
          for (int e = 0; e < 8; ++e)
            if (c + e < C) val[e >> 1] |= (int)((uint32_t)s[e] << ((e & 1) * 16));
        }
      }
      v[i] = val;
      amax = fmaxf(amax, amax8(val));
    }
    amax = wave_max(amax);
    __syncthreads();
    if ((tid & 63) == 0) wmax[tid >> 6] = amax;
    __syncthreads();
    amax = fmaxf(fmaxf(fmaxf(wmax[0], wmax[1]), fmaxf(wmax[2], wmax[3])), 1e-4f);
    const float mult = (1.0f / amax) * fmax_;  // torch evaluates `448.0 / amax` as reciprocal * 448
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      const int r = r0 + rr + 16 * i;
      if (r >= R || c >= C) continue;
      float f[8];
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        const uint32_t w = (uint32_t)v[i][e];
        f[2 * e] = bf16_bits_to_f32(w & 0xffffu) * mult;
        f[2 * e + 1] = bf16_bits_to_f32(w >> 16) * mult;
      }
      uint2 pk;
      pk.x = cvt4<FMT>(f[0], f[1], f[2], f[3]);
      pk.y = cvt4<FMT>(f[4], f[5], f[6], f[7]);
      uint8_t* d = dst + (int64_t)r * C + c;
      if (vec_ok) {
        *(uint2*)d = pk;
      } else {
#pragma unroll
        for (int e = 0; e < 8; ++e)
          if (c + e < C) d[e] = (uint8_t)(((e < 4) ? pk.x : pk.y) >> ((e & 3) * 8));
      }
    }
    if (tid == 0) scales[tile] = amax / fmax_;
  }
}

template <int FMT>
__global__ void cvt_fp8_kernel(const float* __restrict__ in, uint8_t* __restrict__ out, int64_t n) {
  const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i < n) out[i] = (uint8_t)cvt_pk<FMT>(in[i], 0.f, 0u, false);
}

}  // namespace

int launch_trans_quant128(const void* x, void* codes, float* scales, const GemmParams& p, int64_t m_expand, int fmt,
                          hipStream_t s) {
  const int64_t tiles = (m_expand >> 7) * (int64_t)(p.N >> 7);
  int64_t grid = (int64_t)num_cus() * 8;
  if (grid > tiles) grid = tiles;
  if (grid < 1) grid = 1;
  const dim3 g((unsigned)grid), b(256);
  const uint16_t* xi = (const uint16_t*)x;
  uint8_t* co = (uint8_t*)codes;
  const bool small = p.G <= 256;
  if (fmt == DT_E4M3) {
    if (small) hipLaunchKernelGGL((trans_quant128_kernel<DT_E4M3, 256>), g, b, 0, s, xi, co, scales, p, m_expand);
    else hipLaunchKernelGGL((trans_quant128_kernel<DT_E4M3, kMaxGroups>), g, b, 0, s, xi, co, scales, p, m_expand);
  } else if (fmt == DT_E5M2) {
    if (small) hipLaunchKernelGGL((trans_quant128_kernel<DT_E5M2, 256>), g, b, 0, s, xi, co, scales, p, m_expand);
    else hipLaunchKernelGGL((trans_quant128_kernel<DT_E5M2, kMaxGroups>), g, b, 0, s, xi, co, scales, p, m_expand);
  } else {
    return set_error("unsupported fp8 format code %d", fmt);
  }
  return check_launch("trans_quant128");
}

int launch_token_cast128(const void* x, void* codes, float* scales, int64_t rows, int kblocks, int mn_major, int fmt,
                         hipStream_t s) {
  const int64_t groups = rows * kblocks;
  if (groups == 0) return 0;
  int64_t grid = ((mn_major ? ((rows + 15) / 16) * kblocks : (groups + 15) / 16) + 1) / 2;
  const int64_t cap = (int64_t)num_cus() * 32;
  if (grid > cap) grid = cap;
  if (fmt == DT_E4M3)
    hipLaunchKernelGGL(token_cast128_kernel<DT_E4M3>, dim3((unsigned)grid), dim3(256), 0, s, (const uint16_t*)x,
                       (uint8_t*)codes, scales, rows, kblocks, mn_major);
  else if (fmt == DT_E5M2)
    hipLaunchKernelGGL(token_cast128_kernel<DT_E5M2>, dim3((unsigned)grid), dim3(256), 0, s, (const uint16_t*)x,
                       (uint8_t*)codes, scales, rows, kblocks, mn_major);
  else
    return set_error("unsupported fp8 format code %d", fmt);
  return check_launch("token_cast128");
}

int launch_block_cast128(const void* x, void* codes, float* scales, int batch, int R, int C, int fmt, hipStream_t s) {
  const int64_t tiles = (int64_t)batch * ((R + 127) / 128) * ((C + 127) / 128);
  if (tiles == 0) return 0;
  int64_t grid = (int64_t)num_cus() * 8;
  if (grid > tiles) grid = tiles;
  if (fmt == DT_E4M3)
    hipLaunchKernelGGL(block_cast128_kernel<DT_E4M3>, dim3((unsigned)grid), dim3(256), 0, s, (const uint16_t*)x,
                       (uint8_t*)codes, scales, batch, R, C);
  else if (fmt == DT_E5M2)
    hipLaunchKernelGGL(block_cast128_kernel<DT_E5M2>, dim3((unsigned)grid), dim3(256), 0, s, (const uint16_t*)x,
                       (uint8_t*)codes, scales, batch, R, C);
  else
    return set_error("unsupported fp8 format code %d", fmt);
  return check_launch("block_cast128");
}

int launch_cvt_fp8(const float* in, void* out, int64_t n, int fmt, hipStream_t s) {
  if (n == 0) return 0;
  const unsigned grid = (unsigned)((n + 255) / 256);
  if (fmt == DT_E4M3) hipLaunchKernelGGL(cvt_fp8_kernel<DT_E4M3>, dim3(grid), dim3(256), 0, s, in, (uint8_t*)out, n);
  else if (fmt == DT_E5M2) hipLaunchKernelGGL(cvt_fp8_kernel<DT_E5M2>, dim3(grid), dim3(256), 0, s, in, (uint8_t*)out, n);
  else return set_error("unsupported fp8 format code %d", fmt);
  return check_launch("cvt_fp8");
}

}  // namespace tgg
