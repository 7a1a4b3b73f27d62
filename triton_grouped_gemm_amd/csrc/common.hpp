// Shared device-side vocabulary for the gfx950 grouped-GEMM kernels.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace tgg {

// Element type codes used across the C ABI.
enum : int { DT_BF16 = 0, DT_F16 = 1, DT_E4M3 = 2, DT_E5M2 = 3 };

// How the groups of a launch are laid out along the row (or K) dimension.
enum : int {
  MODE_MG = 0,      // M-grouped: group g owns rows [prefix(sizes)[g], +sizes[g])
  MODE_MG_PAD = 1,  // M-grouped, rows physically padded: starts are prefix(round_up(sizes, align))
  MODE_MASKED = 2,  // group g owns rows [g*m_stride, g*m_stride + sizes[g])
  MODE_KG = 3,      // K-grouped: group g reduces over k in [k_start[g], k_end[g])
  MODE_KG_COUNT = 4 // K-grouped: k segments are prefix(sizes)
};

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8_t;
typedef __attribute__((ext_vector_type(4))) __bf16 bf16x4_t;
typedef __attribute__((ext_vector_type(8))) _Float16 f16x8_t;
typedef __attribute__((ext_vector_type(4))) _Float16 f16x4_t;
typedef __attribute__((ext_vector_type(16))) float f32x16_t;
typedef __attribute__((ext_vector_type(4))) float f32x4_t;
typedef __attribute__((ext_vector_type(8))) int i32x8_t;
typedef __attribute__((ext_vector_type(4))) int i32x4_t;
typedef __attribute__((ext_vector_type(2))) int i32x2_t;
typedef __attribute__((ext_vector_type(4))) short i16x4_t;
typedef __attribute__((ext_vector_type(8))) short i16x8_t;

#define TGG_DEV __device__ __forceinline__

TGG_DEV int lane_id() { return threadIdx.x & 63; }

// fp32 -> 16-bit output element, round to nearest even.
template <int DT> struct Out16;
template <> struct Out16<DT_BF16> {
  static TGG_DEV uint16_t cvt(float x) {
    __bf16 b = (__bf16)x;
    return __builtin_bit_cast(uint16_t, b);
  }
};
template <> struct Out16<DT_F16> {
  static TGG_DEV uint16_t cvt(float x) {
    _Float16 h = (_Float16)x;
    return __builtin_bit_cast(uint16_t, h);
  }
};

// Two fp32 -> one dword of two 16-bit outputs (first value in the low half), round to nearest even.  Written
// as a vector conversion so that it becomes one packed convert instead of two converts, a shift and an or.
typedef __attribute__((ext_vector_type(2))) float f32x2_t;
typedef __attribute__((ext_vector_type(2))) __bf16 bf16x2_t;
typedef __attribute__((ext_vector_type(2))) _Float16 f16x2_t;
template <int DT> TGG_DEV uint32_t pack2(float a, float b) {
  const f32x2_t v = {a, b};
  if (DT == DT_BF16) return __builtin_bit_cast(uint32_t, __builtin_convertvector(v, bf16x2_t));
  return __builtin_bit_cast(uint32_t, __builtin_convertvector(v, f16x2_t));
}
template <int DT> TGG_DEV uint2 pack4(float a, float b, float c, float d) {
  uint2 r;
  r.x = pack2<DT>(a, b);
  r.y = pack2<DT>(c, d);
  return r;
}

// Everything a grouped GEMM launch needs.  Strides are in elements.
// C[tile](m, n) = sum_k Aop(m, k) * Bop(g, n, k), with
//   Aop(m, k) = A[m * a_sm + k * a_sk],  Bop(g, n, k) = B[g * b_sg + n * b_sn + k * b_sk].
struct GemmParams {
  const void* A;
  const void* B;
  void* C;
  const void* sizes;      // per-group row counts / masked_m / token counts (int32 or int64)
  const int32_t* k_start; // MODE_KG only
  const int32_t* k_end;   // MODE_KG only
  const int32_t* row_start; // MODE_MG_PAD, optional: group g's rows start at row_start[g] (groups placed in any order)
  const float* scale_m;   // per-row scale (channel modes) or nullptr
  const float* scale_n;   // per-(group, column) scale, indexed g*N + n, or nullptr
  const float* sa;        // block-scaled activation scales: element (row, kb) at row * sa_rs + kb * sa_ks
  const float* sb;        // block-scaled: [G, ceil(N/128), ceil(K/128)] weight scales
  int64_t m_total;        // rows of A/C that may be touched (M-grouped), Mdim for K-grouped
  int64_t m_stride;       // MODE_MASKED: rows between consecutive groups
  int64_t k_total;        // K-grouped: length of the shared reduction axis (segments are clipped to it)
  int64_t a_sm, a_sk;
  int64_t b_sg, b_sn, b_sk;
  int64_t c_sg;           // K-grouped: elements between consecutive groups' outputs
  int64_t scale_m_sg;     // K-grouped channel mode: scale_m stride between groups
  int64_t sa_rs, sa_ks;   // strides (in floats) of the block-scaled activation scales
  int sizes_i64;
  int G;
  int mode;
  int align;              // MODE_MG_PAD alignment
  int N;
  int K;                  // reduction length (M-grouped); unused for K-grouped
  int grid_limit;         // >0 caps the persistent grid
  int tile_split;         // tuned kernels: 1 = per-XCD contiguous tile ranges (see sched_walk)
  int n_chunk;            // column tiles per chunk of the tile order, 0 = automatic (see sched_tile)
  int32_t* queue;         // K-grouped tuned kernels: tile-id counter in device memory (zero at launch), or null = static walk
  int store_nt;           // tuned kernels: 1 = non-temporal output stores
  // FP8 K-grouped by token counts: the tuned kernel copies 16-byte chunks, so it needs every count (hence every
  // segment start) to be a multiple of 16; the shape-agnostic kernel takes anything.  Only the device knows the
  // counts, so both kernels are launched and each looks at the counts first: 1 = run only if all counts are
  // multiples of 16 (tuned), 2 = run only if one is not (shape-agnostic), 0 = always run.
  int kg_gate;
  // 16-bit launches that the four-wave kernel could take but whose groups may be small (masked; M-grouped with fewer
  // than 512 rows per group on average): it pays only where the eight-wave kernels would choose their 256x256 tiles,
  // which depends on the sizes, and only the device knows them.  Both kernels are
  // launched and each evaluates the same predicate on its group table first (sched_wide_tiles_chosen):
  // 1 = run only if it holds (four-wave), 2 = run only if it does not (eight-wave), 0 = always run.
  int wide_gate;
  // fused 1x128 quantisation of the output (tuned 16-bit M-grouped kernels): C then holds fp8 codes [rows, N] and
  // the scale of (row, 128-column block) goes to q_scales[row * q_rs + block * q_bs]
  float* q_scales;
  int64_t q_rs, q_bs;
  int q_fmt;              // DT_E4M3 / DT_E5M2; 0 = no quantisation
};

}  // namespace tgg
