// extern "C" surface of libtgg_amd.so: argument validation, GemmParams assembly, dispatch.
#include <stdarg.h>
#include <stdio.h>
#include <string.h>

#include <atomic>
#include <vector>

#include "../../include/tgg_amd.h"
#include "common.hpp"
#include "generic_addr.hpp"
#include "launch.hpp"
#include "sched.hpp"

namespace tgg {

static thread_local char g_err[512] = "";
// Process-wide options (tgg_set_option): test and tuning hooks.  Atomic so that a thread that flips one while another
// thread launches is a race on which value that launch sees, not undefined behaviour; a launch reads each option once.
static std::atomic<int> g_force_generic{0};
static std::atomic<int> g_tile_split{1};
static std::atomic<int> g_store_nt{1};
static std::atomic<int> g_n_chunk{0};
static std::atomic<int> g_kg_second_launch{1};
static std::atomic<int> g_four_wave{1};  // 0 = eight-wave kernels only, 1 = four-wave kernel on large M-grouped NT launches (default), 2 = on every launch it can take

int set_error(const char* fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_err, sizeof(g_err), fmt, ap);
  va_end(ap);
  return 1;
}

int check_launch(const char* what) {
  hipError_t e = hipGetLastError();
  if (e == hipSuccess) return 0;
  snprintf(g_err, sizeof(g_err), "%s: %s", what, hipGetErrorString(e));
  return 2;
}

int num_cus() {
  static int cached[64] = {0};
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) return 256;
  if (cached[dev] == 0) {
    int n = 0;
    if (hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || n <= 0) n = 256;
    cached[dev] = n;
  }
  return cached[dev];
}

int launch_trans_quant128(const void*, void*, float*, const GemmParams&, int64_t, int, hipStream_t);
int launch_token_cast128(const void*, void*, float*, int64_t, int, int, int, hipStream_t);
int launch_block_cast128(const void*, void*, float*, int, int, int, int, hipStream_t);
int launch_cvt_fp8(const float*, void*, int64_t, int, hipStream_t);
bool fast_supported(const GemmParams& p, int dt, int layout);
int launch_fast_16bit(const GemmParams& p, int dt, int layout, hipStream_t s);
bool w4_supported(const GemmParams& p, int dt, int layout, bool any_size);
bool w4_decided_on_device(const GemmParams& p);
int launch_w4_16bit(const GemmParams& p, int dt, int layout, hipStream_t s);
bool fast_quant_supported(const GemmParams& p, int dt, int layout);
int launch_fast_16bit_quant(const GemmParams& p, int dt, int layout, hipStream_t s);
void set_fast_variant(int v);
void set_fp8_variant(int v);

static bool aligned16(const void* p) { return (((uintptr_t)p) & 15) == 0; }

// max_groups: TGG_MAX_GROUPS for the two plain 16-bit entry points (M-grouped, K-grouped), whose shape-agnostic
// kernel is exercised on the GPU above 512 groups; TGG_MAX_GROUPS_OTHER for every other GEMM entry point.
static int check_common(const void* A, const void* B, const void* C, const void* sizes, int G, int N,
                        int max_groups = TGG_MAX_GROUPS_OTHER) {
  if (!A || !B || !C) return set_error("null operand pointer");
  if (!sizes) return set_error("null group-size pointer");
  if (G < 1 || G > max_groups) return set_error("G=%d outside [1, %d]", G, max_groups);
  if (N < 1) return set_error("N=%d must be positive", N);
  if (!aligned16(A) || !aligned16(B) || !aligned16(C)) return set_error("operand pointers must be 16-byte aligned");
  return 0;
}

static GemmParams zero_params() {
  GemmParams p;
  memset(&p, 0, sizeof(p));
  p.tile_split = g_tile_split;
  p.store_nt = g_store_nt;
  p.n_chunk = g_n_chunk;
  return p;
}


// GemmParams of each GEMM entry point, assembled in one place: the entry points launch with them and
// tgg_debug_generic_extents walks the same parameter blocks on the host.
static GemmParams params_m_grouped(const void* A, const void* B, void* C, const void* sizes, int sizes_i64, int G,
                                   int64_t M, int N, int K, int trans_b, int num_cu) {
  GemmParams p = zero_params();
  p.A = A; p.B = B; p.C = C; p.sizes = sizes; p.sizes_i64 = sizes_i64; p.G = G;
  p.mode = MODE_MG; p.m_total = M; p.N = N; p.K = K;
  p.a_sm = K; p.a_sk = 1;
  p.b_sg = (int64_t)N * K;
  if (trans_b) { p.b_sn = K; p.b_sk = 1; } else { p.b_sn = 1; p.b_sk = N; }
  p.grid_limit = num_cu;
  return p;
}

// rows physically padded to `align` per group, or (row_start given) every group's rows at its own start
static GemmParams params_padded(const void* A, const void* B, void* C, const void* sizes, int sizes_i64,
                                const int32_t* row_start, int G, int64_t M, int N, int K, int align, int num_cu) {
  GemmParams p = zero_params();
  p.A = A; p.B = B; p.C = C; p.sizes = sizes; p.sizes_i64 = sizes_i64; p.G = G;
  p.mode = MODE_MG_PAD; p.align = row_start ? 1 : align; p.row_start = row_start; p.m_total = M; p.N = N; p.K = K;
  p.a_sm = K; p.a_sk = 1; p.b_sg = (int64_t)N * K; p.b_sn = K; p.b_sk = 1;
  p.grid_limit = num_cu;
  return p;
}

static GemmParams params_masked(const void* A, const void* B, void* C, const void* masked_m, int masked_i64, int G,
                                int64_t m_stride, int64_t M, int N, int K, int trans_b, int num_cu) {
  GemmParams p = zero_params();
  p.A = A; p.B = B; p.C = C; p.sizes = masked_m; p.sizes_i64 = masked_i64; p.G = G;
  p.mode = MODE_MASKED; p.m_stride = m_stride; p.m_total = M; p.N = N; p.K = K;
  p.a_sm = K; p.a_sk = 1; p.b_sg = (int64_t)N * K;
  if (trans_b) { p.b_sn = K; p.b_sk = 1; } else { p.b_sn = 1; p.b_sk = N; }
  p.grid_limit = num_cu;
  return p;
}

static GemmParams params_k_grouped(const void* A, const void* B, void* C, const int32_t* start, const int32_t* end,
                                   int G, int Mdim, int N, int64_t Ktot, int num_cu, int32_t* queue) {
  GemmParams p = zero_params();
  p.A = A; p.B = B; p.C = C; p.k_start = start; p.k_end = end; p.G = G;
  p.mode = MODE_KG; p.m_total = Mdim; p.k_total = Ktot; p.N = N; p.K = 0;
  p.a_sm = 1; p.a_sk = Mdim; p.b_sg = 0; p.b_sn = 1; p.b_sk = N; p.c_sg = (int64_t)Mdim * N;
  p.grid_limit = num_cu;
  p.queue = queue;
  return p;
}

static GemmParams params_fp8_channel(const void* Aq, const float* a_scale, const void* Bq, const float* b_scale,
                                     void* C, const void* sizes, int sizes_i64, int G, int64_t M, int N, int K,
                                     int num_cu) {
  GemmParams p = zero_params();
  p.A = Aq; p.B = Bq; p.C = C; p.sizes = sizes; p.sizes_i64 = sizes_i64; p.G = G;
  p.scale_m = a_scale; p.scale_n = b_scale;
  p.mode = MODE_MG; p.m_total = M; p.N = N; p.K = K;
  p.a_sm = K; p.a_sk = 1; p.b_sg = (int64_t)N * K; p.b_sn = K; p.b_sk = 1;
  p.grid_limit = num_cu;
  return p;
}

static GemmParams params_fp8_k_channel(const void* x, const float* xs, const void* y, const float* ys, void* out,
                                       const int32_t* tokens, int G, int M, int N, int64_t Ktot, int num_cu,
                                       int32_t* queue) {
  GemmParams p = zero_params();
  p.A = x; p.B = y; p.C = out; p.sizes = tokens; p.sizes_i64 = 0; p.G = G;
  p.scale_m = xs; p.scale_n = ys; p.scale_m_sg = M;
  p.mode = MODE_KG_COUNT; p.m_total = M; p.k_total = Ktot; p.N = N; p.K = 0;
  p.a_sm = Ktot; p.a_sk = 1; p.b_sg = 0; p.b_sn = Ktot; p.b_sk = 1; p.c_sg = (int64_t)M * N;
  p.grid_limit = num_cu;
  p.queue = queue;
  return p;
}

static GemmParams params_fp8_block(const void* Aq, const float* sa, const void* Bq, const float* sb, void* C,
                                   const void* sizes, int sizes_i64, const int32_t* row_start, int G, int64_t M, int N,
                                   int K, int align, int sa_mn_major, int num_cu) {
  GemmParams p = zero_params();
  p.A = Aq; p.B = Bq; p.C = C; p.sizes = sizes; p.sizes_i64 = sizes_i64; p.G = G;
  p.sa = sa; p.sb = sb;
  const int kblocks = (K + 127) / 128;
  if (sa_mn_major) { p.sa_rs = 1; p.sa_ks = M; } else { p.sa_rs = kblocks; p.sa_ks = 1; }
  p.mode = MODE_MG_PAD; p.align = row_start ? 1 : align; p.row_start = row_start; p.m_total = M; p.N = N; p.K = K;
  p.a_sm = K; p.a_sk = 1; p.b_sg = (int64_t)N * K; p.b_sn = K; p.b_sk = 1;
  p.grid_limit = num_cu;
  return p;
}

static int dispatch_16bit(const GemmParams& p, int dt, int layout, hipStream_t s) {
  const int force_generic = g_force_generic.load(), four_wave = g_four_wave.load();
  if (!force_generic && four_wave && w4_supported(p, dt, layout, four_wave == 2)) {
    if (!w4_decided_on_device(p) || four_wave == 2) return launch_w4_16bit(p, dt, layout, s);
    // whether 256-row tiles pay depends on the sizes; both kernels look at them and exactly one runs
    GemmParams q = p;
    q.wide_gate = 1;
    if (int e = launch_w4_16bit(q, dt, layout, s)) return e;
    q.wide_gate = 2;
    return launch_fast_16bit(q, dt, layout, s);
  }
  if (!force_generic && fast_supported(p, dt, layout)) return launch_fast_16bit(p, dt, layout, s);
  return launch_generic_16bit(p, dt, layout, s);
}

}  // namespace tgg

using namespace tgg;

// Host-side run of the device scheduler (same functions, see sched.hpp).
template <int BM, int BN>
static int tile_order_host(const GemmParams& p, int grid, int split, int64_t* out, int64_t capacity, int64_t* num_tiles) {
  SchedTable* t = new SchedTable;
  for (int g = 0; g < p.G; ++g) sched_load_group(p, *t, g);
  sched_prefix<BM>(p, *t);
  if (p.mode == MODE_KG || p.mode == MODE_KG_COUNT) sched_order_groups_serial(p, *t);
  const int64_t total = sched_num_tiles<BM, BN>(p, *t);
  *num_tiles = total;
  int64_t n = 0;
  for (int b = 0; b < grid; ++b) {
    const TileWalk w = sched_walk_of(total, split != 0, grid, b);
    int64_t pos = 0;
    int g_prev = -1;  // the kernels pass the previous tile's group as a search hint: it must not change the answer
    for (int64_t id = w.first; id < w.end; id += w.stride, ++pos) {
      const Tile tl = sched_tile<BM, BN>(p, *t, id);
      const Tile th = sched_tile<BM, BN>(p, *t, id, g_prev);
      if (th.g != tl.g || th.row0 != tl.row0 || th.rows != tl.rows || th.n0 != tl.n0 || th.k0 != tl.k0 || th.k1 != tl.k1) {
        delete t;
        return set_error("hinted tile lookup differs at tile %lld (hint %d)", (long long)id, g_prev);
      }
      g_prev = tl.g;
      if (n < capacity) {
        int64_t* r = out + n * 6;
        r[0] = b; r[1] = pos; r[2] = tl.g; r[3] = tl.row0; r[4] = tl.rows; r[5] = tl.n0;
      }
      ++n;
    }
  }
  delete t;
  return n <= capacity ? 0 : set_error("tile order needs %lld rows, capacity %lld", (long long)n, (long long)capacity);
}


// Host-side walk of the shape-agnostic kernel's address arithmetic (generic_addr.hpp) over every tile of a launch:
// lowest and highest element each operand is touched at.  out[op][0..1], op = A, B, C, scale_m, scale_n, sa, sb;
// an operand that is never touched reports {INT64_MAX, -1}.
template <bool A_KMAJOR, bool B_KMAJOR>
static void generic_extents_host(const GemmParams& p, int epi, int64_t* out) {
  SchedTable* t = new SchedTable;
  for (int g = 0; g < p.G; ++g) sched_load_group(p, *t, g);
  if (p.mode != MODE_KG) sched_prefix<kGenericBM>(p, *t);
  if (generic_kmode(p)) sched_order_groups_serial(p, *t);
  const int64_t total = sched_num_tiles<kGenericBM, kGenericBN>(p, *t);
  for (int op = 0; op < 7; ++op) { out[2 * op] = INT64_MAX; out[2 * op + 1] = -1; }
  auto touch = [&](int op, int64_t lo, int64_t hi) {
    if (lo < out[2 * op]) out[2 * op] = lo;
    if (hi > out[2 * op + 1]) out[2 * op + 1] = hi;
  };
  for (int64_t id = 0; id < total; ++id) {
    const Tile tl = sched_tile<kGenericBM, kGenericBN>(p, *t, id);
    const GenericTileIo io = generic_tile_io<A_KMAJOR>(p, tl);
    const int64_t klen = tl.k1 - tl.k0;
    const int kt_n = (int)((klen + kGenericBK - 1) / kGenericBK);
    if (kt_n > 0 && io.a_lim > 0) {
      if (A_KMAJOR) touch(0, io.a_elem + generic_elem_kmajor(0, p.a_sm, tl.k0), io.a_elem + generic_elem_kmajor(io.a_lim - 1, p.a_sm, tl.k1 - 1));
      else touch(0, io.a_elem + generic_elem_mnmajor(tl.k0, p.a_sk, 0), io.a_elem + generic_elem_mnmajor(tl.k1 - 1, p.a_sk, io.a_lim - 1));
    }
    if (kt_n > 0 && io.b_lim > 0) {
      if (B_KMAJOR) touch(1, io.b_elem + generic_elem_kmajor(0, p.b_sn, tl.k0), io.b_elem + generic_elem_kmajor(io.b_lim - 1, p.b_sn, tl.k1 - 1));
      else touch(1, io.b_elem + generic_elem_mnmajor(tl.k0, p.b_sk, 0), io.b_elem + generic_elem_mnmajor(tl.k1 - 1, p.b_sk, io.b_lim - 1));
    }
    if (tl.rows > 0 && io.b_lim > 0) {
      touch(2, io.c_elem + tl.n0, io.c_elem + (int64_t)(tl.rows - 1) * p.N + tl.n0 + io.b_lim - 1);
      if (epi == 1) {
        touch(3, generic_scale_m_index(p, tl, 0), generic_scale_m_index(p, tl, tl.rows - 1));
        touch(4, generic_scale_n_index(p, tl, tl.n0), generic_scale_n_index(p, tl, tl.n0 + io.b_lim - 1));
      }
    }
    if (epi == 2 && kt_n > 0) {
      const int kb_last = generic_scale_block_of_slab(kt_n - 1);
      touch(6, generic_sb_index(p, tl, 0), generic_sb_index(p, tl, kb_last));
      if (tl.rows > 0) {
        for (int kb = 0; kb <= kb_last; kb += (kb_last > 0 ? kb_last : 1)) {
          touch(5, generic_sa_index(p, tl, 0, kb), generic_sa_index(p, tl, 0, kb));
          touch(5, generic_sa_index(p, tl, tl.rows - 1, kb), generic_sa_index(p, tl, tl.rows - 1, kb));
        }
      }
    }
  }
  delete t;
}

extern "C" {

int tgg_m_grouped_gemm(const void* A, const void* B, void* C, const void* sizes, int sizes_i64, int G, int64_t M,
                       int N, int K, int trans_b, int dtype, int num_cu, void* stream) {
  if (int e = check_common(A, B, C, sizes, G, N, TGG_MAX_GROUPS)) return e;
  if (M < 0 || K < 0) return set_error("negative M or K");
  if (dtype != TGG_BF16 && dtype != TGG_F16) return set_error("data type code %d not supported", dtype);
  if ((K & 7) || (N & 7)) return set_error("N and K must be multiples of 8 (16-byte rows), got N=%d K=%d", N, K);
  if (M == 0) return 0;
  const GemmParams p = params_m_grouped(A, B, C, sizes, sizes_i64, G, M, N, K, trans_b, num_cu);
  return dispatch_16bit(p, dtype, trans_b ? 0 : 1, (hipStream_t)stream);
}

int tgg_m_grouped_gemm_fp8_out(const void* A, const void* B, void* codes, float* scales, const void* sizes,
                               int sizes_i64, int G, int64_t M, int N, int K, int trans_b, int dtype, int fmt,
                               int scales_mn_major, int num_cu, void* stream) {
  if (int e = check_common(A, B, codes, sizes, G, N)) return e;
  if (!scales) return set_error("null scale pointer");
  if (M < 0 || K < 0) return set_error("negative M or K");
  if (dtype != TGG_BF16 && dtype != TGG_F16) return set_error("data type code %d not supported", dtype);
  if (fmt != DT_E4M3 && fmt != DT_E5M2) return set_error("unsupported fp8 format code %d", fmt);
  if ((K & 7) || (N & 127)) return set_error("K must be a multiple of 8 and N of 128, got N=%d K=%d", N, K);
  if (M == 0) return 0;
  GemmParams p = params_m_grouped(A, B, codes, sizes, sizes_i64, G, M, N, K, trans_b, num_cu);
  p.q_scales = scales;
  p.q_fmt = fmt;
  if (scales_mn_major) { p.q_rs = 1; p.q_bs = M; } else { p.q_rs = N / 128; p.q_bs = 1; }
  const int layout = trans_b ? 0 : 1;
  if (!fast_quant_supported(p, dtype, layout))
    return set_error("shape outside the fused kernel's domain (G <= 512, K * 512 and N * 128 below 2^30 bytes): "
                     "run tgg_m_grouped_gemm followed by tgg_per_token_cast_to_fp8, which gives the same bits");
  return launch_fast_16bit_quant(p, dtype, layout, (hipStream_t)stream);
}

int tgg_m_grouped_gemm_padded(const void* A, const void* B, void* C, const void* sizes, int sizes_i64, int G,
                              int64_t M, int N, int K, int align, int dtype, int num_cu, void* stream) {
  if (int e = check_common(A, B, C, sizes, G, N)) return e;
  if (M < 0 || K < 0) return set_error("negative M or K");
  if (align < 1) return set_error("alignment must be positive, got %d", align);
  if (dtype != TGG_BF16 && dtype != TGG_F16) return set_error("data type code %d not supported", dtype);
  if ((K & 7) || (N & 7)) return set_error("N and K must be multiples of 8 (16-byte rows), got N=%d K=%d", N, K);
  if (M == 0) return 0;
  const GemmParams p = params_padded(A, B, C, sizes, sizes_i64, nullptr, G, M, N, K, align, num_cu);
  return dispatch_16bit(p, dtype, 0, (hipStream_t)stream);
}

int tgg_m_grouped_gemm_placed(const void* A, const void* B, void* C, const void* sizes, int sizes_i64,
                              const int32_t* row_start, int G, int64_t M, int N, int K, int dtype, int num_cu,
                              void* stream) {
  if (int e = check_common(A, B, C, sizes, G, N)) return e;
  if (!row_start) return set_error("null row_start pointer");
  if (M < 0 || K < 0) return set_error("negative M or K");
  if (M >= (1ll << 31)) return set_error("M=%lld does not fit 32-bit row starts", (long long)M);
  if (dtype != TGG_BF16 && dtype != TGG_F16) return set_error("data type code %d not supported", dtype);
  if ((K & 7) || (N & 7)) return set_error("N and K must be multiples of 8 (16-byte rows), got N=%d K=%d", N, K);
  if (M == 0) return 0;
  const GemmParams p = params_padded(A, B, C, sizes, sizes_i64, row_start, G, M, N, K, 1, num_cu);
  return dispatch_16bit(p, dtype, 0, (hipStream_t)stream);
}

int tgg_m_grouped_gemm_masked(const void* A, const void* B, void* C, const void* masked_m, int masked_i64, int G,
                              int64_t m_stride, int64_t M, int N, int K, int trans_b, int dtype, int num_cu,
                              void* stream) {
  if (int e = check_common(A, B, C, masked_m, G, N)) return e;
  if (M < 0 || K < 0 || m_stride < 0) return set_error("negative M, K or m_stride");
  if (dtype != TGG_BF16 && dtype != TGG_F16) return set_error("data type code %d not supported", dtype);
  if ((K & 7) || (N & 7)) return set_error("N and K must be multiples of 8 (16-byte rows), got N=%d K=%d", N, K);
  if (M == 0 || m_stride == 0) return 0;
  const GemmParams p = params_masked(A, B, C, masked_m, masked_i64, G, m_stride, M, N, K, trans_b, num_cu);
  return dispatch_16bit(p, dtype, trans_b ? 0 : 1, (hipStream_t)stream);
}

int tgg_k_grouped_gemm(const void* A, const void* B, void* C, const int32_t* start, const int32_t* end, int G,
                       int Mdim, int N, int64_t Ktot, int dtype, int num_cu, void* stream) {
  return tgg_k_grouped_gemm_queued(A, B, C, start, end, G, Mdim, N, Ktot, dtype, num_cu, nullptr, stream);
}

int tgg_k_grouped_gemm_queued(const void* A, const void* B, void* C, const int32_t* start, const int32_t* end, int G,
                              int Mdim, int N, int64_t Ktot, int dtype, int num_cu, int32_t* queue, void* stream) {
  if (int e = check_common(A, B, C, start, G, N, TGG_MAX_GROUPS)) return e;
  if (!end) return set_error("null group_end pointer");
  if (Mdim < 1 || Ktot < 0) return set_error("bad Mdim=%d or Ktot=%lld", Mdim, (long long)Ktot);
  if (dtype != TGG_BF16 && dtype != TGG_F16) return set_error("data type code %d not supported", dtype);
  if ((Mdim & 7) || (N & 7)) return set_error("Mdim and N must be multiples of 8 (16-byte rows), got %d, %d", Mdim, N);
  const GemmParams p = params_k_grouped(A, B, C, start, end, G, Mdim, N, Ktot, num_cu, queue);
  return dispatch_16bit(p, dtype, 2, (hipStream_t)stream);
}

static bool is_fp8(int f) { return f == TGG_E4M3 || f == TGG_E5M2; }

int tgg_m_grouped_gemm_fp8_channel(const void* Aq, const float* a_scale, const void* Bq, const float* b_scale,
                                   void* C, const void* sizes, int sizes_i64, int G, int64_t M, int N, int K,
                                   int fmt_a, int fmt_b, int out_dtype, int num_cu, void* stream) {
  if (int e = check_common(Aq, Bq, C, sizes, G, N)) return e;
  if (!a_scale || !b_scale) return set_error("null scale pointer");
  if (M < 0 || K < 0) return set_error("negative M or K");
  if (!is_fp8(fmt_a) || !is_fp8(fmt_b)) return set_error("fp8 format codes must be E4M3 or E5M2");
  if (K & 15) return set_error("K must be a multiple of 16 for fp8 operands, got %d", K);
  if (M == 0) return 0;
  const GemmParams p = params_fp8_channel(Aq, a_scale, Bq, b_scale, C, sizes, sizes_i64, G, M, N, K, num_cu);
  if (!g_force_generic.load() && fast_fp8_supported(p, false)) return launch_fast_fp8_channel(p, fmt_a, fmt_b, out_dtype, (hipStream_t)stream);
  return launch_generic_fp8_channel(p, fmt_a, fmt_b, out_dtype, (hipStream_t)stream);
}

int tgg_k_grouped_gemm_fp8_channel(const void* x, const float* xs, const void* y, const float* ys, void* out,
                                   const int32_t* tokens, int G, int M, int N, int64_t Ktot, int fmt_a, int fmt_b,
                                   int num_cu, void* stream) {
  return tgg_k_grouped_gemm_fp8_channel_queued(x, xs, y, ys, out, tokens, G, M, N, Ktot, fmt_a, fmt_b, num_cu, nullptr, stream);
}

int tgg_k_grouped_gemm_fp8_channel_queued(const void* x, const float* xs, const void* y, const float* ys, void* out,
                                          const int32_t* tokens, int G, int M, int N, int64_t Ktot, int fmt_a,
                                          int fmt_b, int num_cu, int32_t* queue, void* stream) {
  if (int e = check_common(x, y, out, tokens, G, N)) return e;
  if (!xs || !ys) return set_error("null scale pointer");
  if (M < 1 || Ktot < 0) return set_error("bad M=%d or Ktot=%lld", M, (long long)Ktot);
  if (!is_fp8(fmt_a) || !is_fp8(fmt_b)) return set_error("fp8 format codes must be E4M3 or E5M2");
  if (Ktot & 15) return set_error("Ktot must be a multiple of 16 for fp8 operands, got %lld", (long long)Ktot);
  GemmParams p = params_fp8_k_channel(x, xs, y, ys, out, tokens, G, M, N, Ktot, num_cu, queue);
  if (!g_force_generic.load() && fast_fp8_supported(p, false)) {
    // The tuned kernel needs every token count to be a multiple of 16 and only the device knows the counts: both
    // kernels are enqueued, each reads the counts first and exactly one of them runs (the other returns at once).
    p.kg_gate = 1;
    if (int e = launch_fast_fp8_channel(p, fmt_a, fmt_b, TGG_BF16, (hipStream_t)stream)) return e;
    if (!g_kg_second_launch.load()) return 0;
    p.kg_gate = 2;
  }
  return launch_generic_fp8_channel(p, fmt_a, fmt_b, TGG_BF16, (hipStream_t)stream);
}

static int fp8_block_impl(const void* Aq, const float* sa, const void* Bq, const float* sb, void* C, const void* sizes,
                          int sizes_i64, const int32_t* row_start, int G, int64_t M, int N, int K, int align,
                          int sa_mn_major, int num_cu, void* stream) {
  if (int e = check_common(Aq, Bq, C, sizes, G, N)) return e;
  if (!sa || !sb) return set_error("null scale pointer");
  if (M < 0 || K < 0) return set_error("negative M or K");
  if (row_start && M >= (1ll << 31)) return set_error("M=%lld does not fit 32-bit row starts", (long long)M);
  if (!row_start && (align < 1 || (align & 127))) return set_error("alignment must be a positive multiple of 128, got %d", align);
  if (K & 15) return set_error("K must be a multiple of 16 for fp8 operands, got %d", K);
  if (M == 0) return 0;
  const GemmParams p = params_fp8_block(Aq, sa, Bq, sb, C, sizes, sizes_i64, row_start, G, M, N, K, align, sa_mn_major, num_cu);
  const int kblocks = (K + 127) / 128;
  if (!g_force_generic.load() && sa_mn_major && kblocks <= 64 && fast_fp8_supported(p, true))
    return launch_fast_fp8_block(p, (hipStream_t)stream);
  return launch_generic_fp8_block(p, (hipStream_t)stream);
}

int tgg_m_grouped_gemm_fp8_block(const void* Aq, const float* sa, const void* Bq, const float* sb, void* C,
                                 const void* sizes, int sizes_i64, int G, int64_t M, int N, int K, int align,
                                 int sa_mn_major, int num_cu, void* stream) {
  return fp8_block_impl(Aq, sa, Bq, sb, C, sizes, sizes_i64, nullptr, G, M, N, K, align, sa_mn_major, num_cu, stream);
}

int tgg_m_grouped_gemm_fp8_block_placed(const void* Aq, const float* sa, const void* Bq, const float* sb, void* C,
                                        const void* sizes, int sizes_i64, const int32_t* row_start, int G, int64_t M,
                                        int N, int K, int sa_mn_major, int num_cu, void* stream) {
  if (!row_start) return set_error("null row_start pointer");
  return fp8_block_impl(Aq, sa, Bq, sb, C, sizes, sizes_i64, row_start, G, M, N, K, 128, sa_mn_major, num_cu, stream);
}

int tgg_trans_per_block_quant_expand_128x(const void* x, void* codes, float* scales, const void* sizes,
                                          int sizes_i64, int G, int64_t M, int N, int64_t M_expand, int fmt,
                                          void* stream) {
  if ((!x && M > 0) || !codes || !scales || !sizes) return set_error("null pointer");
  if (G < 1 || G > TGG_MAX_GROUPS) return set_error("G=%d outside [1, %d]", G, TGG_MAX_GROUPS);
  if (N < 128 || (N & 127)) return set_error("N must be a positive multiple of 128, got %d", N);
  if (M < 0 || M_expand < 0 || (M_expand & 127)) return set_error("M_expand must be a multiple of 128");
  if (M_expand < ((M + 127) / 128) * 128) return set_error("M_expand=%lld too small for M=%lld", (long long)M_expand, (long long)M);
  if (!aligned16(x) || !aligned16(codes)) return set_error("operand pointers must be 16-byte aligned");
  if (M_expand == 0) return 0;
  GemmParams p = zero_params();
  p.sizes = sizes; p.sizes_i64 = sizes_i64; p.G = G; p.mode = MODE_MG; p.m_total = M; p.N = N;
  return launch_trans_quant128(x, codes, scales, p, M_expand, fmt, (hipStream_t)stream);
}

int tgg_per_token_cast_to_fp8(const void* x, void* codes, float* scales, int64_t M, int K, int fmt,
                              int scales_mn_major, void* stream) {
  if (!x || !codes || !scales) return set_error("null pointer");
  if (M < 0 || K < 0 || (K & 127)) return set_error("K must be a multiple of 128, got %d", K);
  if (!aligned16(x) || !aligned16(codes)) return set_error("operand pointers must be 16-byte aligned");
  return launch_token_cast128(x, codes, scales, M, K / 128, scales_mn_major, fmt, (hipStream_t)stream);
}

int tgg_per_block_cast_to_fp8(const void* x, void* codes, float* scales, int batch, int R, int C, int fmt,
                              void* stream) {
  if (!x || !codes || !scales) return set_error("null pointer");
  if (batch < 0 || R < 0 || C < 0) return set_error("negative shape");
  if (!aligned16(x) || !aligned16(codes)) return set_error("operand pointers must be 16-byte aligned");
  return launch_block_cast128(x, codes, scales, batch, R, C, fmt, (hipStream_t)stream);
}

int tgg_cvt_f32_to_fp8(const float* in, void* out, int64_t n, int fmt, void* stream) {
  if (!in || !out || n < 0) return set_error("bad arguments");
  return launch_cvt_fp8(in, out, n, fmt, (hipStream_t)stream);
}

// ---- MoE permute / unpermute ----------------------------------------------------------------------------------
static int moe_row_bytes(int hidden, int dtype, int64_t* row_bytes) {
  int esz;
  if (dtype == DT_BF16 || dtype == DT_F16) esz = 2;
  else if (dtype == DT_E4M3 || dtype == DT_E5M2) esz = 1;
  else if (dtype == 4) esz = 4;
  else return set_error("unsupported activation dtype code %d", dtype);
  if (hidden < 1) return set_error("hidden size must be positive");
  *row_bytes = (int64_t)hidden * esz;
  if (*row_bytes % 16 != 0) return set_error("rows must be a multiple of 16 bytes (hidden=%d, %d-byte elements)", hidden, esz);
  return 0;
}

int tgg_moe_sort_workspace_bytes(int64_t num_tokens, int topk, int num_experts, int64_t* bytes) {
  if (!bytes) return set_error("null pointer");
  if (num_tokens < 0 || topk < 1) return set_error("bad num_tokens / topk");
  if (num_experts < 1 || num_experts > 1024) return set_error("num_experts=%d outside [1, 1024]", num_experts);
  *bytes = moe_sort_workspace_bytes(num_tokens * topk, num_experts);
  return 0;
}

int tgg_moe_permute_map(const int32_t* indices, int64_t num_tokens, int topk, int num_experts, int64_t num_out_tokens,
                        int32_t* row_id_map, void* tokens_per_expert, int counts_i64, void* workspace,
                        int64_t workspace_bytes, void* stream) {
  if (num_tokens < 0 || topk < 1) return set_error("bad num_tokens / topk");
  if (num_tokens * topk >= (1ll << 31)) return set_error("num_tokens * topk must stay below 2^31");
  if (num_experts < 1 || num_experts > 1024) return set_error("num_experts=%d outside [1, 1024]", num_experts);
  if (!workspace || (num_tokens > 0 && (!indices || !row_id_map))) return set_error("null pointer");
  if (workspace_bytes < moe_sort_workspace_bytes(num_tokens * topk, num_experts))
    return set_error("workspace of %lld bytes is too small (need %lld)", (long long)workspace_bytes,
                     (long long)moe_sort_workspace_bytes(num_tokens * topk, num_experts));
  const int64_t capacity = num_out_tokens > 0 ? num_out_tokens : num_tokens * topk;
  return launch_moe_permute_map(indices, num_tokens, topk, num_experts, capacity, row_id_map, tokens_per_expert,
                                counts_i64, workspace, (hipStream_t)stream);
}

int tgg_moe_permute_map_static(const int32_t* indices, int64_t num_tokens, int topk, int num_experts,
                               int64_t num_out_tokens, int32_t* row_id_map, void* tokens_per_expert, int counts_i64,
                               void* stream) {
  if (num_tokens < 0 || topk < 1) return set_error("bad num_tokens / topk");
  if (num_tokens >= (1ll << 31) / topk) return set_error("num_tokens * topk must stay below 2^31");
  if (num_experts < 1 || num_experts > 1024) return set_error("num_experts=%d outside [1, 1024]", num_experts);
  if (num_tokens > 0 && (!indices || !row_id_map)) return set_error("null pointer");
  const int64_t capacity = num_out_tokens > 0 ? num_out_tokens : num_tokens * topk;
  return launch_moe_permute_map_static(indices, num_tokens, topk, num_experts, capacity, row_id_map, tokens_per_expert,
                                       counts_i64, (hipStream_t)stream);
}

int tgg_moe_permute_rows(const void* input, void* permuted, const int32_t* row_id_map, int64_t num_tokens, int topk,
                         int hidden, int dtype, void* stream) {
  int64_t rb;
  if (moe_row_bytes(hidden, dtype, &rb)) return 1;
  if (num_tokens < 0 || topk < 1) return set_error("bad num_tokens / topk");
  if (num_tokens > 0 && (!input || !permuted || !row_id_map)) return set_error("null pointer");
  if (!aligned16(input) || !aligned16(permuted)) return set_error("activation pointers must be 16-byte aligned");
  return launch_moe_permute_rows(input, permuted, row_id_map, num_tokens, topk, rb, (hipStream_t)stream);
}

int tgg_moe_unpermute(const void* input, void* output, const int32_t* row_id_map, const float* probs,
                      int64_t num_tokens, int topk, int hidden, int dtype, void* stream) {
  int64_t rb;
  if (moe_row_bytes(hidden, dtype, &rb)) return 1;
  if (dtype == DT_E4M3 || dtype == DT_E5M2) return set_error("unpermute computes in fp32 on bf16 / fp16 / fp32 rows only");
  if (num_tokens < 0 || topk < 1) return set_error("bad num_tokens / topk");
  if (num_tokens > 0 && (!input || !output || !row_id_map)) return set_error("null pointer");
  if (!aligned16(input) || !aligned16(output)) return set_error("activation pointers must be 16-byte aligned");
  return launch_moe_unpermute(input, output, row_id_map, probs, num_tokens, topk, rb, dtype, (hipStream_t)stream);
}

int tgg_moe_unpermute_bwd(const void* grad_output, const void* fwd_input, const int32_t* row_id_map, const float* probs,
                          void* act_grad, float* prob_grad, int64_t num_tokens, int topk, int hidden, int dtype,
                          void* stream) {
  int64_t rb;
  if (moe_row_bytes(hidden, dtype, &rb)) return 1;
  if (dtype == DT_E4M3 || dtype == DT_E5M2) return set_error("unpermute computes in fp32 on bf16 / fp16 / fp32 rows only");
  if (num_tokens < 0 || topk < 1) return set_error("bad num_tokens / topk");
  if (num_tokens > 0 && (!grad_output || !act_grad || !row_id_map)) return set_error("null pointer");
  if (prob_grad && (!probs || !fwd_input)) return set_error("prob_grad needs probs and the forward input");
  if (!aligned16(grad_output) || !aligned16(act_grad) || !aligned16(fwd_input))
    return set_error("activation pointers must be 16-byte aligned");
  return launch_moe_unpermute_bwd(grad_output, fwd_input, row_id_map, probs, act_grad, prob_grad, num_tokens, topk, rb,
                                  dtype, (hipStream_t)stream);
}

int tgg_debug_tile_order(const int64_t* sizes, int G, int mode, int64_t m_total, int64_t aux, int N, int tile,
                         int grid, int split, int64_t* out, int64_t capacity, int64_t* num_tiles) {
  if (!sizes || !out || !num_tiles) return set_error("null pointer");
  if (G < 1 || G > TGG_MAX_GROUPS) return set_error("G=%d outside [1, %d]", G, TGG_MAX_GROUPS);
  if (N < 1 || grid < 1 || m_total < 0) return set_error("bad N / grid / m_total");
  if (mode != MODE_MG && mode != MODE_MG_PAD && mode != MODE_MASKED && mode != MODE_KG_COUNT)
    return set_error("mode %d not supported by the tile-order hook", mode);
  GemmParams p = zero_params();
  p.sizes = sizes;
  p.sizes_i64 = 1;
  p.G = G;
  p.mode = mode;
  p.m_total = m_total;
  p.N = N;
  p.align = mode == MODE_MG_PAD ? (int)aux : 1;
  p.m_stride = mode == MODE_MASKED ? aux : 0;
  p.k_total = mode == MODE_KG_COUNT ? aux : 0;
  if (mode == MODE_MG_PAD && p.align < 1) return set_error("alignment must be positive");
  if (tile == 256) return tile_order_host<256, 256>(p, grid, split, out, capacity, num_tiles);
  if (tile == 128) return tile_order_host<128, 128>(p, grid, split, out, capacity, num_tiles);
  return set_error("tile must be 256 (tuned kernels) or 128 (shape-agnostic kernel)");
}

int tgg_debug_generic_extents(int kind, const int64_t* sizes, const int32_t* row_start, int G, int64_t M, int64_t aux,
                              int N, int K, int64_t* out) {
  if (!sizes || !out) return set_error("null pointer");
  if (G < 1 || G > TGG_MAX_GROUPS) return set_error("G=%d outside [1, %d]", G, TGG_MAX_GROUPS);
  if (N < 1 || M < 0 || K < 0) return set_error("bad M / N / K");
  // Non-null dummies: the walk computes offsets, it dereferences only `sizes`, `row_start` and the k ranges.
  static char dummy;
  const void* D = &dummy;
  std::vector<int32_t> counts(sizes, sizes + G), ks(G), ke(G);
  switch (kind) {
    case 0: case 1: {  // tgg_m_grouped_gemm, trans_b = 1 / 0
      const GemmParams p = params_m_grouped(D, D, &dummy, sizes, 1, G, M, N, K, kind == 0, -1);
      if (kind == 0) generic_extents_host<true, true>(p, 0, out); else generic_extents_host<true, false>(p, 0, out);
      return 0;
    }
    case 2: {  // tgg_m_grouped_gemm_masked, aux = m_stride
      const GemmParams p = params_masked(D, D, &dummy, sizes, 1, G, aux, M, N, K, 1, -1);
      generic_extents_host<true, true>(p, 0, out);
      return 0;
    }
    case 3: case 4: {  // tgg_m_grouped_gemm_padded (aux = align) / _placed (row_start)
      if (kind == 4 && !row_start) return set_error("placed launches need row_start");
      if (kind == 3 && aux < 1) return set_error("alignment must be positive");
      const GemmParams p = params_padded(D, D, &dummy, sizes, 1, kind == 4 ? row_start : nullptr, G, M, N, K, (int)aux, -1);
      generic_extents_host<true, true>(p, 0, out);
      return 0;
    }
    case 5: {  // tgg_k_grouped_gemm: sizes = token counts, M = Mdim, aux = Ktot
      int64_t at = 0;
      for (int g = 0; g < G; ++g) { ks[g] = (int32_t)at; at += sizes[g] < 0 ? 0 : sizes[g]; ke[g] = (int32_t)at; }
      const GemmParams p = params_k_grouped(D, D, &dummy, ks.data(), ke.data(), G, (int)M, N, aux, -1, nullptr);
      generic_extents_host<false, false>(p, 0, out);
      return 0;
    }
    case 6: {  // tgg_m_grouped_gemm_fp8_channel
      const GemmParams p = params_fp8_channel(D, (const float*)D, D, (const float*)D, &dummy, sizes, 1, G, M, N, K, -1);
      generic_extents_host<true, true>(p, 1, out);
      return 0;
    }
    case 7: {  // tgg_k_grouped_gemm_fp8_channel: sizes = token counts (int32 in the ABI), M rows of x, aux = Ktot
      const GemmParams p = params_fp8_k_channel(D, (const float*)D, D, (const float*)D, &dummy, counts.data(), G, (int)M, N, aux, -1, nullptr);
      generic_extents_host<true, true>(p, 1, out);
      return 0;
    }
    case 8: case 9: case 10: {  // tgg_m_grouped_gemm_fp8_block: aux = align; 8 = sa [M, KB], 9 = sa [KB, M], 10 = placed ([KB, M])
      if (kind == 10 && !row_start) return set_error("placed launches need row_start");
      const GemmParams p = params_fp8_block(D, (const float*)D, D, (const float*)D, &dummy, sizes, 1,
                                            kind == 10 ? row_start : nullptr, G, M, N, K, (int)aux, kind != 8, -1);
      generic_extents_host<true, true>(p, 2, out);
      return 0;
    }
  }
  return set_error("unknown kind %d", kind);
}

int tgg_debug_queue_order(int grid, int draws, int32_t* out) {
  if (!out) return set_error("null pointer");
  if (grid < 8 || (grid & 7) != 0) return set_error("a grid of %d workgroups draws from one counter: ids in order", grid);
  if (draws < 0) return set_error("negative number of draws");
  for (int xq = 0; xq < 8; ++xq)
    for (int n = 0; n < draws; ++n) out[(int64_t)xq * draws + n] = sched_queue_id(n, xq, grid >> 3);
  return 0;
}

int tgg_debug_row_tiles(const int64_t* sizes, int G, int mode, int64_t m_total, int64_t aux, int tile, int n_chunk,
                        int64_t* out, int64_t capacity, int64_t* num_row_tiles) {
  if (!sizes || !out || !num_row_tiles) return set_error("null pointer");
  if (G < 1 || G > TGG_MAX_GROUPS) return set_error("G=%d outside [1, %d]", G, TGG_MAX_GROUPS);
  if (m_total < 0) return set_error("bad m_total");
  if (mode != MODE_MG && mode != MODE_MG_PAD && mode != MODE_MASKED)
    return set_error("mode %d not supported by the row-tile hook", mode);
  if (tile != 128 && tile != 256) return set_error("tile must be 128 or 256");
  GemmParams p = zero_params();
  p.sizes = sizes;
  p.sizes_i64 = 1;
  p.G = G;
  p.mode = mode;
  p.m_total = m_total;
  p.N = 128;
  p.n_chunk = n_chunk;  // must not influence the row-tile lookup
  p.align = mode == MODE_MG_PAD ? (int)aux : 1;
  p.m_stride = mode == MODE_MASKED ? aux : 0;
  if (mode == MODE_MG_PAD && p.align < 1) return set_error("alignment must be positive");
  SchedTable* t = new SchedTable;
  for (int g = 0; g < G; ++g) sched_load_group(p, *t, g);
  if (tile == 128) sched_prefix<128>(p, *t); else sched_prefix<256>(p, *t);
  const int total = t->tile0[G];
  *num_row_tiles = total;
  int g_prev = -1;
  for (int mt = 0; mt < total; ++mt) {
    const RowTile a = tile == 128 ? sched_row_tile<128>(*t, G, mt) : sched_row_tile<256>(*t, G, mt);
    const RowTile h = tile == 128 ? sched_row_tile<128>(*t, G, mt, g_prev) : sched_row_tile<256>(*t, G, mt, g_prev);
    if (a.g != h.g || a.row0 != h.row0 || a.rows != h.rows) {
      delete t;
      return set_error("hinted row-tile lookup differs at row tile %d (hint %d)", mt, g_prev);
    }
    g_prev = a.g;
    if (mt < capacity) { out[mt * 3] = a.g; out[mt * 3 + 1] = a.row0; out[mt * 3 + 2] = a.rows; }
  }
  delete t;
  return total <= capacity ? 0 : set_error("row tiles need %d entries, capacity %lld", total, (long long)capacity);
}

int tgg_set_option(const char* key, int value) {
  if (key && strcmp(key, "force_generic") == 0) { g_force_generic = value != 0; return 0; }
  if (key && strcmp(key, "variant") == 0) { set_fast_variant(value); set_fp8_variant(value); return 0; }
  if (key && strcmp(key, "tile_split") == 0) { g_tile_split = value != 0; return 0; }
  if (key && strcmp(key, "n_chunk") == 0) { g_n_chunk = value < 0 ? 0 : value; return 0; }
  if (key && strcmp(key, "kg_second_launch") == 0) { g_kg_second_launch = value != 0; return 0; }
  if (key && strcmp(key, "four_wave") == 0) { g_four_wave = value < 0 ? 0 : (value > 2 ? 2 : value); return 0; }
  if (key && strcmp(key, "store_nt") == 0) { g_store_nt = value != 0; return 0; }
  return set_error("unknown option '%s'", key ? key : "(null)");
}

const char* tgg_last_error(void) { return g_err; }
int tgg_version(void) { return 100; }

}  // extern "C"
