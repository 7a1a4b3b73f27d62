// MoE token permute / unpermute for gfx950: the steps either side of the grouped GEMMs that turn
// [tokens, hidden] activations plus a [tokens, topK] expert assignment into expert-contiguous rows and back.
//
// Sorting is a stable counting sort specialised to the key range (expert ids < 1024), not a general radix
// sort: it needs no temporary storage beyond one small table, and the per-expert row counts that the grouped
// GEMM takes as `size_per_group` fall out of it.
//   count   1024 assignments per workgroup (flat order t * topK + k).  Inside a wave an assignment's rank among
//           equal experts comes from ballots; per-wave counts meet in LDS; the workgroup writes each
//           assignment's rank inside the chunk and the chunk's per-expert totals table[e][chunk].
//   scan    one workgroup per expert turns its row of the table into exclusive prefixes and keeps the total;
//           one workgroup then scans the totals into the experts' first rows.
//   place   destination = expert start + prefix of the chunk + rank in chunk; row_id_map[k * tokens + t] gets
//           it (or -1 for dropped assignments: expert -1, or destination beyond the capacity).
// The row movers are plain streaming kernels (16-byte accesses, one workgroup per token, fp32 arithmetic):
//   permute_rows    reads each token row once and writes it to its up to topK destinations
//   unpermute       out[t] = sum_k prob[t,k] * in[row_id_map[k,t]]
//   unpermute_bwd   act_grad[dest] = prob[t,k] * grad[t];  prob_grad[t,k] = <grad[t], fwd_in[dest]>
#include <mutex>

#include "common.hpp"
#include "launch.hpp"

namespace tgg {

namespace {

constexpr int kChunk = 1024;      // assignments per workgroup of the counting pass
constexpr int kMaxExperts = 1024;

// table[e * chunks + c] = assignments of expert e in chunk c; rank[i] = rank of assignment i among the
// assignments of the same expert in its chunk, in flat order.
__global__ __launch_bounds__(kChunk) void moe_count_kernel(const int32_t* __restrict__ indices, int64_t n,
                                                           int num_experts, int chunks,
                                                           int32_t* __restrict__ table, int32_t* __restrict__ rank) {
  extern __shared__ int32_t wave_cnt[];  // [16 waves][num_experts]
  const int tid = threadIdx.x, wave = tid >> 6;
  const int64_t i = (int64_t)blockIdx.x * kChunk + tid;
  for (int x = tid; x < 16 * num_experts; x += kChunk) wave_cnt[x] = 0;
  __syncthreads();
  int e = -1;
  if (i < n) {
    e = indices[i];
    if (e < 0 || e >= num_experts) e = -1;  // dropped assignment
  }
  // rank among equal experts inside the wave: peel off one distinct expert per round
  int my_rank = 0;
  bool pending = e >= 0;
  const int lane = tid & 63;
  while (true) {
    const uint64_t todo = __ballot(pending);
    if (todo == 0) break;
    const int leader = __builtin_ctzll(todo);
    const int e0 = __builtin_amdgcn_readlane(e, leader);
    const uint64_t same = __ballot(pending && e == e0);
    if (pending && e == e0) {
      my_rank = __builtin_popcountll(same & ((1ull << lane) - 1));
      if (lane == leader) wave_cnt[wave * num_experts + e0] = __builtin_popcountll(same);
      pending = false;
    }
  }
  __syncthreads();
  // exclusive prefix over the 16 waves, per expert; the chunk total goes to the table
  for (int x = tid; x < num_experts; x += kChunk) {
    int run = 0;
    for (int w = 0; w < 16; ++w) {
      const int c = wave_cnt[w * num_experts + x];
      wave_cnt[w * num_experts + x] = run;
      run += c;
    }
    table[(int64_t)x * chunks + blockIdx.x] = run;
  }
  __syncthreads();
  if (i < n) rank[i] = e >= 0 ? wave_cnt[wave * num_experts + e] + my_rank : 0;
}

// Workgroup-wide exclusive scan of one value per thread (256 threads); returns the prefix, total in *total.
TGG_DEV int block_exclusive_scan_256(int v, int* lds /* 8 ints */, int* total) {
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  int incl = v;
#pragma unroll
  for (int d = 1; d < 64; d <<= 1) {
    const int up = __shfl_up(incl, d, 64);
    if (lane >= d) incl += up;
  }
  if (lane == 63) lds[wave] = incl;
  __syncthreads();
  int base = 0, sum = 0;
  for (int w = 0; w < 4; ++w) {
    const int c = lds[w];
    if (w < wave) base += c;
    sum += c;
  }
  __syncthreads();
  *total = sum;
  return base + incl - v;
}

// One workgroup per expert: its table row becomes exclusive prefixes over the chunks; totals[e] = row sum.
__global__ __launch_bounds__(256) void moe_scan_rows_kernel(int32_t* __restrict__ table, int chunks,
                                                            int32_t* __restrict__ totals) {
  __shared__ int lds[8];
  int32_t* row = table + (int64_t)blockIdx.x * chunks;
  int carry = 0;
  for (int c0 = 0; c0 < chunks; c0 += 256) {
    const int c = c0 + threadIdx.x;
    const int v = c < chunks ? row[c] : 0;
    int total;
    const int pre = block_exclusive_scan_256(v, lds, &total);
    if (c < chunks) row[c] = carry + pre;
    carry += total;
  }
  if (threadIdx.x == 0) totals[blockIdx.x] = carry;
}

// One workgroup: first destination row of every expert, and the per-expert counts in the caller's integer type.
__global__ __launch_bounds__(256) void moe_scan_experts_kernel(const int32_t* __restrict__ totals, int num_experts,
                                                               int32_t* __restrict__ expert_start,
                                                               void* __restrict__ counts_out, int counts_i64) {
  __shared__ int lds[8];
  int carry = 0;
  for (int e0 = 0; e0 < num_experts; e0 += 256) {
    const int e = e0 + threadIdx.x;
    const int v = e < num_experts ? totals[e] : 0;
    int total;
    const int pre = block_exclusive_scan_256(v, lds, &total);
    if (e < num_experts) {
      expert_start[e] = carry + pre;
      if (counts_out) {
        if (counts_i64) ((int64_t*)counts_out)[e] = v; else ((int32_t*)counts_out)[e] = v;
      }
    }
    carry += total;
  }
}

__global__ __launch_bounds__(256) void moe_place_kernel(const int32_t* __restrict__ indices, int64_t n, int64_t tokens,
                                                        int topk, int num_experts, int chunks, int64_t capacity,
                                                        const int32_t* __restrict__ table,
                                                        const int32_t* __restrict__ expert_start,
                                                        const int32_t* __restrict__ rank,
                                                        int32_t* __restrict__ row_id_map) {
  const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (i >= n) return;
  const int e = indices[i];
  int dest = -1;
  if (e >= 0 && e < num_experts) {
    const int64_t d = (int64_t)expert_start[e] + table[(int64_t)e * chunks + (int)(i / kChunk)] + rank[i];
    if (d < capacity) dest = (int)d;
  }
  const int64_t t = i / topk;
  const int k = (int)(i - t * topk);
  row_id_map[(int64_t)k * tokens + t] = dest;
}

// One workgroup per token: the row is read once (16 bytes per lane and step) and stored to every destination.
__global__ __launch_bounds__(256) void moe_permute_rows_kernel(const i32x4_t* __restrict__ in, i32x4_t* __restrict__ out,
                                                               const int32_t* __restrict__ row_id_map,
                                                               int64_t tokens, int topk, int chunks16) {
  const int64_t t = blockIdx.x;
  const i32x4_t* src = in + t * chunks16;
  for (int c = threadIdx.x; c < chunks16; c += 256) {
    const i32x4_t v = src[c];
    for (int k = 0; k < topk; ++k) {
      const int dest = row_id_map[(int64_t)k * tokens + t];  // wave-uniform
      if (dest >= 0) out[(int64_t)dest * chunks16 + c] = v;
    }
  }
}

template <int DT> struct Elem;  // 16 bytes <-> fp32 values
template <> struct Elem<DT_BF16> {
  static constexpr int N = 8;
  static TGG_DEV void load(const void* p, float (&f)[8]) {
    const i32x4_t v = *(const i32x4_t*)p;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      f[2 * j] = __builtin_bit_cast(float, (uint32_t)v[j] << 16);
      f[2 * j + 1] = __builtin_bit_cast(float, (uint32_t)v[j] & 0xffff0000u);
    }
  }
  static TGG_DEV void store(void* p, const float (&f)[8]) {
    const uint2 a = pack4<DT_BF16>(f[0], f[1], f[2], f[3]), b = pack4<DT_BF16>(f[4], f[5], f[6], f[7]);
    i32x4_t v = {(int)a.x, (int)a.y, (int)b.x, (int)b.y};
    *(i32x4_t*)p = v;
  }
};
template <> struct Elem<DT_F16> {
  static constexpr int N = 8;
  static TGG_DEV void load(const void* p, float (&f)[8]) {
    const f16x8_t v = *(const f16x8_t*)p;
#pragma unroll
    for (int j = 0; j < 8; ++j) f[j] = (float)v[j];
  }
  static TGG_DEV void store(void* p, const float (&f)[8]) {
    const uint2 a = pack4<DT_F16>(f[0], f[1], f[2], f[3]), b = pack4<DT_F16>(f[4], f[5], f[6], f[7]);
    i32x4_t v = {(int)a.x, (int)a.y, (int)b.x, (int)b.y};
    *(i32x4_t*)p = v;
  }
};
constexpr int DT_F32 = 4;  // only the permute kernels know fp32 activations
template <> struct Elem<DT_F32> {
  static constexpr int N = 4;
  static TGG_DEV void load(const void* p, float (&f)[4]) {
    const f32x4_t v = *(const f32x4_t*)p;
#pragma unroll
    for (int j = 0; j < 4; ++j) f[j] = v[j];
  }
  static TGG_DEV void store(void* p, const float (&f)[4]) {
    f32x4_t v = {f[0], f[1], f[2], f[3]};
    *(f32x4_t*)p = v;
  }
};

// out[t, :] = sum_k prob[t, k] * in[row_id_map[k * tokens + t], :]   (prob == nullptr: plain sum)
template <int DT>
__global__ __launch_bounds__(256) void moe_unpermute_kernel(const char* __restrict__ in, char* __restrict__ out,
                                                            const int32_t* __restrict__ row_id_map,
                                                            const float* __restrict__ prob, int64_t tokens, int topk,
                                                            int chunks16) {
  constexpr int N = Elem<DT>::N;
  const int64_t t = blockIdx.x;
  for (int c = threadIdx.x; c < chunks16; c += 256) {
    float acc[N];
#pragma unroll
    for (int j = 0; j < N; ++j) acc[j] = 0.f;
    for (int k = 0; k < topk; ++k) {
      const int src = row_id_map[(int64_t)k * tokens + t];
      if (src < 0) continue;
      const float w = prob ? prob[t * topk + k] : 1.f;
      float f[N];
      Elem<DT>::load(in + ((int64_t)src * chunks16 + c) * 16, f);
#pragma unroll
      for (int j = 0; j < N; ++j) acc[j] += w * f[j];
    }
    Elem<DT>::store(out + (t * chunks16 + c) * 16, acc);
  }
}

// act_grad[dest, :] = prob[t, k] * grad[t, :];  prob_grad[t, k] = sum_h grad[t, h] * fwd_in[dest, h]
template <int DT>
__global__ __launch_bounds__(256) void moe_unpermute_bwd_kernel(const char* __restrict__ grad, const char* __restrict__ fwd_in,
                                                                const int32_t* __restrict__ row_id_map,
                                                                const float* __restrict__ prob, char* __restrict__ act_grad,
                                                                float* __restrict__ prob_grad, int64_t tokens, int topk,
                                                                int chunks16) {
  constexpr int N = Elem<DT>::N;
  __shared__ float partial[4];
  const int64_t t = blockIdx.x;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  for (int k = 0; k < topk; ++k) {
    const int dest = row_id_map[(int64_t)k * tokens + t];
    const float w = prob ? prob[t * topk + k] : 1.f;
    float dot = 0.f;
    if (dest >= 0) {
      for (int c = threadIdx.x; c < chunks16; c += 256) {
        float g[N], s[N];
        Elem<DT>::load(grad + (t * chunks16 + c) * 16, g);
#pragma unroll
        for (int j = 0; j < N; ++j) s[j] = w * g[j];
        Elem<DT>::store(act_grad + ((int64_t)dest * chunks16 + c) * 16, s);
        if (prob_grad) {
          float x[N];
          Elem<DT>::load(fwd_in + ((int64_t)dest * chunks16 + c) * 16, x);
#pragma unroll
          for (int j = 0; j < N; ++j) dot += g[j] * x[j];
        }
      }
    }
    if (prob_grad) {
#pragma unroll
      for (int d = 32; d > 0; d >>= 1) dot += __shfl_xor(dot, d, 64);
      if (lane == 0) partial[wave] = dot;
      __syncthreads();
      if (threadIdx.x == 0) prob_grad[t * topk + k] = partial[0] + partial[1] + partial[2] + partial[3];
      __syncthreads();
    }
  }
}

size_t align256(size_t x) { return (x + 255) & ~(size_t)255; }

struct SortWorkspace {
  int32_t *table, *totals, *expert_start, *rank;
  size_t bytes;
};

SortWorkspace carve(void* base, int64_t n, int num_experts) {
  const int64_t chunks = (n + kChunk - 1) / kChunk;
  SortWorkspace w;
  size_t off = 0;
  char* b = (char*)base;
  w.table = (int32_t*)(b + off); off += align256((size_t)num_experts * (size_t)(chunks > 0 ? chunks : 1) * 4);
  w.totals = (int32_t*)(b + off); off += align256((size_t)num_experts * 4);
  w.expert_start = (int32_t*)(b + off); off += align256((size_t)num_experts * 4);
  w.rank = (int32_t*)(b + off); off += align256((size_t)(n > 0 ? n : 1) * 4);
  w.bytes = off;
  return w;
}

}  // namespace

int64_t moe_sort_workspace_bytes(int64_t n, int num_experts) { return (int64_t)carve(nullptr, n, num_experts).bytes; }

int launch_moe_permute_map(const int32_t* indices, int64_t tokens, int topk, int num_experts, int64_t capacity,
                           int32_t* row_id_map, void* counts, int counts_i64, void* workspace, hipStream_t s) {
  const int64_t n = tokens * topk;
  const int chunks = (int)((n + kChunk - 1) / kChunk);
  const SortWorkspace w = carve(workspace, n, num_experts);
  if (n == 0) {  // no assignments: every expert is empty
    hipLaunchKernelGGL(moe_scan_rows_kernel, dim3(num_experts), dim3(256), 0, s, w.table, 0, w.totals);
    hipLaunchKernelGGL(moe_scan_experts_kernel, dim3(1), dim3(256), 0, s, w.totals, num_experts, w.expert_start, counts, counts_i64);
    return check_launch("moe_permute_map");
  }
  static bool attr_set[64] = {false};
  int dev = 0;
  (void)hipGetDevice(&dev);
  if (dev >= 0 && dev < 64 && !attr_set[dev]) {
    if (hipFuncSetAttribute((const void*)moe_count_kernel, hipFuncAttributeMaxDynamicSharedMemorySize,
                            16 * kMaxExperts * (int)sizeof(int32_t)) != hipSuccess)
      return check_launch("hipFuncSetAttribute(moe_count)");
    attr_set[dev] = true;
  }
  hipLaunchKernelGGL(moe_count_kernel, dim3(chunks), dim3(kChunk), 16 * num_experts * sizeof(int32_t), s, indices, n,
                     num_experts, chunks, w.table, w.rank);
  hipLaunchKernelGGL(moe_scan_rows_kernel, dim3(num_experts), dim3(256), 0, s, w.table, chunks, w.totals);
  hipLaunchKernelGGL(moe_scan_experts_kernel, dim3(1), dim3(256), 0, s, w.totals, num_experts, w.expert_start, counts, counts_i64);
  hipLaunchKernelGGL(moe_place_kernel, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, s, indices, n, tokens, topk,
                     num_experts, chunks, capacity, w.table, w.expert_start, w.rank, row_id_map);
  return check_launch("moe_permute_map");
}

// ---- the sort without a caller-provided workspace ---------------------------------------------------------------
// For callers that cannot allocate (HIP graph capture, serving loops): the sort's temporaries live in a fixed
// array in device memory that is part of the library's code object.  Sized for the largest problem the entry point
// accepts: 2^20 assignments, 1024 experts (table 4 MiB + rank 4 MiB + two 4 KiB expert rows).  Every GPU the
// library runs on holds its own copy at its own address until the process ends; all calls on one GPU share it, so
// calls that overlap on one GPU (different streams) race.  Nothing in it has to start at zero: the counting pass
// writes every table entry and rank it later reads, the scans write totals and starts.
constexpr int64_t kStaticMaxAssignments = 1ll << 20;
constexpr size_t kStaticScratchBytes = (size_t)kMaxExperts * (kStaticMaxAssignments / kChunk) * 4 + 2 * (size_t)kMaxExperts * 4 +
                                       (size_t)kStaticMaxAssignments * 4;
static __device__ __align__(256) unsigned char scratch[kStaticScratchBytes];

// Device address of this GPU's copy of `scratch`, looked up once per device (the array's name is only a host-side
// handle for hipGetSymbolAddress; it is never passed to a kernel or a memory call).
static int static_scratch_ptr(void** out) {
  static std::mutex mu;
  static void* ptr[64] = {nullptr};
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess) return check_launch("hipGetDevice");
  if (dev < 0 || dev >= 64) return set_error("device ordinal %d outside [0, 64)", dev);
  std::lock_guard<std::mutex> lock(mu);
  if (!ptr[dev]) {
    void* p = nullptr;
    const hipError_t e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
    if (e != hipSuccess || !p) {
      (void)hipGetLastError();
      return set_error("hipGetSymbolAddress(scratch) failed on device %d: %s", dev, hipGetErrorString(e));
    }
    ptr[dev] = p;
  }
  *out = ptr[dev];
  return 0;
}

int64_t moe_static_max_assignments() { return kStaticMaxAssignments; }

int launch_moe_permute_map_static(const int32_t* indices, int64_t tokens, int topk, int num_experts, int64_t capacity,
                                  int32_t* row_id_map, void* counts, int counts_i64, hipStream_t s) {
  const int64_t n = tokens * topk;
  if (n > kStaticMaxAssignments)
    return set_error("num_tokens * topk = %lld exceeds the %lld assignments the built-in scratch array holds; "
                     "use tgg_moe_permute_map with a workspace", (long long)n, (long long)kStaticMaxAssignments);
  if (carve(nullptr, n, num_experts).bytes > kStaticScratchBytes)
    return set_error("sort temporaries of %zu bytes exceed the built-in scratch array (%zu bytes)",
                     carve(nullptr, n, num_experts).bytes, kStaticScratchBytes);
  void* ws = nullptr;
  if (int e = static_scratch_ptr(&ws)) return e;
  return launch_moe_permute_map(indices, tokens, topk, num_experts, capacity, row_id_map, counts, counts_i64, ws, s);
}

int launch_moe_permute_rows(const void* in, void* out, const int32_t* row_id_map, int64_t tokens, int topk,
                            int64_t row_bytes, hipStream_t s) {
  if (tokens == 0) return 0;
  hipLaunchKernelGGL(moe_permute_rows_kernel, dim3((unsigned)tokens), dim3(256), 0, s, (const i32x4_t*)in, (i32x4_t*)out,
                     row_id_map, tokens, topk, (int)(row_bytes / 16));
  return check_launch("moe_permute_rows");
}

int launch_moe_unpermute(const void* in, void* out, const int32_t* row_id_map, const float* prob, int64_t tokens,
                         int topk, int64_t row_bytes, int dt, hipStream_t s) {
  if (tokens == 0) return 0;
  const int c16 = (int)(row_bytes / 16);
  const dim3 grid((unsigned)tokens), block(256);
  if (dt == DT_BF16) hipLaunchKernelGGL(moe_unpermute_kernel<DT_BF16>, grid, block, 0, s, (const char*)in, (char*)out, row_id_map, prob, tokens, topk, c16);
  else if (dt == DT_F16) hipLaunchKernelGGL(moe_unpermute_kernel<DT_F16>, grid, block, 0, s, (const char*)in, (char*)out, row_id_map, prob, tokens, topk, c16);
  else hipLaunchKernelGGL(moe_unpermute_kernel<DT_F32>, grid, block, 0, s, (const char*)in, (char*)out, row_id_map, prob, tokens, topk, c16);
  return check_launch("moe_unpermute");
}

int launch_moe_unpermute_bwd(const void* grad, const void* fwd_in, const int32_t* row_id_map, const float* prob,
                             void* act_grad, float* prob_grad, int64_t tokens, int topk, int64_t row_bytes, int dt,
                             hipStream_t s) {
  if (tokens == 0) return 0;
  const int c16 = (int)(row_bytes / 16);
  const dim3 grid((unsigned)tokens), block(256);
  if (dt == DT_BF16) hipLaunchKernelGGL(moe_unpermute_bwd_kernel<DT_BF16>, grid, block, 0, s, (const char*)grad, (const char*)fwd_in, row_id_map, prob, (char*)act_grad, prob_grad, tokens, topk, c16);
  else if (dt == DT_F16) hipLaunchKernelGGL(moe_unpermute_bwd_kernel<DT_F16>, grid, block, 0, s, (const char*)grad, (const char*)fwd_in, row_id_map, prob, (char*)act_grad, prob_grad, tokens, topk, c16);
  else hipLaunchKernelGGL(moe_unpermute_bwd_kernel<DT_F32>, grid, block, 0, s, (const char*)grad, (const char*)fwd_in, row_id_map, prob, (char*)act_grad, prob_grad, tokens, topk, c16);
  return check_launch("moe_unpermute_bwd");
}

}  // namespace tgg
