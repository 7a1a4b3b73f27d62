// Host-side helpers shared by the launchers: error reporting and device queries.
#pragma once
#include <hip/hip_runtime.h>

namespace tgg {

// Records a message retrievable through tgg_last_error() and returns a non-zero code.
int set_error(const char* fmt, ...);
// hipGetLastError() after a launch; 0 when clean.
int check_launch(const char* what);
// Compute units of the current device (cached per device).
int num_cus();

struct GemmParams;
int launch_generic_16bit(const GemmParams& p, int dt, int layout, hipStream_t s);
int launch_generic_fp8_channel(const GemmParams& p, int ta, int tb, int out_dt, hipStream_t s);
int launch_generic_fp8_block(const GemmParams& p, hipStream_t s);
bool fast_fp8_supported(const GemmParams& p, bool block_scaled);
int launch_fast_fp8_channel(const GemmParams& p, int ta, int tb, int out_dt, hipStream_t s);
int launch_fast_fp8_block(const GemmParams& p, hipStream_t s);


// MoE permute / unpermute (moe_permute.hip)
int64_t moe_sort_workspace_bytes(int64_t n, int num_experts);
int launch_moe_permute_map(const int32_t* indices, int64_t tokens, int topk, int num_experts, int64_t capacity,
                           int32_t* row_id_map, void* counts, int counts_i64, void* workspace, hipStream_t s);
int64_t moe_static_max_assignments();
int launch_moe_permute_map_static(const int32_t* indices, int64_t tokens, int topk, int num_experts, int64_t capacity,
                                  int32_t* row_id_map, void* counts, int counts_i64, hipStream_t s);
int launch_moe_permute_rows(const void* in, void* out, const int32_t* row_id_map, int64_t tokens, int topk,
                            int64_t row_bytes, hipStream_t s);
int launch_moe_unpermute(const void* in, void* out, const int32_t* row_id_map, const float* prob, int64_t tokens,
                         int topk, int64_t row_bytes, int dt, hipStream_t s);
int launch_moe_unpermute_bwd(const void* grad, const void* fwd_in, const int32_t* row_id_map, const float* prob,
                             void* act_grad, float* prob_grad, int64_t tokens, int topk, int64_t row_bytes, int dt,
                             hipStream_t s);

}  // namespace tgg
