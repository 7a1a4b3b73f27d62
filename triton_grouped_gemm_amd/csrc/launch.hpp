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

}  // namespace tgg
