// Internals shared by the translation units of libfrhip.so (not part of the ABI).
#pragma once

#include <hip/hip_runtime.h>

#include "../../include/frhip.h"

namespace frhip {

// Records `code` and a message for frhip_error_string(); returns `code`.
int set_error(int code, const char* msg);
// Converts a hipError_t into the ABI's return convention (0 or positive code).
int hip_result(hipError_t e, const char* what);
// hipGetLastError() after a launch.
int check_launch(const char* kernel);
// Workgroups per launch for the row-streaming kernels: compute units of the
// current device times FRHIP_WGS_PER_CU (default 1: with one 512-thread
// workgroup per CU most decode launches are a single register-resident batch per wave).
int decode_grid();
int compute_units();
// Device address of the current device's built-in decode scratch (looked up once per device).
int static_scratch(void** ptr);
// Lets the long-row kernels of the current device use more than 64 KB of dynamic LDS.
int allow_large_lds();
// Rows t = 0 .. T-1 of x ([T][C] binary16) normalised and mixed with the row before them (row -1 is
// `state`): out[i][t] = mix(LN(x[t]), LN(x[t-1]), mix[i]) for i < nmix, xx_last = LN(x[T-1]).  Any C;
// with T = 1 it serves the one-token operators of models wider than their fused kernels take.
int launch_ln_mix(int T, int C, const void* x, const void* state, const void* ln_w, const void* ln_b,
                  const void* const* mix, void* const* out, int nmix, void* xx_last, hipStream_t st);

}  // namespace frhip
