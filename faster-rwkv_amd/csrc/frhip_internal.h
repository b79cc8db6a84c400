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

}  // namespace frhip
