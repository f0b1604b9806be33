// Host-side helpers shared by the translation units of libflashoptim_hip.so: the thread-local error text,
// HIP error translation and the cached compute-unit count.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

namespace fo_host {

// Stores a printf-formatted message for fo_last_error() and returns `code`.
int fail(int code, const char* fmt, ...) __attribute__((format(printf, 2, 3)));
// 0 for hipSuccess; otherwise records "<what>: <hip error string>" and returns the hipError_t value.
int check_hip(hipError_t e, const char* what);
// Compute units of the calling thread's current device (cached per thread and device), 0 on failure.
int compute_units();
const char* last_error();

constexpr int kBlocksPerCu = 8;           // persistent-grid cap: blocks per compute unit
constexpr int kDefaultTilesPerChunk = 8;  // multi-tensor work item = 8 tiles = 32768 elements

}  // namespace fo_host
