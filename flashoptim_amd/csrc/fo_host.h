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

// The library's one debug switch: FO_DEBUG_WG_PER_CU=<n> in the environment (1..32, read once) makes every step
// kernel ask for n resident workgroups per compute unit instead of its own measured optimum; 0 when unset.  What
// results is the next count the LDS allocation units can enforce at or above n (fo_step.h: plan_residency; a launch
// can request at most 64 KiB, so nothing below 3), further limited by a kernel's cap of wavefronts per SIMD; the
// residency queries of the diagnostics build report it.
int debug_workgroups_per_cu();

// Shared argument check of the multi-tensor entry points: counts, dtype code and table pointers.
int validate_multi_tables(const void* descs, int64_t n_tensors, const void* chunks, int64_t n_chunks, int dtype);

}  // namespace fo_host
