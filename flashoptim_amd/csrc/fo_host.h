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

// Override, from FO_STEP_LDS_PAD in the environment, of the unused dynamic LDS that every step-kernel workgroup
// requests to bound the workgroups resident on a compute unit; -1 when unset (read once; for tuning).
int step_lds_pad_bytes();

// Tiles per work item of the multi-tensor chunk table when the caller passes tiles_per_chunk <= 0.
// FO_TILES_PER_CHUNK in the environment overrides it (read once; for tuning).
int default_tiles_per_chunk();

// Shared argument check of the multi-tensor entry points: counts, dtype code and table pointers.
int validate_multi_tables(const void* descs, int64_t n_tensors, const void* chunks, int64_t n_chunks, int dtype);

}  // namespace fo_host
