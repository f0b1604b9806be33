// Library-wide pieces of libflashoptim_hip.so: error text, device queries and the host-side chunk-table builder
// of the multi-tensor launcher; in the diagnostics build (FO_DIAG) also the calibration copy kernel.
#include "fo_device.h"
#include "fo_host.h"
#include "../../include/flashoptim_hip.h"
#ifdef FO_DIAG
#include "../../include/flashoptim_hip_diag.h"
#endif

#include <cstdarg>
#include <cstdio>
#include <cstdlib>

#ifdef FO_DIAG
namespace fo {

constexpr int kCopyThreads = 64;

// Plain copy in the step kernels' geometry (one-wavefront workgroups, one 128-bit non-temporal load and store per
// lane, each workgroup retires after 1 KiB): calibrates byte counters and shows the attainable streaming rate.
// Every workgroup makes `passes` such accesses, `stride_vec` vectors apart (1 for ordinary sizes).
__global__ __launch_bounds__(kCopyThreads) void copy_kernel(u32x4* __restrict__ dst, const u32x4* __restrict__ src, int64_t n_vec,
                                                            int64_t stride_vec, int passes) {
    int64_t i = (int64_t)blockIdx.x * kCopyThreads + threadIdx.x;
    for (int k = 0; k < passes && i < n_vec; ++k, i += stride_vec) {
        Pack<4, 4> v;
        load_vec<4, 4>(v, src, i * 4);
        store_vec<4, 4>(v, dst, i * 4);
    }
}


}  // namespace fo
#endif  // FO_DIAG

namespace fo_host {

static thread_local char g_err[512] = "";

int fail(int code, const char* fmt, ...) {
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(g_err, sizeof(g_err), fmt, ap);
    va_end(ap);
    return code;
}

int check_hip(hipError_t e, const char* what) {
    if (e == hipSuccess) return 0;
    snprintf(g_err, sizeof(g_err), "%s: %s", what, hipGetErrorString(e));
    return (int)e;
}

const char* last_error() { return g_err; }

int debug_workgroups_per_cu() {
    static const int value = [] {
        const char* e = getenv("FO_DEBUG_WG_PER_CU");
        const int v = e ? atoi(e) : 0;
        return (v >= 1 && v <= 32) ? v : 0;
    }();
    return value;
}

int validate_multi_tables(const void* descs, int64_t n_tensors, const void* chunks, int64_t n_chunks, int dtype) {
    if (n_tensors < 0 || n_chunks < 0) return fail(FO_ERR_INVALID_ARGUMENT, "negative count");
    if (dtype < FO_F32 || dtype > FO_F16) return fail(FO_ERR_INVALID_ARGUMENT, "unknown dtype %d", dtype);
    if (n_chunks > 0 && (!descs || !chunks)) return fail(FO_ERR_INVALID_ARGUMENT, "descs/chunks must not be NULL");
    return 0;
}

int compute_units() {
    static thread_local int cached_dev = -1, cached_cus = 0;
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess) return 0;
    if (dev != cached_dev) {
        int cus = 0;
        if (hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess) return 0;
        cached_dev = dev; cached_cus = cus;
    }
    return cached_cus;
}

}  // namespace fo_host

using namespace fo_host;

extern "C" {

int fo_version(void) { return 100; }
const char* fo_last_error(void) { return last_error(); }

int fo_device_compute_units(int device) {
    int cus = 0;
    hipError_t e = hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, device);
    if (e != hipSuccess) { check_hip(e, "hipDeviceGetAttribute"); return FO_ERR_NO_DEVICE; }
    return cus;
}

int64_t fo_count_chunks(const int64_t* numels, int64_t n_tensors, int tiles_per_chunk) {
    if (!numels || n_tensors < 0) return fail(FO_ERR_INVALID_ARGUMENT, "bad tensor length array");
    const int64_t tpc = tiles_per_chunk > 0 ? tiles_per_chunk : 1;
    int64_t total = 0;
    for (int64_t i = 0; i < n_tensors; ++i) {
        if (numels[i] < 0) return fail(FO_ERR_INVALID_ARGUMENT, "tensor %lld has negative length", (long long)i);
        const int64_t tiles = (numels[i] + fo::kTileElems - 1) / fo::kTileElems;
        total += (tiles + tpc - 1) / tpc;
    }
    return total;
}

int64_t fo_build_chunks(const int64_t* numels, int64_t n_tensors, int tiles_per_chunk, fo_chunk* out, int64_t capacity) {
    const int64_t need = fo_count_chunks(numels, n_tensors, tiles_per_chunk);
    if (need < 0) return need;
    if (!out || capacity < need) return fail(FO_ERR_INVALID_ARGUMENT, "chunk buffer too small (%lld < %lld)", (long long)capacity, (long long)need);
    if (n_tensors > INT32_MAX) return fail(FO_ERR_INVALID_ARGUMENT, "too many tensors");
    const int64_t tpc = tiles_per_chunk > 0 ? tiles_per_chunk : 1;
    int64_t c = 0;
    for (int64_t i = 0; i < n_tensors; ++i) {
        const int64_t tiles = (numels[i] + fo::kTileElems - 1) / fo::kTileElems;
        if (tiles > INT32_MAX) return fail(FO_ERR_INVALID_ARGUMENT, "tensor %lld too large", (long long)i);
        for (int64_t t0 = 0; t0 < tiles; t0 += tpc) {
            out[c].tensor = (int32_t)i;
            out[c].first_tile = (int32_t)t0;
            out[c].n_tiles = (int32_t)((tiles - t0) < tpc ? (tiles - t0) : tpc);
            out[c].reserved = 0;
            ++c;
        }
    }
    return c;
}

#ifdef FO_DIAG
int fo_copy_bytes(void* dst, const void* src, int64_t n_bytes, void* stream) {
    if (n_bytes < 0 || (n_bytes & 15)) return fail(FO_ERR_INVALID_ARGUMENT, "n_bytes must be a non-negative multiple of 16");
    if (n_bytes == 0) return 0;
    if (!dst || !src || (((uintptr_t)dst | (uintptr_t)src) & 15)) return fail(FO_ERR_INVALID_ARGUMENT, "copy pointers must be 16-byte aligned");
    const int64_t n_vec = n_bytes / 16;
    const int64_t want = (n_vec + fo::kCopyThreads - 1) / fo::kCopyThreads;
    // one access per workgroup up to 2^31 - 1 workgroups (2 TiB); beyond that every workgroup makes several passes
    const int passes = (int)((want + INT32_MAX - 1) / INT32_MAX);
    const int64_t grid = (want + passes - 1) / passes;
    hipLaunchKernelGGL(fo::copy_kernel, dim3((unsigned)grid), dim3(fo::kCopyThreads), 0, (hipStream_t)stream,
                       (fo::u32x4*)dst, (const fo::u32x4*)src, n_vec, grid * fo::kCopyThreads, passes);
    return check_hip(hipGetLastError(), "copy kernel launch");
}

#endif  // FO_DIAG

}  // extern "C"
