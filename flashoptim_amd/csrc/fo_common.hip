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

// Counts, per compute unit, how many workgroups of this kernel are resident at once: every one-wavefront workgroup
// registers on its compute unit's counter (hardware id registers name the unit), lingers for a bounded number of
// clock ticks so that the unit fills up, and signs off.  Launched with a given dynamic LDS size it shows how many
// workgroups that size really admits, independent of what the runtime's occupancy query says.
constexpr int kProbeSlots = 4096;  // 16 XCC ids x 8 shader engine ids x 32 (shader array, compute unit) ids
__global__ __launch_bounds__(64) void residency_probe_kernel(unsigned* __restrict__ now, unsigned* __restrict__ most,
                                                             long long linger_ticks) {
    extern __shared__ unsigned char unused_lds[];
    unsigned hw_id, xcc_id;
    asm volatile("s_getreg_b32 %0, hwreg(HW_REG_HW_ID)" : "=s"(hw_id));
    asm volatile("s_getreg_b32 %0, hwreg(HW_REG_XCC_ID)" : "=s"(xcc_id));
    const unsigned cu = (hw_id >> 8) & 0x1fu, se = (hw_id >> 13) & 0x7u;  // cu_id with the shader array bit; se_id
    const unsigned slot = ((xcc_id & 0xfu) * 8u + se) * 32u + cu;
    if (threadIdx.x == 0) {
        const unsigned mine = atomicAdd(&now[slot], 1u) + 1u;
        atomicMax(&most[slot], mine);
        const long long start = wall_clock64();
        // bounded twice over (clock ticks and iterations): every wavefront leaves
        for (int i = 0; i < 20000 && wall_clock64() - start < linger_ticks; ++i) __builtin_amdgcn_s_sleep(8);
        atomicSub(&now[slot], 1u);
    }
    if (threadIdx.x == 4096) unused_lds[0] = 0;  // never true: keeps the dynamic allocation referenced
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

int fo_probe_residency(int dynamic_lds_bytes, void* counters, int64_t counters_bytes, int* most_resident, void* stream) {
    if (dynamic_lds_bytes < 0 || dynamic_lds_bytes > 65536) return fail(FO_ERR_INVALID_ARGUMENT, "dynamic_lds_bytes must be within 0 .. 65536");
    if (!counters || counters_bytes < (int64_t)(2 * fo::kProbeSlots * sizeof(unsigned)))
        return fail(FO_ERR_INVALID_ARGUMENT, "counters must hold %d bytes of device memory", (int)(2 * fo::kProbeSlots * sizeof(unsigned)));
    if (!most_resident) return fail(FO_ERR_INVALID_ARGUMENT, "most_resident must not be NULL");
    unsigned* now = static_cast<unsigned*>(counters);
    unsigned* most = now + fo::kProbeSlots;
    hipStream_t s = (hipStream_t)stream;
    if (int rc = check_hip(hipMemsetAsync(now, 0, 2 * fo::kProbeSlots * sizeof(unsigned), s), "hipMemsetAsync")) return rc;
    const int cus = compute_units();
    if (cus <= 0) return fail(FO_ERR_NO_DEVICE, "no compute units reported");
    // 64 workgroups per compute unit, each lingering 20 us of the 100 MHz wall clock: the units fill to their limit
    hipLaunchKernelGGL(fo::residency_probe_kernel, dim3((unsigned)cus * 64u), dim3(64), (size_t)dynamic_lds_bytes, s, now, most, 2000LL);
    if (int rc = check_hip(hipGetLastError(), "residency probe launch")) return rc;
    static thread_local unsigned host[fo::kProbeSlots];
    if (int rc = check_hip(hipMemcpyAsync(host, most, sizeof(host), hipMemcpyDeviceToHost, s), "hipMemcpyAsync")) return rc;
    if (int rc = check_hip(hipStreamSynchronize(s), "hipStreamSynchronize")) return rc;
    unsigned best = 0;
    for (unsigned v : host) best = v > best ? v : best;
    *most_resident = (int)best;
    return 0;
}
#endif  // FO_DIAG

}  // extern "C"
