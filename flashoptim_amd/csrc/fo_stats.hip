// Largest magnitude of every tensor of a list in one launch: the statistic behind check_numerics
// (ref: /root/reference/flashoptim/optimizers.py:656-673 computes tensor.abs().max().item() per tensor, one
// device synchronisation each).  Read-only scan; each workgroup folds its chunk into one value per wavefront and
// merges it into out[tensor] with an integer atomic max on the fp32 bit pattern (non-negative floats order like
// unsigned integers; a NaN's pattern is above infinity's, so a NaN anywhere in the tensor comes out as NaN,
// as torch's max does).
#include "fo_device.h"
#include "fo_host.h"
#include "../../include/flashoptim_hip.h"

namespace fo {

constexpr int kStatsThreads = 256;

template <int DT>
__device__ __forceinline__ u32 absmax_of_range(const void* x, int64_t begin, int64_t end, bool aligned) {
    constexpr int EPL = DTypeInfo<DT>::epl;
    constexpr int EB = DTypeInfo<DT>::bytes;
    u32 best = 0;
    constexpr int64_t kStride = (int64_t)kStatsThreads * EPL;
    int64_t first = begin + (int64_t)threadIdx.x * EPL;
    if (aligned) {  // four independent loads in flight per thread while whole strides remain
        for (; first + 3 * kStride + EPL <= end; first += 4 * kStride) {
            Pack<EB, EPL> raw[4];
#pragma unroll
            for (int j = 0; j < 4; ++j) load_vec<EB, EPL>(raw[j], x, first + j * kStride);
#pragma unroll
            for (int j = 0; j < 4; ++j)
#pragma unroll
                for (int k = 0; k < EPL; ++k) best = max(best, as_u32(widen<DT, EPL>(raw[j], k)) & 0x7fffffffu);
        }
    }
    for (; first < end; first += kStride) {
        Pack<EB, EPL> raw;
        if (aligned && first + EPL <= end) load_vec<EB, EPL>(raw, x, first);
        else load_guarded<EB, EPL>(raw, x, first, end);
#pragma unroll
        for (int k = 0; k < EPL; ++k) best = max(best, as_u32(widen<DT, EPL>(raw, k)) & 0x7fffffffu);
    }
    return best;
}

__device__ __forceinline__ void merge_wave_max(u32 best, u32* out) {
#pragma unroll
    for (int off = 32; off >= 1; off >>= 1) best = max(best, (u32)__shfl_xor((int)best, off, 64));
    if ((threadIdx.x & 63) == 0 && best != 0) atomicMax(out, best);
}

template <int DT>
__global__ __launch_bounds__(kStatsThreads) void absmax_multi_kernel(const fo_tensor_desc* __restrict__ descs,
                                                                     const fo_chunk* __restrict__ chunks, float* out) {
    const fo_chunk ck = chunks[blockIdx.x];
    const fo_tensor_desc* d = descs + ck.tensor;
    const void* x = d->param;
    const int64_t n = d->n;
    const int64_t begin = (int64_t)ck.first_tile * kTileElems;
    int64_t end = begin + (int64_t)ck.n_tiles * kTileElems;
    if (end > n) end = n;
    const u32 best = absmax_of_range<DT>(x, begin, end, ((uintptr_t)x & 15u) == 0);
    merge_wave_max(best, reinterpret_cast<u32*>(out) + ck.tensor);
}

}  // namespace fo

using namespace fo_host;

extern "C" int fo_multi_absmax(const fo_tensor_desc* descs, int64_t n_tensors, const fo_chunk* chunks, int64_t n_chunks,
                               int dtype, float* out, void* stream) {
    if (int rc = validate_multi_tables(descs, n_tensors, chunks, n_chunks, dtype)) return rc;
    if (n_chunks == 0) return 0;
    if (!out) return fail(FO_ERR_INVALID_ARGUMENT, "out must not be NULL");
    if (n_chunks > INT32_MAX) return fail(FO_ERR_INVALID_ARGUMENT, "chunk table too large for one launch (%lld chunks)", (long long)n_chunks);
    const dim3 grid((unsigned)n_chunks), block(fo::kStatsThreads);
    hipStream_t s = (hipStream_t)stream;
    switch (dtype) {
        case FO_F32: hipLaunchKernelGGL(fo::absmax_multi_kernel<fo::DT_F32>, grid, block, 0, s, descs, chunks, out); break;
        case FO_BF16: hipLaunchKernelGGL(fo::absmax_multi_kernel<fo::DT_BF16>, grid, block, 0, s, descs, chunks, out); break;
        default: hipLaunchKernelGGL(fo::absmax_multi_kernel<fo::DT_F16>, grid, block, 0, s, descs, chunks, out); break;
    }
    return check_hip(hipGetLastError(), "absmax kernel launch");
}
