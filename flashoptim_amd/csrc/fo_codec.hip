// Standalone group codec and ECC kernels for gfx950 with their C entry points: the cold-path companions of
// the fused step kernels (state initialisation, uncompressed checkpoints, fp32 export/import of master
// weights).  They share the access shape of the step kernels (fo_device.h) and use correctly rounded division /
// square root, so that their output equals an IEEE
// evaluation of the reference formulas operation by operation.
//
// "ref:" cites /root/reference/flashoptim/optimizers.py.
#include "fo_device.h"
#include "fo_host.h"
#include "../../include/flashoptim_hip.h"

namespace fo {

constexpr int kCodecThreads = 256;

struct CodecFlags {
    int is_signed, do_sqrt, softsign;
};

// ref:2610-2676 _triton_quantize_kernel
template <int XDT, bool FAST>
__device__ __forceinline__ void quantize_lane(const void* x, void* codes, uint16_t* scales, int64_t first, int64_t n, CodecFlags f) {
    constexpr int EPL = DTypeInfo<XDT>::epl;
    Pack<DTypeInfo<XDT>::bytes, EPL> xraw;
    load_lane<DTypeInfo<XDT>::bytes, EPL, FAST>(xraw, x, first, n);
    float v[EPL];
    float am = 0.0f;
#pragma unroll
    for (int k = 0; k < EPL; ++k) {
        float t = widen<XDT, EPL>(xraw, k);
        if (f.do_sqrt) t = sqrt_rn(t);                                      // ref:2650-2651
        v[k] = t;
        am = fmaxf(am, fabsf(t));
    }
    am = fmaxf(group_max<EPL>(am), 1e-12f);                                 // ref:2657-2658
    const float out_max = f.is_signed ? 127.0f : 255.0f;
    u32 q[EPL];
#pragma unroll
    for (int k = 0; k < EPL; ++k) {
        const float nrm = div_rn(v[k], am);                                 // ref:2661
        const float t = f.softsign ? div_rn(2.0f * nrm, 1.0f + fabsf(nrm)) : nrm;   // ref:2664-2667
        q[k] = (u32)(int)floorf(t * out_max + 0.5f);                        // ref:2670-2671
    }
    Pack<1, EPL> out;
    pack_codes<1, EPL>(q, out);
    store_lane<1, EPL, FAST>(out, codes, first, n);
    if ((FAST || first < n) && (threadIdx.x & (32 / EPL - 1)) == 0) store_scale(scales, first >> 5, f32_to_f16_bits(am));   // ref:2675-2676
}

// ref:2541-2607 _triton_dequantize_kernel
template <bool FAST>
__device__ __forceinline__ void dequantize_lane(const void* codes, const uint16_t* scales, float* out, int64_t first, int64_t n, CodecFlags f) {
    constexpr int EPL = 4;
    Pack<1, EPL> craw;
    load_lane<1, EPL, FAST>(craw, codes, first, n);
    float scale = 1.0f;                                                     // ref:2577-2582 masked scales read 1.0
    if (FAST || first < n) scale = f16_bits_to_f32(scales[first >> 5]);
    const float in_max = f.is_signed ? 127.0f : 255.0f;
    Pack<4, EPL> o;
#pragma unroll
    for (int k = 0; k < EPL; ++k) {
        const u32 b = byte_of<EPL>(craw, k);
        const float q = f.is_signed ? (float)(int8_t)b : (float)b;
        const float t = div_rn(q, in_max);                                  // ref:2591
        const float nrm = f.softsign ? div_rn(t, 2.0f - fabsf(t)) : t;      // ref:2594-2597
        float xv = nrm * scale;                                             // ref:2600
        if (f.do_sqrt) xv = xv * xv;                                        // ref:2603-2604
        o.w[k] = as_u32(xv);
    }
    store_lane<4, EPL, FAST>(o, out, first, n);
}

// ref:2779-2803 _reconstruct_fp32_kernel
template <int DT, int ECCB, bool FAST>
__device__ __forceinline__ void ecc_join_lane(const void* narrow, const void* ecc, float* out, int64_t first, int64_t n) {
    constexpr int EPL = 4;
    Pack<DTypeInfo<DT>::bytes, EPL> nraw;
    Pack<ECCB, EPL> eraw;
    load_lane<DTypeInfo<DT>::bytes, EPL, FAST>(nraw, narrow, first, n);
    load_lane<ECCB, EPL, FAST>(eraw, ecc, first, n);
    Pack<4, EPL> o;
#pragma unroll
    for (int k = 0; k < EPL; ++k) o.w[k] = as_u32(ecc_join<DT, ECCB>(widen<DT, EPL>(nraw, k), ecc_to_float<ECCB, EPL>(eraw, k)));
    store_lane<4, EPL, FAST>(o, out, first, n);
}

// ref:2806-2832 _compute_ecc_bits_kernel
template <int DT, int ECCB, bool FAST>
__device__ __forceinline__ void ecc_split_lane(const float* x, const void* narrow, void* ecc, int64_t first, int64_t n) {
    constexpr int EPL = 4;
    Pack<4, EPL> xraw;
    Pack<DTypeInfo<DT>::bytes, EPL> nraw;
    load_lane<4, EPL, FAST>(xraw, x, first, n);
    load_lane<DTypeInfo<DT>::bytes, EPL, FAST>(nraw, narrow, first, n);
    u32 eb[EPL];
#pragma unroll
    for (int k = 0; k < EPL; ++k) eb[k] = ecc_split_bits<DT, ECCB, true>(as_f32(xraw.w[k]), widen<DT, EPL>(nraw, k));
    Pack<ECCB, EPL> eout;
    pack_codes<ECCB, EPL>(eb, eout);
    store_lane<ECCB, EPL, FAST>(eout, ecc, first, n);
}

// Tile loop shared by the four kernels: blocks stride over 4096-element tiles, wavefronts over the tile's
// sub-tiles of 64 x EPL elements; `first` is the lane's first element.
#define FO_TILE_LOOP(N, EPL_, ALIGNED, CALL_FAST, CALL_SLOW)                                      \
    {                                                                                             \
        constexpr int kSub_ = 64 * (EPL_);                                                        \
        const int lane_ = threadIdx.x & 63, wave_ = threadIdx.x >> 6;                             \
        const int64_t n_tiles_ = ((N) + kTileElems - 1) / kTileElems;                             \
        for (int64_t tile_ = blockIdx.x; tile_ < n_tiles_; tile_ += gridDim.x) {                  \
            const int64_t base_ = tile_ * (int64_t)kTileElems;                                    \
            const bool fast_ = (ALIGNED) && base_ + kTileElems <= (N);                            \
            for (int s_ = wave_; s_ < kTileElems / kSub_; s_ += kCodecThreads / 64) {             \
                const int64_t first = base_ + s_ * kSub_ + lane_ * (EPL_);                        \
                if (fast_) { CALL_FAST; } else { CALL_SLOW; }                                     \
            }                                                                                     \
        }                                                                                         \
    }

template <int XDT>
__global__ __launch_bounds__(kCodecThreads) void quantize_kernel(const void* x, void* codes, uint16_t* scales, int64_t n, CodecFlags f) {
    const bool aligned = ((((uintptr_t)x) | ((uintptr_t)codes)) & 15u) == 0;
    FO_TILE_LOOP(n, DTypeInfo<XDT>::epl, aligned, (quantize_lane<XDT, true>(x, codes, scales, first, n, f)), (quantize_lane<XDT, false>(x, codes, scales, first, n, f)))
}

__global__ __launch_bounds__(kCodecThreads) void dequantize_kernel(const void* codes, const uint16_t* scales, float* out, int64_t n, CodecFlags f) {
    const bool aligned = ((((uintptr_t)out) | ((uintptr_t)codes)) & 15u) == 0;
    FO_TILE_LOOP(n, 4, aligned, (dequantize_lane<true>(codes, scales, out, first, n, f)), (dequantize_lane<false>(codes, scales, out, first, n, f)))
}

template <int DT, int ECCB>
__global__ __launch_bounds__(kCodecThreads) void ecc_join_kernel(const void* narrow, const void* ecc, float* out, int64_t n) {
    const bool aligned = ((((uintptr_t)narrow) | ((uintptr_t)ecc) | ((uintptr_t)out)) & 15u) == 0;
    FO_TILE_LOOP(n, 4, aligned, (ecc_join_lane<DT, ECCB, true>(narrow, ecc, out, first, n)), (ecc_join_lane<DT, ECCB, false>(narrow, ecc, out, first, n)))
}

template <int DT, int ECCB>
__global__ __launch_bounds__(kCodecThreads) void ecc_split_kernel(const float* x, const void* narrow, void* ecc, int64_t n) {
    const bool aligned = ((((uintptr_t)narrow) | ((uintptr_t)ecc) | ((uintptr_t)x)) & 15u) == 0;
    FO_TILE_LOOP(n, 4, aligned, (ecc_split_lane<DT, ECCB, true>(x, narrow, ecc, first, n)), (ecc_split_lane<DT, ECCB, false>(x, narrow, ecc, first, n)))
}

}  // namespace fo

namespace {
using namespace fo_host;

// One short-lived workgroup per 4096-element tile (one pass streams better than a persistent grid here); the
// kernels' tile loop only iterates for tensors beyond 2^31 - 1 tiles.
unsigned grid_for(int64_t n) {
    const int64_t tiles = (n + fo::kTileElems - 1) / fo::kTileElems;
    return (unsigned)(tiles < INT32_MAX ? tiles : INT32_MAX);
}

}  // namespace

extern "C" {

int fo_quantize(const void* x, int x_dtype, void* codes, void* scales, int64_t n, int is_signed, int do_sqrt, int softsign,
                void* stream) {
    if (n < 0) return fail(FO_ERR_INVALID_ARGUMENT, "n must be >= 0");
    if (x_dtype < FO_F32 || x_dtype > FO_F16) return fail(FO_ERR_INVALID_ARGUMENT, "unknown dtype %d", x_dtype);
    if (n == 0) return 0;  // ref:2485
    if (!x || !codes || !scales) return fail(FO_ERR_INVALID_ARGUMENT, "x, codes and scales must not be NULL");
    if (((uintptr_t)x & (x_dtype == FO_F32 ? 3 : 1)) || ((uintptr_t)scales & 1)) return fail(FO_ERR_INVALID_ARGUMENT, "x or scales not aligned to their element size");
    if (compute_units() <= 0) return fail(FO_ERR_NO_DEVICE, "no HIP device");
    const fo::CodecFlags f{is_signed ? 1 : 0, do_sqrt ? 1 : 0, softsign ? 1 : 0};
    const dim3 grid(grid_for(n)), block(fo::kCodecThreads);
    hipStream_t s = (hipStream_t)stream;
    switch (x_dtype) {
        case FO_F32: hipLaunchKernelGGL(fo::quantize_kernel<fo::DT_F32>, grid, block, 0, s, x, codes, (uint16_t*)scales, n, f); break;
        case FO_BF16: hipLaunchKernelGGL(fo::quantize_kernel<fo::DT_BF16>, grid, block, 0, s, x, codes, (uint16_t*)scales, n, f); break;
        default: hipLaunchKernelGGL(fo::quantize_kernel<fo::DT_F16>, grid, block, 0, s, x, codes, (uint16_t*)scales, n, f); break;
    }
    return check_hip(hipGetLastError(), "quantize kernel launch");
}

int fo_dequantize(const void* codes, const void* scales, float* out, int64_t n, int is_signed, int do_sqrt, int softsign,
                  void* stream) {
    if (n < 0) return fail(FO_ERR_INVALID_ARGUMENT, "n must be >= 0");
    if (n == 0) return 0;  // ref:2533
    if (!codes || !scales || !out) return fail(FO_ERR_INVALID_ARGUMENT, "codes, scales and out must not be NULL");
    if (((uintptr_t)out & 3) || ((uintptr_t)scales & 1)) return fail(FO_ERR_INVALID_ARGUMENT, "out or scales not aligned to their element size");
    if (compute_units() <= 0) return fail(FO_ERR_NO_DEVICE, "no HIP device");
    const fo::CodecFlags f{is_signed ? 1 : 0, do_sqrt ? 1 : 0, softsign ? 1 : 0};
    hipLaunchKernelGGL(fo::dequantize_kernel, dim3(grid_for(n)), dim3(fo::kCodecThreads), 0, (hipStream_t)stream, codes,
                       (const uint16_t*)scales, out, n, f);
    return check_hip(hipGetLastError(), "dequantize kernel launch");
}

static int validate_ecc_args(const void* a, const void* b, const void* c, int narrow_dtype, int ecc_bytes, int64_t n) {
    if (n < 0) return fail(FO_ERR_INVALID_ARGUMENT, "n must be >= 0");
    if (narrow_dtype != FO_BF16 && narrow_dtype != FO_F16) return fail(FO_ERR_INVALID_ARGUMENT, "narrow dtype must be bf16 or fp16 (got %d)", narrow_dtype);  // ref:2858-2867, 2927-2930
    if (ecc_bytes != 1 && ecc_bytes != 2) return fail(FO_ERR_INVALID_ARGUMENT, "ecc_bytes must be 1 or 2 (got %d)", ecc_bytes);  // ref:2868-2869, 2944-2948
    if (n > 0 && (!a || !b || !c)) return fail(FO_ERR_INVALID_ARGUMENT, "NULL pointer");
    return 0;
}

#define FO_ECC_DISPATCH(KERNEL, ...)                                                                                     \
    if (narrow_dtype == FO_BF16 && ecc_bytes == 1) hipLaunchKernelGGL((fo::KERNEL<fo::DT_BF16, 1>), grid, block, 0, s, __VA_ARGS__); \
    else if (narrow_dtype == FO_BF16) hipLaunchKernelGGL((fo::KERNEL<fo::DT_BF16, 2>), grid, block, 0, s, __VA_ARGS__);  \
    else if (ecc_bytes == 1) hipLaunchKernelGGL((fo::KERNEL<fo::DT_F16, 1>), grid, block, 0, s, __VA_ARGS__);            \
    else hipLaunchKernelGGL((fo::KERNEL<fo::DT_F16, 2>), grid, block, 0, s, __VA_ARGS__);

int fo_ecc_join(const void* narrow, int narrow_dtype, const void* ecc, int ecc_bytes, float* out, int64_t n, void* stream) {
    if (int rc = validate_ecc_args(narrow, ecc, out, narrow_dtype, ecc_bytes, n)) return rc;
    if (n == 0) return 0;
    if (((uintptr_t)narrow & 1) || ((uintptr_t)out & 3) || (ecc_bytes == 2 && ((uintptr_t)ecc & 1))) return fail(FO_ERR_INVALID_ARGUMENT, "pointer not aligned to its element size");
    if (compute_units() <= 0) return fail(FO_ERR_NO_DEVICE, "no HIP device");
    const dim3 grid(grid_for(n)), block(fo::kCodecThreads);
    hipStream_t s = (hipStream_t)stream;
    FO_ECC_DISPATCH(ecc_join_kernel, narrow, ecc, out, n)
    return check_hip(hipGetLastError(), "ecc join kernel launch");
}

int fo_ecc_split(const float* x, const void* narrow, int narrow_dtype, void* ecc, int ecc_bytes, int64_t n, void* stream) {
    if (int rc = validate_ecc_args(x, narrow, ecc, narrow_dtype, ecc_bytes, n)) return rc;
    if (n == 0) return 0;
    if (((uintptr_t)narrow & 1) || ((uintptr_t)x & 3) || (ecc_bytes == 2 && ((uintptr_t)ecc & 1))) return fail(FO_ERR_INVALID_ARGUMENT, "pointer not aligned to its element size");
    if (compute_units() <= 0) return fail(FO_ERR_NO_DEVICE, "no HIP device");
    const dim3 grid(grid_for(n)), block(fo::kCodecThreads);
    hipStream_t s = (hipStream_t)stream;
    FO_ECC_DISPATCH(ecc_split_kernel, x, narrow, ecc, n)
    return check_hip(hipGetLastError(), "ecc split kernel launch");
}

}  // extern "C"
