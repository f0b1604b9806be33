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

constexpr int kCodecThreads = 64;   // one wavefront per workgroup, like the step kernels

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

// Value of code byte b before the group scale: q / IN_MAX, then y / (2 - |y|) when the softsign companding is on
// (ref:2591-2597), each operation correctly rounded.  Evaluated by the compiler, one table per flag combination;
// a lookup replaces two IEEE divisions per element.
template <bool SIGNED, bool SOFTSIGN> struct CodeTable {
    float v[256];
    constexpr CodeTable() : v() {
        for (int b = 0; b < 256; ++b) {
            const int q = (SIGNED && b >= 128) ? b - 256 : b;
            const float t = (float)q / (SIGNED ? 127.0f : 255.0f);
            const float a = t < 0.0f ? -t : t;
            v[b] = SOFTSIGN ? t / (2.0f - a) : t;
        }
    }
};
__device__ const CodeTable<false, false> kCodeTableU = CodeTable<false, false>();
__device__ const CodeTable<false, true> kCodeTableUS = CodeTable<false, true>();
__device__ const CodeTable<true, false> kCodeTableS = CodeTable<true, false>();
__device__ const CodeTable<true, true> kCodeTableSS = CodeTable<true, true>();

// ref:2541-2607 _triton_dequantize_kernel
template <bool FAST>
__device__ __forceinline__ void dequantize_load(const void* codes, const uint16_t* scales, int64_t first, int64_t n,
                                                Pack<1, 4>& craw, uint16_t& scale_bits) {
    load_lane<1, 4, FAST>(craw, codes, first, n);
    scale_bits = 0x3c00;                                                    // ref:2577-2582 masked scales read 1.0
    if (FAST || first < n) scale_bits = scales[first >> 5];
}
template <bool FAST>
__device__ __forceinline__ void dequantize_finish(const Pack<1, 4>& craw, uint16_t scale_bits, const float* lut, float* out,
                                                  int64_t first, int64_t n, CodecFlags f) {
    const float scale = f16_bits_to_f32(scale_bits);
    Pack<4, 4> o;
#pragma unroll
    for (int k = 0; k < 4; ++k) {
        float xv = lut[byte_of<4>(craw, k)] * scale;                        // ref:2591-2600
        if (f.do_sqrt) xv = xv * xv;                                        // ref:2603-2604
        o.w[k] = as_u32(xv);
    }
    store_lane<4, 4, FAST>(o, out, first, n);
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

// Work loop shared by the four kernels, in the step kernels' geometry: a workgroup is one wavefront and takes one
// span of 64 x EPL elements (it only iterates for tensors beyond 2^31 - 1 spans); `first` is the lane's first element.
#define FO_SPAN_LOOP(N, EPL_, ALIGNED, CALL_FAST, CALL_SLOW)                                      \
    {                                                                                             \
        constexpr int64_t kSpan_ = 64 * (EPL_);                                                   \
        const int64_t n_spans_ = ((N) + kSpan_ - 1) / kSpan_;                                     \
        for (int64_t span_ = blockIdx.x; span_ < n_spans_; span_ += gridDim.x) {                  \
            const int64_t first = span_ * kSpan_ + (int64_t)threadIdx.x * (EPL_);                 \
            if ((ALIGNED) && (span_ + 1) * kSpan_ <= (N)) { CALL_FAST; } else { CALL_SLOW; }      \
        }                                                                                         \
    }

template <int XDT>
__global__ __launch_bounds__(kCodecThreads) void quantize_kernel(const void* x, void* codes, uint16_t* scales, int64_t n, CodecFlags f) {
    const bool aligned = ((((uintptr_t)x) | ((uintptr_t)codes)) & 15u) == 0;
    FO_SPAN_LOOP(n, DTypeInfo<XDT>::epl, aligned, (quantize_lane<XDT, true>(x, codes, scales, first, n, f)), (quantize_lane<XDT, false>(x, codes, scales, first, n, f)))
}

// A workgroup (one wavefront) takes kDequantSpans neighbouring spans of 256 elements, so that the 1 KiB table it
// copies to LDS serves more than one span (4 spans: 5.6 TB/s, 1 span: 4.7; reading the table through the vector
// cache instead: 3.5); all code loads are issued before the table is committed.  Four of every five bytes are
// written, and write-only streams reach 5.7-6.0 TB/s on this part.
constexpr int kDequantSpans = 4;
__global__ __launch_bounds__(kCodecThreads) void dequantize_kernel(const void* codes, const uint16_t* scales, float* out, int64_t n, CodecFlags f) {
    constexpr int kSpans = kDequantSpans;
    constexpr int64_t kSpan = 64 * 4;
    const bool aligned = ((((uintptr_t)out) | ((uintptr_t)codes)) & 15u) == 0;
    const float* table = f.is_signed ? (f.softsign ? kCodeTableSS.v : kCodeTableS.v) : (f.softsign ? kCodeTableUS.v : kCodeTableU.v);
    __shared__ __align__(16) float lut[256];
    const u32x4 frag = *reinterpret_cast<const u32x4*>(table + 4 * threadIdx.x);
    bool committed = false;
    const int64_t n_blocks = (n + kSpan * kSpans - 1) / (kSpan * kSpans);
    for (int64_t blk = blockIdx.x; blk < n_blocks; blk += gridDim.x) {
        const int64_t base = blk * kSpan * kSpans;
        const bool fast = aligned && base + kSpan * kSpans <= n;
        Pack<1, 4> craw[kSpans];
        uint16_t scale_bits[kSpans];
#pragma unroll
        for (int i = 0; i < kSpans; ++i) {
            const int64_t first = base + i * kSpan + (int64_t)threadIdx.x * 4;
            if (fast) dequantize_load<true>(codes, scales, first, n, craw[i], scale_bits[i]);
            else dequantize_load<false>(codes, scales, first, n, craw[i], scale_bits[i]);
        }
        if (!committed) {
            *reinterpret_cast<u32x4*>(lut + 4 * threadIdx.x) = frag;
            __syncthreads();  // one wavefront: no hardware barrier is needed, the compiler drops it
            committed = true;
        }
#pragma unroll
        for (int i = 0; i < kSpans; ++i) {
            const int64_t first = base + i * kSpan + (int64_t)threadIdx.x * 4;
            if (fast) dequantize_finish<true>(craw[i], scale_bits[i], lut, out, first, n, f);
            else dequantize_finish<false>(craw[i], scale_bits[i], lut, out, first, n, f);
        }
    }
}

template <int DT, int ECCB>
__global__ __launch_bounds__(kCodecThreads) void ecc_join_kernel(const void* narrow, const void* ecc, float* out, int64_t n) {
    const bool aligned = ((((uintptr_t)narrow) | ((uintptr_t)ecc) | ((uintptr_t)out)) & 15u) == 0;
    FO_SPAN_LOOP(n, 4, aligned, (ecc_join_lane<DT, ECCB, true>(narrow, ecc, out, first, n)), (ecc_join_lane<DT, ECCB, false>(narrow, ecc, out, first, n)))
}

template <int DT, int ECCB>
__global__ __launch_bounds__(kCodecThreads) void ecc_split_kernel(const float* x, const void* narrow, void* ecc, int64_t n) {
    const bool aligned = ((((uintptr_t)narrow) | ((uintptr_t)ecc) | ((uintptr_t)x)) & 15u) == 0;
    FO_SPAN_LOOP(n, 4, aligned, (ecc_split_lane<DT, ECCB, true>(x, narrow, ecc, first, n)), (ecc_split_lane<DT, ECCB, false>(x, narrow, ecc, first, n)))
}

}  // namespace fo

namespace {
using namespace fo_host;

// One short-lived workgroup per span of 64 x EPL elements (one pass streams better than a persistent grid here).
unsigned grid_for(int64_t n, int epl) {
    const int64_t spans = (n + 64 * epl - 1) / (64 * epl);
    return (unsigned)(spans < INT32_MAX ? spans : INT32_MAX);
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
    const dim3 grid(grid_for(n, x_dtype == FO_F32 ? 4 : 8)), block(fo::kCodecThreads);
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
    hipLaunchKernelGGL(fo::dequantize_kernel, dim3(grid_for(n, 4 * fo::kDequantSpans)), dim3(fo::kCodecThreads), 0, (hipStream_t)stream, codes,
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
    const dim3 grid(grid_for(n, 4)), block(fo::kCodecThreads);
    hipStream_t s = (hipStream_t)stream;
    FO_ECC_DISPATCH(ecc_join_kernel, narrow, ecc, out, n)
    return check_hip(hipGetLastError(), "ecc join kernel launch");
}

int fo_ecc_split(const float* x, const void* narrow, int narrow_dtype, void* ecc, int ecc_bytes, int64_t n, void* stream) {
    if (int rc = validate_ecc_args(x, narrow, ecc, narrow_dtype, ecc_bytes, n)) return rc;
    if (n == 0) return 0;
    if (((uintptr_t)narrow & 1) || ((uintptr_t)x & 3) || (ecc_bytes == 2 && ((uintptr_t)ecc & 1))) return fail(FO_ERR_INVALID_ARGUMENT, "pointer not aligned to its element size");
    if (compute_units() <= 0) return fail(FO_ERR_NO_DEVICE, "no HIP device");
    const dim3 grid(grid_for(n, 4)), block(fo::kCodecThreads);
    hipStream_t s = (hipStream_t)stream;
    FO_ECC_DISPATCH(ecc_split_kernel, x, narrow, ecc, n)
    return check_hip(hipGetLastError(), "ecc split kernel launch");
}

}  // extern "C"
