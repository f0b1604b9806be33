// Shared scaffolding of the fused step kernels: tensor descriptors, the master-weight read/write and
// requantisation helpers, the two grid shapes (single tensor by value / chunk table over many tensors) and
// the host-side launch + dispatch templates.
//
// Work decomposition.  A wavefront processes sub-tiles of 64 x EPL consecutive elements (EPL = 8 for bf16/fp16,
// 4 for fp32; see fo_device.h for the access shape); a workgroup of FO_BLOCK_THREADS threads covers
// FO_BLOCK_THREADS/64 x FO_SUBTILES_PER_WAVE neighbouring sub-tiles (its "span") and retires.  Workgroups are
// deliberately tiny and short-lived: streaming from HBM is measurably better with many one-wavefront workgroups
// that each touch every stream once than with larger or persistent ones.  The multi-tensor grid addresses work
// through a chunk table in units of 4096-element tiles; a tile is an integer number of spans.  A quantisation
// group is 32/EPL neighbouring lanes, so the group absmax is in-register maxes plus two or three DPP moves.
// LDS only holds the table that turns a first-moment code byte into its dequantised value.
//
// "ref:" cites /root/reference/flashoptim/optimizers.py.
#pragma once

#include "fo_device.h"
#include "fo_host.h"
#include "../../include/flashoptim_hip.h"

#ifndef FO_BLOCK_THREADS
#define FO_BLOCK_THREADS 64
#endif
#ifndef FO_SUBTILES_PER_WAVE
#define FO_SUBTILES_PER_WAVE 1
#endif
#ifndef FO_LUT_REPL
#define FO_LUT_REPL 1
#endif

namespace fo {

constexpr int kBlockThreads = FO_BLOCK_THREADS;
constexpr int kBlockWaves = kBlockThreads / 64;
constexpr int kPerWave = FO_SUBTILES_PER_WAVE;
using StepLut = Lut<FO_LUT_REPL, kBlockThreads>;

struct TensorPtrs {
    void* param;
    const void* grad;
    void* ecc;
    void* mom;
    uint16_t* mom_scales;
    void* var;
    uint16_t* var_scales;
    int64_t n;
};

__device__ __forceinline__ TensorPtrs load_desc(const fo_tensor_desc* d) {
    TensorPtrs t;
    t.param = d->param; t.grad = d->grad; t.ecc = d->ecc; t.mom = d->mom;
    t.mom_scales = static_cast<uint16_t*>(d->mom_scales);
    t.var = d->var; t.var_scales = static_cast<uint16_t*>(d->var_scales); t.n = d->n;
    return t;
}

// Vector accesses need every streamed pointer 16-byte aligned (tiles start at multiples of 4096 elements).
__device__ __forceinline__ bool all_aligned16(const TensorPtrs& t) {
    const uintptr_t bits = (uintptr_t)t.param | (uintptr_t)t.grad | (uintptr_t)t.ecc | (uintptr_t)t.mom | (uintptr_t)t.var;
    return (bits & 15u) == 0;
}

// ------------------------------------------------------------------------------------------------
// shared pieces of the step kernels
// ------------------------------------------------------------------------------------------------

// Reads the lane's parameter values as fp32 masters (ref:2299-2309).
template <int DT, int ECCB, int EPL>
__device__ __forceinline__ void read_master(float (&p)[EPL], const Pack<DTypeInfo<DT>::bytes, EPL>& praw,
                                            const Pack<ECCB, EPL>& eraw) {
#pragma unroll
    for (int k = 0; k < EPL; ++k) {
        const float w = widen<DT, EPL>(praw, k);
        if constexpr (ECCB > 0) p[k] = ecc_join<DT, ECCB>(w, ecc_to_float<ECCB, EPL>(eraw, k));
        else p[k] = w;
    }
}

// Narrows the updated masters and derives the new ECC (ref:2377-2387).
template <int DT, int ECCB, int EPL>
__device__ __forceinline__ void write_master(const float (&p)[EPL], Pack<DTypeInfo<DT>::bytes, EPL>& pout,
                                             Pack<ECCB, EPL>& eout) {
    u32 eb[EPL];
#pragma unroll
    for (int k = 0; k < EPL; k += 2) {
        float wa, wb;
        narrow_pair<DT, EPL>(pout, k, p[k], p[k + 1], wa, wb);
        if constexpr (ECCB > 0) {
            eb[k] = ecc_split_bits<DT, ECCB, false>(p[k], wa);
            eb[k + 1] = ecc_split_bits<DT, ECCB, false>(p[k + 1], wb);
        }
    }
    if constexpr (ECCB > 0) pack_codes<ECCB, EPL>(eb, eout);
}

// Quantises the lane's first-moment values against the group absmax `am` (shared by the group's lanes,
// clamped at 1e-12): code = rne(127 * 2x/(1+|x|)), x = m/am  ==  rne(254 * m / (am + |m|))
// (ref:2407-2418 with the two divisions merged algebraically; one hardware reciprocal per element).
template <int EPL>
__device__ __forceinline__ void quantize_mom(const float (&m)[EPL], float am, Pack<1, EPL>& out) {
    u32 b[EPL];
#pragma unroll
    for (int k = 0; k < EPL; ++k) {
        const float t = m[k] * __builtin_amdgcn_rcpf(am + fabsf(m[k]));
        b[k] = as_u32(fmaf(t, 254.0f, kMagic));
    }
    pack_codes<1, EPL>(b, out);
}

// Quantises sqrt(v): code = rne(255 * r / av) with 255/av formed once per lane from the hardware reciprocal
// (ref:2408-2419; av >= 1e-12, so the reciprocal is a normal number).
template <int EPL>
__device__ __forceinline__ void quantize_var(const float (&r)[EPL], float av, Pack<1, EPL>& out) {
    const float scale = 255.0f * __builtin_amdgcn_rcpf(av);
    u32 b[EPL];
#pragma unroll
    for (int k = 0; k < EPL; ++k) b[k] = as_u32(fmaf(r[k], scale, kMagic));
    pack_codes<1, EPL>(b, out);
}

template <int DT, int EPL>
__device__ __forceinline__ void narrow_all(const float (&x)[EPL], Pack<DTypeInfo<DT>::bytes, EPL>& out) {
#pragma unroll
    for (int k = 0; k < EPL; k += 2) {
        float wa, wb;
        narrow_pair<DT, EPL>(out, k, x[k], x[k + 1], wa, wb);
    }
}

// ------------------------------------------------------------------------------------------------
// kernels
// ------------------------------------------------------------------------------------------------

// Elements one workgroup covers.
template <class Op> struct Span {
    static constexpr int kSub = 64 * Op::kEpl;                       // elements per sub-tile
    static constexpr int kElems = kBlockWaves * kPerWave * kSub;     // elements per workgroup
    static constexpr int kPerTile = kTileElems / kElems;             // workgroups per 4096-element tile
    static_assert(kElems <= kTileElems && kTileElems % kElems == 0, "a tile must be a whole number of workgroup spans");
};

// Order of the spans.  The hardware deals workgroups round-robin to the 8 XCDs (workgroup b runs on XCD b % 8),
// each with its own L2, so with the identity order used here the 8 XCDs sweep the tensor together, 1 KiB of
// parameters each.  A 128-byte line of fp16 group scales (2048 elements) is then read through four L2s:
// rocprofv3's FETCH_SIZE shows the scale reads four times over (+0.375 B per element).  Giving each XCD runs of
// four consecutive spans removes that over-fetch exactly but streams 5 % slower (4 KiB per XCD instead of
// 1 KiB), so the identity order stays.

// One span starting at element `base` of tensor t.  All loads are issued first, `between()` runs while they are
// in flight (the workgroup commits the LDS table there), then the sub-tiles are finished one after the other.
template <class Op, class Between>
__device__ __forceinline__ void run_span(const TensorPtrs& t, int64_t base, bool aligned, const typename Op::Hyper& h,
                                         const float* lut_lane, Between&& between) {
    constexpr int kSub = Span<Op>::kSub;
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    // wavefront w takes sub-tiles w, w + W, ... of the span
    const int64_t first0 = base + (int64_t)wave * kSub + lane * Op::kEpl;
    constexpr int64_t kStride = (int64_t)kBlockWaves * kSub;
    typename Op::Raw raw[kPerWave];
    // workgroup-uniform choice of the access mode
    if (aligned) {
        if (base + Span<Op>::kElems <= t.n) {
#pragma unroll
            for (int i = 0; i < kPerWave; ++i) Op::template load<kVector>(t, first0 + i * kStride, raw[i]);
            between();
#pragma unroll
            for (int i = 0; i < kPerWave; ++i) Op::template finish<kVector>(t, first0 + i * kStride, raw[i], h, lut_lane);
        } else {
#pragma unroll
            for (int i = 0; i < kPerWave; ++i) Op::template load<kLane>(t, first0 + i * kStride, raw[i]);
            between();
#pragma unroll
            for (int i = 0; i < kPerWave; ++i) Op::template finish<kLane>(t, first0 + i * kStride, raw[i], h, lut_lane);
        }
    } else {
        between();
#pragma unroll 1
        for (int i = 0; i < kPerWave; ++i) {
            Op::template load<kGuarded>(t, first0 + i * kStride, raw[0]);
            Op::template finish<kGuarded>(t, first0 + i * kStride, raw[0], h, lut_lane);
        }
    }
}

// Commits the first-moment table to LDS once per workgroup, at the first call.
template <bool NEEDED> struct LutCommit {
    float* lut; StepLut::Frag frag; bool done;
    __device__ __forceinline__ void operator()() {
        if constexpr (NEEDED) {
            if (!done) { StepLut::commit(lut, frag); done = true; }
        }
    }
};

template <class Op>
__global__ __launch_bounds__(kBlockThreads) void step_single_kernel(TensorPtrs t, typename Op::Hyper h) {
    __shared__ __align__(16) float lut[Op::kNeedsLut ? StepLut::kFloats : 4];
    const int64_t base = (int64_t)blockIdx.x * Span<Op>::kElems;
    LutCommit<Op::kNeedsLut> commit{lut, {}, false};
    if constexpr (Op::kNeedsLut) commit.frag = StepLut::fetch();
    run_span<Op>(t, base, all_aligned16(t), h, StepLut::lane_base(lut), commit);
}

// Workgroup b works on chunk b / kPerTile and takes span b % kPerTile of each of the chunk's tiles.
template <class Op>
__global__ __launch_bounds__(kBlockThreads) void step_multi_kernel(const fo_tensor_desc* __restrict__ descs,
                                                                   const fo_chunk* __restrict__ chunks, typename Op::Hyper h) {
    __shared__ __align__(16) float lut[Op::kNeedsLut ? StepLut::kFloats : 4];
    constexpr int kPerTile = Span<Op>::kPerTile;
    const unsigned b = blockIdx.x;
    const fo_chunk ck = chunks[b / kPerTile];
    const TensorPtrs t = load_desc(descs + ck.tensor);
    LutCommit<Op::kNeedsLut> commit{lut, {}, false};
    if constexpr (Op::kNeedsLut) commit.frag = StepLut::fetch();
    const float* lut_lane = StepLut::lane_base(lut);
    const bool aligned = all_aligned16(t);
    const int64_t in_tile = (int64_t)(b % kPerTile) * Span<Op>::kElems;
    for (int i = 0; i < ck.n_tiles; ++i) {
        const int64_t base = ((int64_t)ck.first_tile + i) * kTileElems + in_tile;
        if (base < t.n) run_span<Op>(t, base, aligned, h, lut_lane, commit);
    }
}

}  // namespace fo

// ==================================================================================================
// host side: argument checks, launch geometry, (dtype, ecc, quantized) -> template instantiation
// ==================================================================================================
namespace fo_host {

inline int validate_common(const void* param, const void* grad, const void* ecc, int64_t n, int dtype, int ecc_bytes) {
    if (n < 0) return fail(FO_ERR_INVALID_ARGUMENT, "n must be >= 0 (got %lld)", (long long)n);
    if (dtype < FO_F32 || dtype > FO_F16) return fail(FO_ERR_INVALID_ARGUMENT, "unknown dtype %d", dtype);
    if (ecc_bytes < 0 || ecc_bytes > 2) return fail(FO_ERR_INVALID_ARGUMENT, "ecc_bytes must be 0, 1 or 2 (got %d)", ecc_bytes);
    if (dtype == FO_F32 && ecc_bytes != 0) return fail(FO_ERR_UNSUPPORTED, "fp32 parameters carry no ECC");
    if (n == 0) return 0;
    if (!param || !grad) return fail(FO_ERR_INVALID_ARGUMENT, "param and grad must not be NULL");
    if (ecc_bytes && !ecc) return fail(FO_ERR_INVALID_ARGUMENT, "ecc_bytes=%d but ecc is NULL", ecc_bytes);
    const uintptr_t elem = dtype == FO_F32 ? 4 : 2;
    if (((uintptr_t)param | (uintptr_t)grad) & (elem - 1)) return fail(FO_ERR_INVALID_ARGUMENT, "param/grad not aligned to their element size");
    if (ecc_bytes == 2 && ((uintptr_t)ecc & 1)) return fail(FO_ERR_INVALID_ARGUMENT, "int16 ecc pointer is odd");
    return 0;
}

inline int validate_state(const void* state, const void* scales, int quantized, int dtype, const char* name) {
    if (!state) return fail(FO_ERR_INVALID_ARGUMENT, "%s must not be NULL", name);
    if (quantized) {
        if (!scales) return fail(FO_ERR_INVALID_ARGUMENT, "%s scales must not be NULL when quantized", name);
        if ((uintptr_t)scales & 1) return fail(FO_ERR_INVALID_ARGUMENT, "%s scales pointer is odd", name);
    } else {
        const uintptr_t elem = dtype == FO_F32 ? 4 : 2;
        if ((uintptr_t)state & (elem - 1)) return fail(FO_ERR_INVALID_ARGUMENT, "%s not aligned to the parameter element size", name);
    }
    return 0;
}


inline int validate_multi(const fo_tensor_desc* descs, int64_t n_tensors, const fo_chunk* chunks, int64_t n_chunks,
                          int dtype, int ecc_bytes) {
    if (int rc = validate_multi_tables(descs, n_tensors, chunks, n_chunks, dtype)) return rc;
    if (ecc_bytes < 0 || ecc_bytes > 2) return fail(FO_ERR_INVALID_ARGUMENT, "ecc_bytes must be 0, 1 or 2 (got %d)", ecc_bytes);
    if (dtype == FO_F32 && ecc_bytes != 0) return fail(FO_ERR_UNSUPPORTED, "fp32 parameters carry no ECC");
    return 0;
}


// Streaming from HBM degrades when a compute unit keeps too many bytes in flight, and a step wavefront has
// several KiB of loads outstanding.  Each kernel family therefore names the LDS footprint it wants per
// workgroup (Op::kLdsBytes; a compute unit has 160 KiB, so 11008 bytes admit 14 workgroups) and the launch
// requests the difference to the kernel's own table as unused dynamic LDS.  The values sit in the middle of the
// measured plateaus, away from the residencies (13 and 16 for Adam) where throughput drops by 4-5 %.
template <class Op> inline unsigned lds_pad_bytes() {
    const int env = step_lds_pad_bytes();
    if (env >= 0) return (unsigned)env;
    constexpr int kStatic = Op::kNeedsLut ? fo::StepLut::kFloats * 4 : 16;
    return Op::kLdsBytes > kStatic ? Op::kLdsBytes - kStatic : 0;
}

template <class Op>
int launch_single(const fo::TensorPtrs& t, const typename Op::Hyper& h, hipStream_t stream) {
    // one pass over the tensor, one short-lived workgroup per span
    const int64_t grid = (t.n + fo::Span<Op>::kElems - 1) / fo::Span<Op>::kElems;
    if (grid > INT32_MAX) return fail(FO_ERR_INVALID_ARGUMENT, "tensor too large for one launch (%lld elements)", (long long)t.n);
    hipLaunchKernelGGL(fo::step_single_kernel<Op>, dim3((unsigned)grid), dim3(fo::kBlockThreads), lds_pad_bytes<Op>(), stream, t, h);
    return check_hip(hipGetLastError(), "step kernel launch");
}

template <class Op>
int launch_multi(const fo_tensor_desc* descs, const fo_chunk* chunks, int64_t n_chunks, const typename Op::Hyper& h, hipStream_t stream) {
    const int64_t grid = n_chunks * fo::Span<Op>::kPerTile;
    if (grid > INT32_MAX) return fail(FO_ERR_INVALID_ARGUMENT, "chunk table too large for one launch (%lld chunks)", (long long)n_chunks);
    hipLaunchKernelGGL(fo::step_multi_kernel<Op>, dim3((unsigned)grid), dim3(fo::kBlockThreads), lds_pad_bytes<Op>(), stream, descs, chunks, h);
    return check_hip(hipGetLastError(), "multi-tensor step kernel launch");
}

// Expands (dtype, ecc_bytes, quantized) into the template instantiation and calls f.template operator()<Op>().
template <template <int, int, bool> class OpT, class F>
int dispatch(int dtype, int ecc_bytes, int quantized, F&& f) {
#define FO_CASE(DT, EB)                                                     \
    if (dtype == DT && ecc_bytes == EB) {                                   \
        return quantized ? f.template operator()<OpT<DT, EB, true>>()       \
                         : f.template operator()<OpT<DT, EB, false>>();     \
    }
    FO_CASE(fo::DT_F32, 0)
    FO_CASE(fo::DT_BF16, 0) FO_CASE(fo::DT_BF16, 1) FO_CASE(fo::DT_BF16, 2)
    FO_CASE(fo::DT_F16, 0) FO_CASE(fo::DT_F16, 1) FO_CASE(fo::DT_F16, 2)
#undef FO_CASE
    return fail(FO_ERR_UNSUPPORTED, "unsupported dtype/ecc combination (%d, %d)", dtype, ecc_bytes);
}

template <class H> struct SingleLauncher {
    fo::TensorPtrs t; H h; hipStream_t s;
    template <class Op> int operator()() { return launch_single<Op>(t, h, s); }
};
template <class H> struct MultiLauncher {
    const fo_tensor_desc* d; const fo_chunk* c; int64_t nc; H h; hipStream_t s;
    template <class Op> int operator()() { return launch_multi<Op>(d, c, nc, h, s); }
};


}  // namespace fo_host
