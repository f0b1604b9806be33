// Shared scaffolding of the fused step kernels: tensor descriptors, the master-weight read/write and
// requantisation helpers, the two grid shapes (single tensor by value / chunk table over many tensors) and
// the host-side launch + dispatch templates.
//
// Work decomposition.  The unit of scheduling is a tile of 4096 consecutive elements of one tensor; a block
// (FO_BLOCK_THREADS threads) walks the tiles of its chunk, each wavefront taking sub-tiles of 64 x EPL
// elements (EPL = 8 for bf16/fp16, 4 for fp32; see fo_device.h for the access shape).  A quantisation group is
// 32/EPL neighbouring lanes, so the group absmax is in-register maxes plus two or three DPP moves.  LDS only
// holds the table that turns a first-moment code byte into its dequantised value.
//
// "ref:" cites /root/reference/flashoptim/optimizers.py.
#pragma once

#include "fo_device.h"
#include "fo_host.h"
#include "../../include/flashoptim_hip.h"

#ifndef FO_BLOCK_THREADS
#define FO_BLOCK_THREADS 512
#endif
#ifndef FO_LUT_REPL
#define FO_LUT_REPL 1
#endif

namespace fo {

constexpr int kBlockThreads = FO_BLOCK_THREADS;
constexpr int kBlockWaves = kBlockThreads / 64;
using StepLut = Lut<FO_LUT_REPL>;

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

// Quantises sqrt(v): code = rne(255 * r / av) with 255/av formed once per lane (ref:2408-2419).
template <int EPL>
__device__ __forceinline__ void quantize_var(const float (&r)[EPL], float av, Pack<1, EPL>& out) {
    const float scale = div_rn(255.0f, av);
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

// One tile: every wavefront of the block takes sub-tiles wave, wave + W, ... of the tile.
template <class Op>
__device__ __forceinline__ void run_tile(const TensorPtrs& t, int64_t tile, bool aligned, const typename Op::Hyper& h,
                                         const float* lut_lane) {
    constexpr int kSub = 64 * Op::kEpl;              // elements per sub-tile
    constexpr int kSubsPerTile = kTileElems / kSub;  // 8 (EPL 8) or 16 (EPL 4)
    const int64_t tile_base = tile * (int64_t)kTileElems;
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    // block-uniform choice: whole tile in range and every stream 16-byte aligned -> straight-line vector path
    if (aligned && (tile_base + kTileElems <= t.n)) {
        for (int s = wave; s < kSubsPerTile; s += kBlockWaves)
            Op::template lane<true>(t, tile_base + s * kSub + lane * Op::kEpl, h, lut_lane);
    } else {
        for (int s = wave; s < kSubsPerTile; s += kBlockWaves)
            Op::template lane<false>(t, tile_base + s * kSub + lane * Op::kEpl, h, lut_lane);
    }
}

template <class Op>
__global__ __launch_bounds__(kBlockThreads) void step_single_kernel(TensorPtrs t, typename Op::Hyper h, int tiles_per_block) {
    __shared__ float lut[Op::kNeedsLut ? StepLut::kFloats : 1];
    if constexpr (Op::kNeedsLut) StepLut::build(lut);
    const float* lut_lane = StepLut::lane_base(lut);
    const bool aligned = all_aligned16(t);
    const int64_t n_tiles = (t.n + kTileElems - 1) / kTileElems;
    const int64_t t0 = (int64_t)blockIdx.x * tiles_per_block;
    const int64_t t1 = t0 + tiles_per_block < n_tiles ? t0 + tiles_per_block : n_tiles;
    for (int64_t tile = t0; tile < t1; ++tile) run_tile<Op>(t, tile, aligned, h, lut_lane);
}

template <class Op>
__global__ __launch_bounds__(kBlockThreads) void step_multi_kernel(const fo_tensor_desc* __restrict__ descs,
                                                                   const fo_chunk* __restrict__ chunks, int64_t n_chunks,
                                                                   typename Op::Hyper h) {
    __shared__ float lut[Op::kNeedsLut ? StepLut::kFloats : 1];
    if constexpr (Op::kNeedsLut) StepLut::build(lut);
    const float* lut_lane = StepLut::lane_base(lut);
    for (int64_t c = blockIdx.x; c < n_chunks; c += gridDim.x) {
        const fo_chunk ck = chunks[c];
        const TensorPtrs t = load_desc(descs + ck.tensor);
        const bool aligned = all_aligned16(t);
        for (int i = 0; i < ck.n_tiles; ++i) run_tile<Op>(t, (int64_t)ck.first_tile + i, aligned, h, lut_lane);
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
    if (n_tensors < 0 || n_chunks < 0) return fail(FO_ERR_INVALID_ARGUMENT, "negative count");
    if (dtype < FO_F32 || dtype > FO_F16) return fail(FO_ERR_INVALID_ARGUMENT, "unknown dtype %d", dtype);
    if (ecc_bytes < 0 || ecc_bytes > 2) return fail(FO_ERR_INVALID_ARGUMENT, "ecc_bytes must be 0, 1 or 2 (got %d)", ecc_bytes);
    if (dtype == FO_F32 && ecc_bytes != 0) return fail(FO_ERR_UNSUPPORTED, "fp32 parameters carry no ECC");
    if (n_chunks > 0 && (!descs || !chunks)) return fail(FO_ERR_INVALID_ARGUMENT, "descs/chunks must not be NULL");
    return 0;
}


template <class Op>
int launch_single(const fo::TensorPtrs& t, const typename Op::Hyper& h, hipStream_t stream) {
    // One pass over the tensor with many short-lived blocks: the hardware scheduler keeps neighbouring tiles
    // in flight together, which streams from HBM measurably better than a persistent grid-stride loop.
    const int64_t n_tiles = (t.n + fo::kTileElems - 1) / fo::kTileElems;
    const int tpb = tiles_per_block();
    const int64_t grid = (n_tiles + tpb - 1) / tpb;
    if (grid > INT32_MAX) return fail(FO_ERR_INVALID_ARGUMENT, "tensor too large for one launch");
    hipLaunchKernelGGL(fo::step_single_kernel<Op>, dim3((unsigned)grid), dim3(fo::kBlockThreads), 0, stream, t, h, tpb);
    return check_hip(hipGetLastError(), "step kernel launch");
}

template <class Op>
int launch_multi(const fo_tensor_desc* descs, const fo_chunk* chunks, int64_t n_chunks, const typename Op::Hyper& h, hipStream_t stream) {
    const int64_t grid = n_chunks < INT32_MAX ? n_chunks : INT32_MAX;  // one chunk per block; the loop covers the rest
    hipLaunchKernelGGL(fo::step_multi_kernel<Op>, dim3((unsigned)grid), dim3(fo::kBlockThreads), 0, stream, descs, chunks, n_chunks, h);
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
