// Shared scaffolding of the fused step kernels: tensor descriptors, the master-weight read/write and
// requantisation helpers, the two grid shapes (single tensor by value / chunk table over many tensors) and
// the host-side launch + dispatch templates.
//
// Work decomposition.  A workgroup is one wavefront; it processes one "span" of 64 x EPL consecutive elements
// (EPL = 8 for bf16/fp16, 4 for fp32; see fo_device.h for the access shape) and retires.  Workgroups are
// deliberately tiny and short-lived: streaming from HBM is measurably better with many one-wavefront workgroups
// that each touch every stream once than with larger or persistent ones.  The multi-tensor grid addresses work
// through a chunk table in units of 4096-element tiles; a tile is an integer number of spans.  A quantisation
// group is 32/EPL neighbouring lanes, so the group absmax is in-register maxes plus two or three DPP moves.
// LDS only holds the 256-entry code tables (moment code -> value, int8 ECC code -> fraction).
//
// "ref:" cites /root/reference/flashoptim/optimizers.py.
#pragma once

#include <mutex>

#include "fo_device.h"
#include "fo_host.h"
#include "../../include/flashoptim_hip.h"

namespace fo {

constexpr int kBlockThreads = 64;  // one wavefront per workgroup

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

// One parameter value as an fp32 master (ref:2299-2309).
// An int8 ECC byte goes through the LDS table of correctly rounded fractions (one lookup instead of a convert and
// two multiply-adds); int16 codes are converted arithmetically.
template <int DT, int ECCB, int EPL>
__device__ __forceinline__ float master_of(const Pack<DTypeInfo<DT>::bytes, EPL>& praw, const Pack<ECCB, EPL>& eraw, int k,
                                           const float* lut) {
    const float w = widen<DT, EPL>(praw, k);
    if constexpr (ECCB == 1) return ecc_join_fraction<DT>(w, lookup_ecc(lut, byte_of<EPL>(eraw, k)));
    else if constexpr (ECCB == 2) return ecc_join<DT, ECCB>(w, ecc_to_float<ECCB, EPL>(eraw, k));
    else return w;
}

// The lane's parameter values as fp32 masters.
template <int DT, int ECCB, int EPL>
__device__ __forceinline__ void read_master(float (&p)[EPL], const Pack<DTypeInfo<DT>::bytes, EPL>& praw,
                                            const Pack<ECCB, EPL>& eraw, const float* lut) {
#pragma unroll
    for (int k = 0; k < EPL; ++k) p[k] = master_of<DT, ECCB, EPL>(praw, eraw, k, lut);
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

// Replaces byte k of the lane's packed codes.
template <int EPL> __device__ __forceinline__ void set_code(Pack<1, EPL>& out, int k, u32 code) {
    const int sh = 8 * (k & 3);
    u32& w = out.w[k >> 2];
    w = (w & ~(0xffu << sh)) | ((code & 0xffu) << sh);
}

// The hardware wavefront as the verified flows of fo_math.h see it from one of its lanes: each() is one call on the
// lane's own state, any() a ballot over the 64 lanes.
template <class Lane> struct HwWave {
    Lane& lane;
    template <class F> __device__ __forceinline__ void each(F&& f) { f(lane); }
    template <class P> __device__ __forceinline__ bool any(P&& p) { return __builtin_amdgcn_ballot_w64(p(lane)) != 0; }
};

// Lane state of requantize_mom_verified / requantize_var_verified for eight values per lane (2-byte parameters):
// the codes are the two dwords that travel to memory; the conversion writes each byte in place (convert_pack8).
struct MomLane8 {
    const float (&m)[8];
    float am;
    Pack<1, 8>& out;
    float x[8], slack[8], least, ram;
    __device__ __forceinline__ void convert_mom(const float (&q)[8]) {
        const float lo[4] = {q[0], q[1], q[2], q[3]}, hi[4] = {q[4], q[5], q[6], q[7]};
        convert_pack8<kFloor, kFloor>(lo, hi, out.w[0], out.w[1]);
    }
    __device__ __forceinline__ void set_mom_code(int k, u32 code) { set_code<8>(out, k, code); }
};
struct VarLane8 {
    const float (&v)[8];
    const float (&r)[8];
    float av_quick, av;
    Pack<1, 8>& out;
    float x[8], slack[8], least, rav;
    __device__ __forceinline__ void convert_var(const float (&q)[8]) {
        const float lo[4] = {q[0], q[1], q[2], q[3]}, hi[4] = {q[4], q[5], q[6], q[7]};
        convert_pack8<kTrunc, kTrunc>(lo, hi, out.w[0], out.w[1]);
    }
    __device__ __forceinline__ void set_var_code(int k, u32 code) { set_code<8>(out, k, code); }
};
// Four values of each moment per lane (fp32 parameters): one dword of codes per state, one conversion block.
struct BothLane4 {
    const float (&m)[4];
    float am;
    const float (&v)[4];
    const float (&r)[4];
    float av_quick, av;
    Pack<1, 4>& mout;
    Pack<1, 4>& vout;
    float xm[4], xv[4], slack_m[4], slack_v[4], least_m, least_v, ram, rav;
    __device__ __forceinline__ void convert_both(const float (&qm)[4], const float (&qv)[4]) {
        convert_pack8<kFloor, kTrunc>(qm, qv, mout.w[0], vout.w[0]);
    }
    __device__ __forceinline__ void set_mom_code(int k, u32 code) { set_code<4>(mout, k, code); }
    __device__ __forceinline__ void set_var_code(int k, u32 code) { set_code<4>(vout, k, code); }
};

// Quantises the lane's first-moment values against the group absmax `am` (shared by the group's lanes, clamped
// at 1e-12); the rounding is the reference's (fo_math.h; ref:2405-2419, 1703-1710).  Through the quick forms,
// every value verified and the failing ones redone with the exact form (fo_math.h: requantize_mom_verified): the
// result is the exact requantiser's, code for code.
template <int EPL>
__device__ __forceinline__ void quantize_mom_quick_verified(const float (&m)[EPL], float am, Pack<1, EPL>& out) {
    static_assert(EPL == 8, "two dwords of codes per lane");
    MomLane8 lane{m, am, out};
    HwWave<MomLane8> wave{lane};
    requantize_mom_verified<8>(wave);
}
// r: hw::sqrt of the lane's second moments v; av_quick / av_exact: hw::sqrt and sqrt_corrected of the group's largest v.
template <int EPL>
__device__ __forceinline__ void quantize_var_quick_verified(const float (&v)[EPL], const float (&r)[EPL], float av_quick,
                                                            float av_exact, Pack<1, EPL>& out) {
    static_assert(EPL == 8, "two dwords of codes per lane");
    VarLane8 lane{v, r, av_quick, av_exact, out};
    HwWave<VarLane8> wave{lane};
    requantize_var_verified<8>(wave);
}
// Four elements per lane (fp32 parameters), both states through the quick forms with verification: one conversion
// block, one repair branch.
__device__ __forceinline__ void quantize_mom_var_quick_verified(const float (&m)[4], float am, const float (&v)[4],
                                                                const float (&r)[4], float av_quick, float av_exact,
                                                                Pack<1, 4>& mout, Pack<1, 4>& vout) {
    BothLane4 lane{m, am, v, r, av_quick, av_exact, mout, vout};
    HwWave<BothLane4> wave{lane};
    requantize_both_verified<4>(wave);
}
// Four elements per lane, one state (momentum kernels on fp32 parameters): plain conversion and byte packing.
__device__ __forceinline__ void quantize_mom(const float (&m)[4], float am, Pack<1, 4>& out) {
    const float ram = hw::rcp(am);
    u32 b[4];
#pragma unroll
    for (int k = 0; k < 4; ++k) b[k] = quantize_mom_code(m[k], am, ram);
    pack_codes<1, 4>(b, out);
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

// Elements one workgroup (= one wavefront) covers: 64 lanes x EPL.
template <class Op> struct Span {
    static constexpr int kElems = 64 * Op::kEpl;
    static constexpr int kPerTile = kTileElems / kElems;             // workgroups per 4096-element tile
    static_assert(kTileElems % kElems == 0, "a tile must be a whole number of workgroup spans");
};

// Order of the spans.  The hardware deals workgroups round-robin to the 8 XCDs (workgroup b runs on XCD b % 8),
// each with its own L2, so with the identity order used here the 8 XCDs sweep the tensor together, 1 KiB of
// parameters each.  A 128-byte line of fp16 group scales (2048 elements) is then read through four L2s:
// rocprofv3's FETCH_SIZE shows the scale reads four times over (+0.375 B per element).  Giving each XCD runs of
// four consecutive spans removes that over-fetch exactly but streams 5 % slower (4 KiB per XCD instead of
// 1 KiB), so the identity order stays.

// One span starting at element `base` of tensor t: all loads are issued first, then the span is finished.
template <class Op>
__device__ __forceinline__ void run_span(const TensorPtrs& t, int64_t base, bool aligned, const typename Op::Hyper& h,
                                         const float* lut) {
    const Where first{base, (int)(threadIdx.x & 63) * Op::kEpl};
    typename Op::Raw raw;
    // workgroup-uniform choice of the access mode
    if (aligned) {
        if (base + Span<Op>::kElems <= t.n) {
            Op::template load<kVector>(t, first, raw);
            Op::template finish<kVector>(t, first, raw, h, lut);
        } else {
            Op::template load<kLane>(t, first, raw);
            Op::template finish<kLane>(t, first, raw, h, lut);
        }
    } else {
        Op::template load<kGuarded>(t, first, raw);
        Op::template finish<kGuarded>(t, first, raw, h, lut);
    }
}

// Op::kMaxWavesPerSimd caps the wavefronts a SIMD holds (8 = the hardware's own limit, i.e. no cap): the code object
// then declares enough registers that no SIMD takes more, and the compute unit's resident workgroups (capped through
// LDS, fo_host::plan_residency) spread evenly over its four SIMDs instead of piling up on some of them.
#define FO_WAVES_ATTR __attribute__((amdgpu_waves_per_eu(1, Op::kMaxWavesPerSimd)))
template <class Op>
__global__ __launch_bounds__(kBlockThreads) FO_WAVES_ATTR void step_single_kernel(TensorPtrs t, typename Op::Hyper h) {
    __shared__ __align__(16) float lut[StepLut<Op::kLutMask>::kFloats];
    const int64_t base = (int64_t)blockIdx.x * Span<Op>::kElems;
    if constexpr (Op::kLutMask != 0) StepLut<Op::kLutMask>::fill(lut, kStepTables<Op::kDtype>.v);
    run_span<Op>(t, base, all_aligned16(t), h, lut);
}

// Workgroup b works on chunk b / kPerTile and takes span b % kPerTile of each of the chunk's tiles.
template <class Op>
__global__ __launch_bounds__(kBlockThreads) FO_WAVES_ATTR void step_multi_kernel(const fo_tensor_desc* __restrict__ descs,
                                                                   const fo_chunk* __restrict__ chunks, typename Op::Hyper h) {
    __shared__ __align__(16) float lut[StepLut<Op::kLutMask>::kFloats];
    constexpr int kPerTile = Span<Op>::kPerTile;
    const unsigned b = blockIdx.x;
    const fo_chunk ck = chunks[b / kPerTile];
    const TensorPtrs t = load_desc(descs + ck.tensor);
    if constexpr (Op::kLutMask != 0) StepLut<Op::kLutMask>::fill(lut, kStepTables<Op::kDtype>.v);
    const bool aligned = all_aligned16(t);
    const int64_t in_tile = (int64_t)(b % kPerTile) * Span<Op>::kElems;
    for (int i = 0; i < ck.n_tiles; ++i) {
        const int64_t base = ((int64_t)ck.first_tile + i) * kTileElems + in_tile;
        if (base < t.n) run_span<Op>(t, base, aligned, h, lut);
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
// several KiB of loads outstanding.  Each kernel family therefore names the number of workgroups it wants
// resident per compute unit (Op::kWorkgroupsPerCu, the best of those measured on MI355X) and the launch requests
// enough unused dynamic LDS to cap the residency there.  MI355X hands out its 160 KiB of LDS per compute unit in 128
// units of 320 dwords, so the counts that can be reached this way are 128 / k: ... 12, 14, 16, 18, 21, 25, 32
// (measured durations fall on exactly these plateaus, whatever finer count the runtime's occupancy query grants).
// The allocation unit is not something the runtime reports: on a device whose LDS per compute unit is not those
// 160 KiB the plan does not assume it and sizes the request from the occupancy query alone (lds / target bytes).
// A family may also cap the wavefronts per SIMD (Op::kMaxWavesPerSimd: the kernel descriptor then declares enough
// registers that a SIMD holds no more; the occupancy query does not see that padding, so the cap is applied here).
struct Residency {
    int target = 0;    // workgroups per compute unit asked for
    int achieved = 0;  // what the LDS request, the occupancy query and the cap per SIMD allow together
    unsigned dynamic_lds = 0;
    int lds_unit_bytes = 0;  // allocation unit assumed (0: unknown device, the occupancy query alone was used)
};

constexpr long kLdsUnitBytes = 1280;     // MI355X: 320 dwords
constexpr long kLdsUnitsPerCu = 128;     // 160 KiB / 1280
constexpr int kSimdsPerCu = 4;

template <class Kernel>
Residency plan_residency(Kernel kernel, int target, int static_lds, int max_waves_per_simd) {
    Residency r;
    r.target = target;
    int dev = 0, lds_per_cu = 0;
    if (hipGetDevice(&dev) != hipSuccess ||
        hipDeviceGetAttribute(&lds_per_cu, hipDeviceAttributeMaxSharedMemoryPerMultiprocessor, dev) != hipSuccess || lds_per_cu <= 0)
        return r;
    // one launch may ask for at most 64 KiB of LDS: fewer than three workgroups per compute unit cannot be enforced
    constexpr long kMaxLdsPerLaunch = 65536;
    long bytes, by_units;
    if (lds_per_cu == kLdsUnitBytes * kLdsUnitsPerCu) {
        // the most LDS units per workgroup that still admit `target` workgroups
        long units = kLdsUnitsPerCu / target;
        const long least = (static_lds + kLdsUnitBytes - 1) / kLdsUnitBytes;
        if (units < least) units = least;
        if (units < 1) units = 1;
        if (units * kLdsUnitBytes > kMaxLdsPerLaunch) units = kMaxLdsPerLaunch / kLdsUnitBytes;
        bytes = units * kLdsUnitBytes;
        by_units = kLdsUnitsPerCu / units;
        r.lds_unit_bytes = (int)kLdsUnitBytes;
    } else {
        bytes = (lds_per_cu / target) & ~255L;
        if (bytes > kMaxLdsPerLaunch) bytes = kMaxLdsPerLaunch;
        if (bytes < static_lds) bytes = static_lds;
        by_units = INT32_MAX;  // unknown unit: trust the query
    }
    const long dyn = bytes > static_lds ? bytes - static_lds : 0;
    int granted = 0;
    if (hipOccupancyMaxActiveBlocksPerMultiprocessor(&granted, kernel, fo::kBlockThreads, (size_t)dyn) != hipSuccess) granted = 0;
    long achieved = granted < by_units ? granted : by_units;
    const long by_simd = (long)kSimdsPerCu * max_waves_per_simd;
    if (achieved > by_simd) achieved = by_simd;
    r.achieved = (int)achieved;
    r.dynamic_lds = (unsigned)dyn;
    return r;
}

// A kernel family may name a second residency for launches over many short tensors (Op::kWorkgroupsPerCuShortTensors):
// every jump of the streams to another tensor's addresses costs machine time, and lists with thousands of such jumps
// measured fastest with more wavefronts resident than a few long tensors want.  A launch counts as such when its
// tensors average less than kShortTensorTiles tiles of 4096 elements.
constexpr int64_t kShortTensorTiles = 256;
inline bool is_short_tensor_list(int64_t n_tensors, int64_t n_tiles) { return n_tiles < kShortTensorTiles * n_tensors; }

// The three launch shapes a kernel family may want different residencies for: the multi-tensor kernel over long
// tensors (Op::kWorkgroupsPerCu), over many short tensors (Op::kWorkgroupsPerCuShortTensors), and the single-tensor
// kernel (Op::kWorkgroupsPerCuSingleTensor).
enum LaunchShape { kLongTensors = 0, kShortTensors = 1, kSingleTensor = 2 };

// Residency of kernel K for Op on the current device (planned at the first launch of that shape there).
template <class Op, class Kernel> const Residency& residency_of(Kernel kernel, LaunchShape shape) {
    constexpr int kMaxDevices = 64;
    static Residency cache[kMaxDevices][3];
    static std::once_flag once[kMaxDevices][3];
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kMaxDevices) dev = 0;
    std::call_once(once[dev][shape], [&] {
        const int forced = debug_workgroups_per_cu();
        constexpr int kStatic = fo::StepLut<Op::kLutMask>::kFloats * 4;
        const int wanted = shape == kShortTensors ? Op::kWorkgroupsPerCuShortTensors
                         : shape == kSingleTensor ? Op::kWorkgroupsPerCuSingleTensor : Op::kWorkgroupsPerCu;
        cache[dev][shape] = plan_residency(kernel, forced > 0 ? forced : wanted, kStatic, Op::kMaxWavesPerSimd);
    });
    return cache[dev][shape];
}

template <class Op>
int launch_single(const fo::TensorPtrs& t, const typename Op::Hyper& h, hipStream_t stream) {
    // one pass over the tensor, one short-lived workgroup per span
    const int64_t grid = (t.n + fo::Span<Op>::kElems - 1) / fo::Span<Op>::kElems;
    if (grid > INT32_MAX) return fail(FO_ERR_INVALID_ARGUMENT, "tensor too large for one launch (%lld elements)", (long long)t.n);
    const unsigned lds = residency_of<Op>(fo::step_single_kernel<Op>, kSingleTensor).dynamic_lds;
    hipLaunchKernelGGL(fo::step_single_kernel<Op>, dim3((unsigned)grid), dim3(fo::kBlockThreads), lds, stream, t, h);
    return check_hip(hipGetLastError(), "step kernel launch");
}

// n_tiles: 4096-element tiles the chunk table covers (n_chunks when a chunk is one tile; an estimate is good enough,
// it only chooses between the two residencies)
template <class Op>
int launch_multi(const fo_tensor_desc* descs, int64_t n_tensors, const fo_chunk* chunks, int64_t n_chunks, int64_t n_tiles,
                 const typename Op::Hyper& h, hipStream_t stream) {
    const int64_t grid = n_chunks * fo::Span<Op>::kPerTile;
    if (grid > INT32_MAX) return fail(FO_ERR_INVALID_ARGUMENT, "chunk table too large for one launch (%lld chunks)", (long long)n_chunks);
    const LaunchShape shape = is_short_tensor_list(n_tensors, n_tiles) ? kShortTensors : kLongTensors;
    const unsigned lds = residency_of<Op>(fo::step_multi_kernel<Op>, shape).dynamic_lds;
    hipLaunchKernelGGL(fo::step_multi_kernel<Op>, dim3((unsigned)grid), dim3(fo::kBlockThreads), lds, stream, descs, chunks, h);
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

// Reports the residency plan of a kernel family (diagnostic entry points): 0 on success.
struct ResidencyQuery {
    int multi; int* target; int* achieved; int* dynamic_lds;   // multi: 0 single-tensor kernel, 1 multi-tensor kernel, 2 the latter over short tensors
    template <class Op> int operator()() {
        const Residency& r = multi ? residency_of<Op>(fo::step_multi_kernel<Op>, multi == 2 ? kShortTensors : kLongTensors)
                                   : residency_of<Op>(fo::step_single_kernel<Op>, kSingleTensor);
        if (target) *target = r.target;
        if (achieved) *achieved = r.achieved;
        if (dynamic_lds) *dynamic_lds = (int)r.dynamic_lds;
        return r.achieved > 0 ? 0 : fail(FO_ERR_NO_DEVICE, "occupancy query failed");
    }
};

template <class H> struct SingleLauncher {
    fo::TensorPtrs t; H h; hipStream_t s;
    template <class Op> int operator()() { return launch_single<Op>(t, h, s); }
};
template <class H> struct MultiLauncher {
    const fo_tensor_desc* d; int64_t nt; const fo_chunk* c; int64_t nc; int64_t tiles; H h; hipStream_t s;
    template <class Op> int operator()() { return launch_multi<Op>(d, nt, c, nc, tiles, h, s); }
};


}  // namespace fo_host
