// Fused Adam / AdamW step kernel for gfx950 and its C entry points (ref: /root/reference/flashoptim/
// optimizers.py:2203-2438, cited as "ref:").
#include "fo_step.h"
#ifdef FO_DIAG
#include "../../include/flashoptim_hip_diag.h"
#endif

#include <mutex>

namespace fo {

// What a lane holds between issuing its loads and consuming them.
template <int DT, int ECCB, bool QUANT> struct AdamRaw {
    static constexpr int EPL = DTypeInfo<DT>::epl;
    Pack<DTypeInfo<DT>::bytes, EPL> p, g;
    Pack<ECCB, EPL> e;
    Pack<QUANT ? 1 : DTypeInfo<DT>::bytes, EPL> m, v;
    uint16_t sm, sv;
};

template <int DT, int ECCB, bool QUANT, int FAST>
__device__ __forceinline__ void adam_load(const TensorPtrs& t, Where w, AdamRaw<DT, ECCB, QUANT>& r) {
    constexpr int EPL = DTypeInfo<DT>::epl;
    constexpr int PB = DTypeInfo<DT>::bytes;
    constexpr int SB = QUANT ? 1 : PB;  // state bytes per element
    const int64_t n = t.n;
    load_lane<PB, EPL, FAST>(r.g, t.grad, w, n);
    load_lane<PB, EPL, FAST>(r.p, t.param, w, n);
    load_lane<ECCB, EPL, FAST>(r.e, t.ecc, w, n);
    load_lane<SB, EPL, FAST>(r.m, t.mom, w, n);
    load_lane<SB, EPL, FAST>(r.v, t.var, w, n);
    r.sm = r.sv = 0x3c00;  // masked scales read 1.0 (ref:2318-2323)
    if constexpr (QUANT) {
        if (FAST == kVector || w.first() < n) {
            r.sm = load_scale(t.mom_scales, w);
            r.sv = load_scale(t.var_scales, w);
        }
    }
}

// Lane state of adam_redo_flagged (fo_math.h): the old weight is still in the lane's raw parameter and ECC words.
template <int DT, int ECCB, bool QUANT> struct AdamRedoLane {
    static constexpr int EPL = DTypeInfo<DT>::epl;
    float (&p)[EPL];
    const float (&slack)[EPL];
    const float (&m)[EPL];
    const float (&v)[EPL];
    const AdamRaw<DT, ECCB, QUANT>& raw;
    const float* lut;
    float least;
    __device__ __forceinline__ float old_master(int k) const { return master_of<DT, ECCB, EPL>(raw.p, raw.e, k, lut); }
};

template <int DT, int ECCB, bool QUANT, bool DECOUPLED, bool EXACT, int FAST>
__device__ __forceinline__ void adam_finish(const TensorPtrs& t, Where w, AdamRaw<DT, ECCB, QUANT>& raw,
                                            const AdamHyper& h, const float* lut) {
    constexpr int EPL = DTypeInfo<DT>::epl;
    constexpr int PB = DTypeInfo<DT>::bytes;
    constexpr int SB = QUANT ? 1 : PB;
    const int64_t n = t.n;
    const bool live_group = FAST == kVector || w.first() < n;  // the lane owns at least one real element
    const float sm = f16_bits_to_f32(raw.sm), sv = f16_bits_to_f32(raw.sv);

    float p[EPL], m[EPL], r[EPL], v[EPL];
    read_master<DT, ECCB, EPL>(p, raw.p, raw.e, lut);
    float slack[EPL];  // folded update: negative where the element has to be redone operation by operation

#pragma unroll
    for (int k = 0; k < EPL; ++k) {
        float g = widen<DT, EPL>(raw.g, k);
        if constexpr (!DECOUPLED) g = g + p[k] * h.wd;                              // ref:2310-2311
        float mn, vn;
        if constexpr (QUANT) {
            adam_moments_quantized(g, lookup_mom(lut, byte_of<EPL>(raw.m, k)), sm, (float)byte_of<EPL>(raw.v, k), sv, h, mn, vn);
        } else {
            adam_moments_plain(g, widen<DT, EPL>(raw.m, k), widen<DT, EPL>(raw.v, k), h, mn, vn);
        }
        // sqrt(v) as the instruction gives it: the quick requantiser form and the folded update are content with it
        const float rk = (QUANT || !EXACT) ? hw::sqrt(vn) : 0.0f;
        if constexpr (EXACT) {
            const float pk = DECOUPLED ? p[k] * h.one_m_wd : p[k];                  // ref:2363-2364
            p[k] = adam_apply_exact(pk, mn, vn, h);                                 // ref:2368-2375
        } else {
            // folded update; `redo` marks the elements it cannot vouch for (fo_math.h).  The old weight stays in
            // raw.p / raw.e for the repair below.
            p[k] = adam_apply_folded<DECOUPLED>(p[k], mn, rk, h, AdamFoldedGuard<DT, ECCB>::value, slack[k]);
        }
        m[k] = mn; r[k] = rk; v[k] = vn;
    }
    if constexpr (!EXACT) {
        // The flagged elements again, operation by operation (fo_math.h: adam_redo_flagged).  A wavefront with no
        // flagged element branches past this; otherwise only the positions flagged in some lane are redone.
        AdamRedoLane<DT, ECCB, QUANT> lane{p, slack, m, v, raw, lut};
        HwWave<AdamRedoLane<DT, ECCB, QUANT>> wave{lane};
        adam_redo_flagged<EPL, DECOUPLED>(wave, h);
    }

    Pack<ECCB, EPL> eout;
    write_master<DT, ECCB, EPL>(p, raw.p, eout);
    store_lane<PB, EPL, FAST>(raw.p, t.param, w, n);
    store_lane<ECCB, EPL, FAST>(eout, t.ecc, w, n);

    if constexpr (QUANT) {
        // group absmax (ref:2399-2404); the square root is monotone, so the largest sqrt(v) is the root of the largest v
        float am = 0.0f, av = 0.0f;
#pragma unroll
        for (int k = 0; k < EPL; k += 2) {  // pairs, so that each step is one three-operand max
            am = fmaxf(fmaxf(am, fabsf(m[k])), fabsf(m[k + 1]));
            av = fmaxf(fmaxf(av, v[k]), v[k + 1]);
        }
        am = fmaxf(group_max<EPL>(am), 1e-12f);
        av = group_max<EPL>(av);                              // the group's largest v
        const float av_quick = fmaxf(hw::sqrt(av), 1e-12f);
        av = fmaxf(sqrt_corrected(av), 1e-12f);               // what the exact requantiser divides by, and the scale
        if constexpr (EPL == 8) {
            quantize_mom_quick_verified<EPL>(m, am, raw.m);
            quantize_var_quick_verified<EPL>(v, r, av_quick, av, raw.v);
        } else {
            quantize_mom_var_quick_verified(m, am, v, r, av_quick, av, raw.m, raw.v);
        }
        store_lane<1, EPL, FAST>(raw.m, t.mom, w, n);
        store_lane<1, EPL, FAST>(raw.v, t.var, w, n);
        if (live_group && (threadIdx.x & (32 / EPL - 1)) == 0) {                    // ref:2424-2434
            store_scale(t.mom_scales, w, f32_to_f16_bits(am));
            store_scale(t.var_scales, w, f32_to_f16_bits(av));
        }
    } else {
        narrow_all<DT, EPL>(m, raw.m);                                              // ref:2435-2438
        narrow_all<DT, EPL>(v, raw.v);
        store_lane<SB, EPL, FAST>(raw.m, t.mom, w, n);
        store_lane<SB, EPL, FAST>(raw.v, t.var, w, n);
    }
}

// EXACT: the update follows the reference operation by operation (fo_math.h: AdamExact names the variants that do so
// by default; the *_exact entry points ask for it on every variant).
template <int DT, int ECCB, bool QUANT, bool DECOUPLED, bool EXACT = AdamExact<DT, ECCB>::value> struct AdamOp {
    using Hyper = AdamHyper;
    static constexpr int kLutMask = (QUANT ? 1 << kTableMom : 0) | (ECCB == 1 ? 1 << kTableEcc : 0);  // LDS code tables
    static constexpr int kDtype = DT;
    // Measured on MI355X with the 8B-parameter step and this file's ILP-oriented instruction schedule, over the
    // residencies the LDS units allow (fo_step.h):
    //   guarded folded update on 2-byte parameters: 16 workgroups per compute unit, at most four wavefronts per SIMD
    //     (14: -4 points, 18 with five per SIMD: -5, 21 with six: -6; 16 without the cap per SIMD: -0.4);
    //   operation-by-operation update on 2-byte parameters (2-byte ECC, fp16 with a 1-byte ECC, the *_exact entry
    //     points): 20 with at most five per SIMD (16/4: -3.5 points, 18/5 and 21/6: -1.3, 25 and 32 uncapped: -3);
    //   fp32 parameters (2.5 KiB of loads per wavefront), multi-tensor kernel: 21, with or without a cap of six or
    //     seven per SIMD (18: -3.8 points, 25: -1.5, 32: -3; 20 with five per SIMD and 24 with six: -1); the
    //     single-tensor kernel, launched tensor by tensor in gradient-release order (fewer registers, no launch
    //     tables): 18 (21: -1.3 points, 25: -1.9).
    static constexpr bool kNarrowExact = EXACT && DT != DT_F32;
    static constexpr int kWorkgroupsPerCu = DT == DT_F32 ? 21 : (kNarrowExact ? 20 : 16);
    static constexpr int kWorkgroupsPerCuShortTensors = kWorkgroupsPerCu;
    static constexpr int kWorkgroupsPerCuSingleTensor = DT == DT_F32 ? 18 : kWorkgroupsPerCu;
    static constexpr int kMaxWavesPerSimd = DT == DT_F32 ? 8 : (kNarrowExact ? 5 : 4);
    static constexpr int kEpl = DTypeInfo<DT>::epl;
    using Raw = AdamRaw<DT, ECCB, QUANT>;
    template <int FAST> __device__ __forceinline__ static void load(const TensorPtrs& t, Where w, Raw& r) {
        adam_load<DT, ECCB, QUANT, FAST>(t, w, r);
    }
    template <int FAST>
    __device__ __forceinline__ static void finish(const TensorPtrs& t, Where w, Raw& r, const Hyper& h, const float* lut) {
        adam_finish<DT, ECCB, QUANT, DECOUPLED, EXACT, FAST>(t, w, r, h, lut);
    }
};


#ifdef FO_DIAG
// The Adam step's memory accesses without its arithmetic: every stream of the step is loaded and stored back
// unchanged through the same load / store code, launch geometry and residency mechanism.  It shows what rate this
// mix of seven loads and six stores per wavefront reaches on the device, next to the step kernels' own rate.
// `mask` arrives as zero from the entry point; folding the gradient words in under it keeps the gradient loads
// alive without changing any byte.
struct StreamsHyper { uint32_t mask; };

template <int DT, int ECCB, bool QUANT> struct AdamStreamsOp {
    using Hyper = StreamsHyper;
    static constexpr int kLutMask = 0;
    static constexpr int kDtype = DT;
    // where this copy streams fastest on MI355X with the 8B-parameter list: 16 with 1-byte ECC (14 and 18 are three
    // to four points slower), 14 with 2-byte ECC (16 one point slower); fp32 parameters (256 elements and 2.5 KiB per
    // wavefront, the codes as 4-byte loads) want every slot: 32 (79.6 %; 25: 79.2 %, 18: 74.6 %)
    static constexpr int kWorkgroupsPerCu = DT == DT_F32 ? 32 : (ECCB == 2 ? 14 : 16);
    static constexpr int kWorkgroupsPerCuShortTensors = kWorkgroupsPerCu;
    static constexpr int kWorkgroupsPerCuSingleTensor = kWorkgroupsPerCu;
    static constexpr int kMaxWavesPerSimd = 8;
    static constexpr int kEpl = DTypeInfo<DT>::epl;
    using Raw = AdamRaw<DT, ECCB, QUANT>;
    template <int FAST> __device__ __forceinline__ static void load(const TensorPtrs& t, Where w, Raw& r) {
        adam_load<DT, ECCB, QUANT, FAST>(t, w, r);
    }
    template <int FAST>
    __device__ __forceinline__ static void finish(const TensorPtrs& t, Where w, Raw& r, const Hyper& h, const float*) {
        constexpr int PB = DTypeInfo<DT>::bytes;
        constexpr int SB = QUANT ? 1 : PB;
#pragma unroll
        for (int i = 0; i < Pack<PB, kEpl>::kDwords; ++i) r.p.w[i] ^= r.g.w[i] & h.mask;
        store_lane<PB, kEpl, FAST>(r.p, t.param, w, t.n);
        store_lane<ECCB, kEpl, FAST>(r.e, t.ecc, w, t.n);
        store_lane<SB, kEpl, FAST>(r.m, t.mom, w, t.n);
        store_lane<SB, kEpl, FAST>(r.v, t.var, w, t.n);
        if constexpr (QUANT) {
            if ((FAST == kVector || w.first() < t.n) && (threadIdx.x & (32 / kEpl - 1)) == 0) {
                store_scale(t.mom_scales, w, r.sm);
                store_scale(t.var_scales, w, r.sv);
            }
        }
    }
};

#endif  // FO_DIAG

}  // namespace fo

namespace {
using namespace fo_host;

template <int DT, int EB, bool Q> using AdamL2Op = fo::AdamOp<DT, EB, Q, false>;  // FlashAdam: decay folded into the gradient
template <int DT, int EB, bool Q> using AdamWOp = fo::AdamOp<DT, EB, Q, true>;    // FlashAdamW: decay applied to the weights
template <int DT, int EB, bool Q> using AdamL2ExactOp = fo::AdamOp<DT, EB, Q, false, true>;
template <int DT, int EB, bool Q> using AdamWExactOp = fo::AdamOp<DT, EB, Q, true, true>;

// exact: the caller asked for the operation-by-operation update on every element; a launch whose folded constants
// are out of range (fo_math.h: make_adam_hyper) takes it too.
template <class L> int dispatch_adam(int dtype, int ecc_bytes, int quantized, int decoupled, int exact, L&& launcher) {
    if (exact || !launcher.h.folded_ok)
        return decoupled ? dispatch<AdamWExactOp>(dtype, ecc_bytes, quantized, launcher)
                         : dispatch<AdamL2ExactOp>(dtype, ecc_bytes, quantized, launcher);
    return decoupled ? dispatch<AdamWOp>(dtype, ecc_bytes, quantized, launcher) : dispatch<AdamL2Op>(dtype, ecc_bytes, quantized, launcher);
}

using fo::make_adam_hyper;

// ------------------------------------------------------------------------------------------------
// launch tables held in a static device array (fo_multi_adam_step_static)
// ------------------------------------------------------------------------------------------------
// Layout of the array: kStaticMaxTensors descriptors, then kStaticMaxChunks chunk entries.  Every device the
// library runs on holds its own copy until the process ends (1.06 MiB).  Calls on one device share it and keep
// the previous call's tables; a call overwrites every entry it uses, so nothing has to be cleared.
constexpr int64_t kStaticMaxTensors = FO_STATIC_MAX_TENSORS;
constexpr int64_t kStaticMaxChunks = FO_STATIC_MAX_CHUNKS;
constexpr size_t kStaticBytes = kStaticMaxTensors * sizeof(fo_tensor_desc) + kStaticMaxChunks * sizeof(fo_chunk);
static __device__ __align__(256) __attribute__((used)) unsigned char scratch[kStaticBytes];

// Device address of `scratch` on the current device.  The array's name is only a host-side handle: the address a
// kernel can use comes from hipGetSymbolAddress, once per device, with that device current.
int static_tables(int* device_out, fo_tensor_desc** descs, fo_chunk** chunks) {
    constexpr int kMaxDevices = 64;
    static void* base[kMaxDevices];
    static std::once_flag once[kMaxDevices];
    static hipError_t status[kMaxDevices];
    int dev = 0;
    if (int rc = check_hip(hipGetDevice(&dev), "hipGetDevice")) return rc;
    if (dev < 0 || dev >= kMaxDevices) return fail(FO_ERR_NO_DEVICE, "device index %d out of range", dev);
    std::call_once(once[dev], [&] { status[dev] = hipGetSymbolAddress(&base[dev], HIP_SYMBOL(scratch)); });
    if (int rc = check_hip(status[dev], "hipGetSymbolAddress(scratch)")) return rc;
    if (!base[dev]) return fail(FO_ERR_NO_DEVICE, "static table array has no device address");
    *device_out = dev;
    *descs = reinterpret_cast<fo_tensor_desc*>(base[dev]);
    *chunks = reinterpret_cast<fo_chunk*>(static_cast<unsigned char*>(base[dev]) + kStaticMaxTensors * sizeof(fo_tensor_desc));
    return 0;
}

// A batch of descriptors travels to the device as a kernel argument (no copy engine, no staging memory):
// workgroup i of the launch writes descriptor i of the batch and the chunk entries of that tensor.
constexpr int kStageBatch = 48;
struct StageBatch {
    fo_tensor_desc desc[kStageBatch];
    int32_t first_chunk[kStageBatch];
    int32_t base_tensor, count, tiles_per_chunk, reserved;
};
static_assert(sizeof(StageBatch) <= 3584, "a batch must fit the kernel argument segment");

__global__ __launch_bounds__(256) void stage_tables_kernel(StageBatch b, fo_tensor_desc* descs, fo_chunk* chunks) {
    const int i = blockIdx.x;
    if (i >= b.count) return;
    const int tensor = b.base_tensor + i;
    if (threadIdx.x == 0) descs[tensor] = b.desc[i];
    const int64_t tiles = (b.desc[i].n + fo::kTileElems - 1) / fo::kTileElems;
    const int64_t n_chunks = (tiles + b.tiles_per_chunk - 1) / b.tiles_per_chunk;
    for (int64_t c = threadIdx.x; c < n_chunks; c += blockDim.x) {
        fo_chunk ck;
        ck.tensor = tensor;
        ck.first_tile = (int32_t)(c * b.tiles_per_chunk);
        const int64_t left = tiles - c * b.tiles_per_chunk;
        ck.n_tiles = (int32_t)(left < b.tiles_per_chunk ? left : b.tiles_per_chunk);
        ck.reserved = 0;
        chunks[b.first_chunk[i] + c] = ck;
    }
}

}  // namespace

extern "C" {

static int adam_step_any(void* mom, void* mom_scales, void* var, void* var_scales, void* param, const void* grad, void* ecc,
                         int64_t n, int dtype, int ecc_bytes, int quantized, float lr, float beta1, float beta2, float eps,
                         float weight_decay, int decoupled, int step, void* stream, int exact) {
    if (int rc = validate_common(param, grad, ecc, n, dtype, ecc_bytes)) return rc;
    if (n == 0) return 0;  // ref:2221-2223
    if (step < 1) return fail(FO_ERR_INVALID_ARGUMENT, "step must be >= 1 (got %d)", step);
    if (int rc = validate_state(mom, mom_scales, quantized, dtype, "mom")) return rc;
    if (int rc = validate_state(var, var_scales, quantized, dtype, "var")) return rc;
    fo::TensorPtrs t{param, grad, ecc_bytes ? ecc : nullptr, mom, (uint16_t*)mom_scales, var, (uint16_t*)var_scales, n};
    SingleLauncher<fo::AdamHyper> L{t, make_adam_hyper(lr, beta1, beta2, eps, weight_decay, step), (hipStream_t)stream};
    return dispatch_adam(dtype, ecc_bytes, quantized, decoupled, exact, L);
}

int fo_adam_step(void* mom, void* mom_scales, void* var, void* var_scales, void* param, const void* grad, void* ecc,
                 int64_t n, int dtype, int ecc_bytes, int quantized, float lr, float beta1, float beta2, float eps,
                 float weight_decay, int decoupled, int step, void* stream) {
    return adam_step_any(mom, mom_scales, var, var_scales, param, grad, ecc, n, dtype, ecc_bytes, quantized, lr, beta1, beta2,
                         eps, weight_decay, decoupled, step, stream, 0);
}

int fo_adam_step_exact(void* mom, void* mom_scales, void* var, void* var_scales, void* param, const void* grad, void* ecc,
                       int64_t n, int dtype, int ecc_bytes, int quantized, float lr, float beta1, float beta2, float eps,
                       float weight_decay, int decoupled, int step, void* stream) {
    return adam_step_any(mom, mom_scales, var, var_scales, param, grad, ecc, n, dtype, ecc_bytes, quantized, lr, beta1, beta2,
                         eps, weight_decay, decoupled, step, stream, 1);
}

static int multi_adam_step_any(const fo_tensor_desc* descs, int64_t n_tensors, const fo_chunk* chunks, int64_t n_chunks,
                               int dtype, int ecc_bytes, int quantized, float lr, float beta1, float beta2, float eps,
                               float weight_decay, int decoupled, int step, void* stream, int exact) {
    if (int rc = validate_multi(descs, n_tensors, chunks, n_chunks, dtype, ecc_bytes)) return rc;
    if (n_chunks == 0) return 0;
    if (step < 1) return fail(FO_ERR_INVALID_ARGUMENT, "step must be >= 1 (got %d)", step);
    MultiLauncher<fo::AdamHyper> L{descs, n_tensors, chunks, n_chunks, n_chunks, make_adam_hyper(lr, beta1, beta2, eps, weight_decay, step), (hipStream_t)stream};
    return dispatch_adam(dtype, ecc_bytes, quantized, decoupled, exact, L);
}

int fo_multi_adam_step(const fo_tensor_desc* descs, int64_t n_tensors, const fo_chunk* chunks, int64_t n_chunks, int dtype,
                       int ecc_bytes, int quantized, float lr, float beta1, float beta2, float eps, float weight_decay,
                       int decoupled, int step, void* stream) {
    return multi_adam_step_any(descs, n_tensors, chunks, n_chunks, dtype, ecc_bytes, quantized, lr, beta1, beta2, eps,
                               weight_decay, decoupled, step, stream, 0);
}

int fo_multi_adam_step_exact(const fo_tensor_desc* descs, int64_t n_tensors, const fo_chunk* chunks, int64_t n_chunks, int dtype,
                             int ecc_bytes, int quantized, float lr, float beta1, float beta2, float eps, float weight_decay,
                             int decoupled, int step, void* stream) {
    return multi_adam_step_any(descs, n_tensors, chunks, n_chunks, dtype, ecc_bytes, quantized, lr, beta1, beta2, eps,
                               weight_decay, decoupled, step, stream, 1);
}

int fo_multi_adam_step_static(const fo_tensor_desc* host_descs, int64_t n_tensors, int dtype, int ecc_bytes, int quantized,
                              float lr, float beta1, float beta2, float eps, float weight_decay, int decoupled, int step,
                              void* stream) {
    if (n_tensors < 0) return fail(FO_ERR_INVALID_ARGUMENT, "negative tensor count");
    if (n_tensors > kStaticMaxTensors)
        return fail(FO_ERR_INVALID_ARGUMENT, "%lld tensors exceed the static table's %lld (use fo_multi_adam_step with caller-owned tables)",
                    (long long)n_tensors, (long long)kStaticMaxTensors);
    if (n_tensors > 0 && !host_descs) return fail(FO_ERR_INVALID_ARGUMENT, "host_descs must not be NULL");
    if (dtype < FO_F32 || dtype > FO_F16) return fail(FO_ERR_INVALID_ARGUMENT, "unknown dtype %d", dtype);
    if (ecc_bytes < 0 || ecc_bytes > 2) return fail(FO_ERR_INVALID_ARGUMENT, "ecc_bytes must be 0, 1 or 2 (got %d)", ecc_bytes);
    if (dtype == FO_F32 && ecc_bytes != 0) return fail(FO_ERR_UNSUPPORTED, "fp32 parameters carry no ECC");
    if (step < 1) return fail(FO_ERR_INVALID_ARGUMENT, "step must be >= 1 (got %d)", step);
    int64_t total_tiles = 0;
    for (int64_t i = 0; i < n_tensors; ++i) {
        const fo_tensor_desc& d = host_descs[i];
        if (d.n < 0) return fail(FO_ERR_INVALID_ARGUMENT, "tensor %lld has negative length", (long long)i);
        if (d.n == 0) continue;
        if (int rc = validate_common(d.param, d.grad, d.ecc, d.n, dtype, ecc_bytes)) return rc;
        if (int rc = validate_state(d.mom, d.mom_scales, quantized, dtype, "mom")) return rc;
        if (int rc = validate_state(d.var, d.var_scales, quantized, dtype, "var")) return rc;
        const int64_t tiles = (d.n + fo::kTileElems - 1) / fo::kTileElems;
        if (tiles > INT32_MAX) return fail(FO_ERR_INVALID_ARGUMENT, "tensor %lld too large", (long long)i);
        total_tiles += tiles;
    }
    if (total_tiles == 0) return 0;
    // the fewest tiles per chunk that keep the chunk table inside the array (every tensor may end with a short chunk)
    int64_t tiles_per_chunk = 1;
    auto count_chunks = [&](int64_t tpc) {
        int64_t c = 0;
        for (int64_t i = 0; i < n_tensors; ++i) c += ((host_descs[i].n + fo::kTileElems - 1) / fo::kTileElems + tpc - 1) / tpc;
        return c;
    };
    int64_t n_chunks = count_chunks(tiles_per_chunk);
    if (n_chunks > kStaticMaxChunks) {  // count <= total_tiles / tpc + n_tensors
        tiles_per_chunk = (total_tiles + (kStaticMaxChunks - n_tensors) - 1) / (kStaticMaxChunks - n_tensors);
        if (tiles_per_chunk > INT32_MAX) return fail(FO_ERR_INVALID_ARGUMENT, "tensor list too large for the static chunk table");
        n_chunks = count_chunks(tiles_per_chunk);
    }
    int dev = 0;
    fo_tensor_desc* d_descs = nullptr;
    fo_chunk* d_chunks = nullptr;
    if (int rc = static_tables(&dev, &d_descs, &d_chunks)) return rc;

    StageBatch b;
    int64_t next_chunk = 0;
    for (int64_t t0 = 0; t0 < n_tensors; t0 += kStageBatch) {
        b.base_tensor = (int32_t)t0;
        b.count = (int32_t)((n_tensors - t0) < kStageBatch ? (n_tensors - t0) : kStageBatch);
        b.tiles_per_chunk = (int32_t)tiles_per_chunk;
        b.reserved = 0;
        for (int i = 0; i < b.count; ++i) {
            b.desc[i] = host_descs[t0 + i];
            b.first_chunk[i] = (int32_t)next_chunk;
            const int64_t tiles = (b.desc[i].n + fo::kTileElems - 1) / fo::kTileElems;
            next_chunk += (tiles + tiles_per_chunk - 1) / tiles_per_chunk;
        }
        hipLaunchKernelGGL(stage_tables_kernel, dim3((unsigned)b.count), dim3(256), 0, (hipStream_t)stream, b, d_descs, d_chunks);
        if (int rc = check_hip(hipGetLastError(), "table staging kernel launch")) return rc;
    }
    MultiLauncher<fo::AdamHyper> L{d_descs, n_tensors, d_chunks, n_chunks, total_tiles, make_adam_hyper(lr, beta1, beta2, eps, weight_decay, step), (hipStream_t)stream};
    return dispatch_adam(dtype, ecc_bytes, quantized, decoupled, 0, L);
}

#ifdef FO_DIAG
int fo_multi_adam_streams_copy(const fo_tensor_desc* descs, int64_t n_tensors, const fo_chunk* chunks, int64_t n_chunks,
                               int dtype, int ecc_bytes, int quantized, void* stream) {
    if (int rc = validate_multi(descs, n_tensors, chunks, n_chunks, dtype, ecc_bytes)) return rc;
    if (n_chunks == 0) return 0;
    MultiLauncher<fo::StreamsHyper> L{descs, n_tensors, chunks, n_chunks, n_chunks, fo::StreamsHyper{0u}, (hipStream_t)stream};
    return dispatch<fo::AdamStreamsOp>(dtype, ecc_bytes, quantized, L);
}

int fo_adam_step_residency(int dtype, int ecc_bytes, int quantized, int decoupled, int multi, int* target, int* achieved,
                           int* dynamic_lds) {
    ResidencyQuery q{multi, target, achieved, dynamic_lds};
    return decoupled ? dispatch<AdamWOp>(dtype, ecc_bytes, quantized, q) : dispatch<AdamL2Op>(dtype, ecc_bytes, quantized, q);
}

#endif  // FO_DIAG

}  // extern "C"
