// Fused SGD / SGDW / Nesterov / Lion step kernels (and the momentum-free SGD step) for gfx950 with their C
// entry points (ref: /root/reference/flashoptim/optimizers.py:1447-1465, 1535-1719, cited as "ref:").
#include "fo_step.h"
#ifdef FO_DIAG
#include "../../include/flashoptim_hip_diag.h"
#endif

namespace fo {

// ------------------------------------------------------------------------------------------------
// SGD / SGDW / Nesterov / Lion / momentum-free SGD (ref:1586-1719, 1447-1465)
// ------------------------------------------------------------------------------------------------
template <int DT, int ECCB, bool QUANT, int KIND> struct MomentumRaw {
    static constexpr int EPL = DTypeInfo<DT>::epl;
    static constexpr int SB = (KIND == KIND_PLAIN) ? 0 : (QUANT ? 1 : DTypeInfo<DT>::bytes);
    Pack<DTypeInfo<DT>::bytes, EPL> p, g;
    Pack<ECCB, EPL> e;
    Pack<SB, EPL> m;
    uint16_t sm;
};

template <int DT, int ECCB, bool QUANT, int KIND, int FAST>
__device__ __forceinline__ void momentum_load(const TensorPtrs& t, Where w, MomentumRaw<DT, ECCB, QUANT, KIND>& r) {
    constexpr int EPL = DTypeInfo<DT>::epl;
    constexpr int PB = DTypeInfo<DT>::bytes;
    constexpr int SB = MomentumRaw<DT, ECCB, QUANT, KIND>::SB;
    const int64_t n = t.n;
    load_lane<PB, EPL, FAST>(r.g, t.grad, w, n);
    load_lane<PB, EPL, FAST>(r.p, t.param, w, n);
    load_lane<ECCB, EPL, FAST>(r.e, t.ecc, w, n);
    load_lane<SB, EPL, FAST>(r.m, t.mom, w, n);
    r.sm = 0x3c00;  // 1.0
    if constexpr (QUANT && KIND != KIND_PLAIN) {
        if (FAST == kVector || w.first() < n) r.sm = load_scale(t.mom_scales, w);                     // ref:1645-1646
    }
}

template <int DT, int ECCB, bool QUANT, int KIND, int FAST>
__device__ __forceinline__ void momentum_finish(const TensorPtrs& t, Where w, MomentumRaw<DT, ECCB, QUANT, KIND>& raw,
                                                const MomentumHyper& h, const float* lut) {
    constexpr int EPL = DTypeInfo<DT>::epl;
    constexpr int PB = DTypeInfo<DT>::bytes;
    constexpr int SB = MomentumRaw<DT, ECCB, QUANT, KIND>::SB;
    const int64_t n = t.n;
    const bool live_group = FAST == kVector || w.first() < n;
    const float sm = f16_bits_to_f32(raw.sm);

    float p[EPL], m[EPL];
    read_master<DT, ECCB, EPL>(p, raw.p, raw.e, lut);

#pragma unroll
    for (int k = 0; k < EPL; ++k) {
        const float g = widen<DT, EPL>(raw.g, k);
        float mo = 0.0f;
        if constexpr (KIND != KIND_PLAIN) {
            if constexpr (QUANT) mo = lookup_mom(lut, byte_of<EPL>(raw.m, k)) * sm;        // ref:1648-1657
            else mo = widen<DT, EPL>(raw.m, k);                                                 // ref:1660-1661
        }
        momentum_element<KIND>(g, p[k], mo, h, m[k]);
    }

    float am = 0.0f;
    if constexpr (KIND != KIND_PLAIN) {
#pragma unroll
        for (int k = 0; k < EPL; k += 2) am = fmaxf(fmaxf(am, fabsf(m[k])), fabsf(m[k + 1]));
    }

    Pack<ECCB, EPL> eout;
    write_master<DT, ECCB, EPL>(p, raw.p, eout);                                    // ref:1684-1694
    store_lane<PB, EPL, FAST>(raw.p, t.param, w, n);
    store_lane<ECCB, EPL, FAST>(eout, t.ecc, w, n);

    if constexpr (KIND != KIND_PLAIN) {
        if constexpr (QUANT) {
            am = fmaxf(group_max<EPL>(am), 1e-12f);                                 // ref:1702-1703
            // 2-byte parameters: through the quick forms, every value verified (fo_math.h): the exact forms' codes
            if constexpr (EPL == 8) quantize_mom_quick_verified<EPL>(m, am, raw.m);
            else quantize_mom(m, am, raw.m);
            store_lane<1, EPL, FAST>(raw.m, t.mom, w, n);
            if (live_group && (threadIdx.x & (32 / EPL - 1)) == 0) store_scale(t.mom_scales, w, f32_to_f16_bits(am));  // ref:1713-1716
        } else {
            narrow_all<DT, EPL>(m, raw.m);                                          // ref:1717-1719
            store_lane<SB, EPL, FAST>(raw.m, t.mom, w, n);
        }
    }
}

template <int DT, int ECCB, bool QUANT, int KIND> struct MomentumOp {
    using Hyper = MomentumHyper;
    static constexpr int kLutMask = ((QUANT && KIND != KIND_PLAIN) ? 1 << kTableMom : 0) | (ECCB == 1 ? 1 << kTableEcc : 0);  // LDS code tables
    static constexpr int kDtype = DT;
    // Measured on MI355X (3 KiB of loads per wavefront) over the residencies the LDS units allow (fo_step.h: 18, 21,
    // 25, 32 around here), Lion on bf16 parameters with a 1-byte ECC.  The 291 tensors of an 8B-parameter model: 21
    // (82.5 % of the HBM peak; 18: 78.2, 25: 78.8, 32: 77.5).  4096 ragged tensors of 1e9 elements in all: 25 (80.9 %;
    // 21: 79.9, 32: 80.5, 18: 77.6).  A launch therefore picks by the average length of its tensors
    // (fo_step.h: is_short_tensor_list).  Capping the wavefronts per SIMD at 6 or 7 changes nothing measurable.
    // (The ILP-oriented schedule that fo_adam.hip is built with would gain half a point on the ragged list at 21 and
    // lose three on the 8B list.)
    static constexpr int kWorkgroupsPerCu = 21;
    static constexpr int kWorkgroupsPerCuShortTensors = 25;
    static constexpr int kWorkgroupsPerCuSingleTensor = kWorkgroupsPerCu;
    static constexpr int kMaxWavesPerSimd = 8;
    static constexpr int kEpl = DTypeInfo<DT>::epl;
    using Raw = MomentumRaw<DT, ECCB, QUANT, KIND>;
    template <int FAST> __device__ __forceinline__ static void load(const TensorPtrs& t, Where w, Raw& r) {
        momentum_load<DT, ECCB, QUANT, KIND, FAST>(t, w, r);
    }
    template <int FAST>
    __device__ __forceinline__ static void finish(const TensorPtrs& t, Where w, Raw& r, const Hyper& h, const float* lut) {
        momentum_finish<DT, ECCB, QUANT, KIND, FAST>(t, w, r, h, lut);
    }
};


#ifdef FO_DIAG
// The momentum step's memory accesses without its arithmetic (see AdamStreamsOp in fo_adam.hip): parameters,
// gradients, ECC, the moment's codes and scales are loaded and everything but the gradients is stored back unchanged
// by the step's own load / store code.
struct MomentumStreamsHyper { uint32_t mask; };

template <int DT, int ECCB, bool QUANT> struct MomentumStreamsOp {
    using Hyper = MomentumStreamsHyper;
    static constexpr int kLutMask = 0;
    static constexpr int kDtype = DT;
    // measured on MI355X: the 8B-parameter list streams fastest at 14 (83.2 %; 16: 82.0 %, 18: 79.6 %), 4096 ragged
    // tensors at 16 (81.8 %; 14: 80.2 %, 18: 81.5 %)
    static constexpr int kWorkgroupsPerCu = 16;
    static constexpr int kWorkgroupsPerCuShortTensors = kWorkgroupsPerCu;
    static constexpr int kWorkgroupsPerCuSingleTensor = kWorkgroupsPerCu;
    static constexpr int kMaxWavesPerSimd = 8;
    static constexpr int kEpl = DTypeInfo<DT>::epl;
    using Raw = MomentumRaw<DT, ECCB, QUANT, KIND_SGD>;
    template <int FAST> __device__ __forceinline__ static void load(const TensorPtrs& t, Where w, Raw& r) {
        momentum_load<DT, ECCB, QUANT, KIND_SGD, FAST>(t, w, r);
    }
    template <int FAST>
    __device__ __forceinline__ static void finish(const TensorPtrs& t, Where w, Raw& r, const Hyper& h, const float*) {
        constexpr int PB = DTypeInfo<DT>::bytes;
#pragma unroll
        for (int i = 0; i < Pack<PB, kEpl>::kDwords; ++i) r.p.w[i] ^= r.g.w[i] & h.mask;
        store_lane<PB, kEpl, FAST>(r.p, t.param, w, t.n);
        store_lane<ECCB, kEpl, FAST>(r.e, t.ecc, w, t.n);
        store_lane<Raw::SB, kEpl, FAST>(r.m, t.mom, w, t.n);
        if constexpr (QUANT) {
            if ((FAST == kVector || w.first() < t.n) && (threadIdx.x & (32 / kEpl - 1)) == 0) store_scale(t.mom_scales, w, r.sm);
        }
    }
};

#endif  // FO_DIAG

}  // namespace fo

namespace {
using namespace fo_host;

template <int DT, int EB, bool Q> using SgdOp = fo::MomentumOp<DT, EB, Q, fo::KIND_SGD>;
template <int DT, int EB, bool Q> using LionOp = fo::MomentumOp<DT, EB, Q, fo::KIND_LION>;
template <int DT, int EB, bool Q> using PlainOp = fo::MomentumOp<DT, EB, Q, fo::KIND_PLAIN>;

using fo::make_momentum_hyper;

}  // namespace

extern "C" {
int fo_momentum_step(void* mom, void* mom_scales, void* param, const void* grad, void* ecc, int64_t n, int dtype,
                     int ecc_bytes, int quantized, float lr, float mom_coef, float update_coef, float weight_decay,
                     int decoupled, int nesterov, int do_lion, void* stream) {
    if (int rc = validate_common(param, grad, ecc, n, dtype, ecc_bytes)) return rc;
    if (n == 0) return 0;  // ref:1551-1553
    if (int rc = validate_state(mom, mom_scales, quantized, dtype, "mom")) return rc;
    fo::TensorPtrs t{param, grad, ecc_bytes ? ecc : nullptr, mom, (uint16_t*)mom_scales, nullptr, nullptr, n};
    SingleLauncher<fo::MomentumHyper> L{t, make_momentum_hyper(lr, mom_coef, update_coef, weight_decay, decoupled, nesterov), (hipStream_t)stream};
    return do_lion ? dispatch<LionOp>(dtype, ecc_bytes, quantized, L) : dispatch<SgdOp>(dtype, ecc_bytes, quantized, L);
}

int fo_sgd_plain_step(void* param, const void* grad, void* ecc, int64_t n, int dtype, int ecc_bytes, float lr,
                      float weight_decay, int decoupled, void* stream) {
    if (int rc = validate_common(param, grad, ecc, n, dtype, ecc_bytes)) return rc;
    if (n == 0) return 0;
    fo::TensorPtrs t{param, grad, ecc_bytes ? ecc : nullptr, nullptr, nullptr, nullptr, nullptr, n};
    SingleLauncher<fo::MomentumHyper> L{t, make_momentum_hyper(lr, 0.0f, 1.0f, weight_decay, decoupled, 0), (hipStream_t)stream};
    return dispatch<PlainOp>(dtype, ecc_bytes, 0, L);
}

int fo_multi_momentum_step(const fo_tensor_desc* descs, int64_t n_tensors, const fo_chunk* chunks, int64_t n_chunks,
                           int dtype, int ecc_bytes, int quantized, float lr, float mom_coef, float update_coef,
                           float weight_decay, int decoupled, int nesterov, int do_lion, void* stream) {
    if (int rc = validate_multi(descs, n_tensors, chunks, n_chunks, dtype, ecc_bytes)) return rc;
    if (n_chunks == 0) return 0;
    MultiLauncher<fo::MomentumHyper> L{descs, n_tensors, chunks, n_chunks, n_chunks, make_momentum_hyper(lr, mom_coef, update_coef, weight_decay, decoupled, nesterov), (hipStream_t)stream};
    return do_lion ? dispatch<LionOp>(dtype, ecc_bytes, quantized, L) : dispatch<SgdOp>(dtype, ecc_bytes, quantized, L);
}

int fo_multi_sgd_plain_step(const fo_tensor_desc* descs, int64_t n_tensors, const fo_chunk* chunks, int64_t n_chunks,
                            int dtype, int ecc_bytes, float lr, float weight_decay, int decoupled, void* stream) {
    if (int rc = validate_multi(descs, n_tensors, chunks, n_chunks, dtype, ecc_bytes)) return rc;
    if (n_chunks == 0) return 0;
    MultiLauncher<fo::MomentumHyper> L{descs, n_tensors, chunks, n_chunks, n_chunks, make_momentum_hyper(lr, 0.0f, 1.0f, weight_decay, decoupled, 0), (hipStream_t)stream};
    return dispatch<PlainOp>(dtype, ecc_bytes, 0, L);
}

#ifdef FO_DIAG
int fo_multi_momentum_streams_copy(const fo_tensor_desc* descs, int64_t n_tensors, const fo_chunk* chunks, int64_t n_chunks,
                                   int dtype, int ecc_bytes, int quantized, void* stream) {
    if (int rc = validate_multi(descs, n_tensors, chunks, n_chunks, dtype, ecc_bytes)) return rc;
    if (n_chunks == 0) return 0;
    MultiLauncher<fo::MomentumStreamsHyper> L{descs, n_tensors, chunks, n_chunks, n_chunks, fo::MomentumStreamsHyper{0u}, (hipStream_t)stream};
    return dispatch<fo::MomentumStreamsOp>(dtype, ecc_bytes, quantized, L);
}

int fo_momentum_step_residency(int dtype, int ecc_bytes, int quantized, int kind, int multi, int* target, int* achieved,
                               int* dynamic_lds) {
    ResidencyQuery q{multi, target, achieved, dynamic_lds};
    if (kind == fo::KIND_LION) return dispatch<LionOp>(dtype, ecc_bytes, quantized, q);
    if (kind == fo::KIND_PLAIN) return dispatch<PlainOp>(dtype, ecc_bytes, 0, q);
    return dispatch<SgdOp>(dtype, ecc_bytes, quantized, q);
}

#endif  // FO_DIAG

}  // extern "C"
