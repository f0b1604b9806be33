// Fused Adam / AdamW step kernel for gfx950 and its C entry points (ref: /root/reference/flashoptim/
// optimizers.py:2203-2438, cited as "ref:").
#include "fo_step.h"

#include <cmath>
#include <limits>

namespace fo {

// Per-launch constants.  Scalars arrive as fp32 like the reference's kernel arguments; 1 - x is formed in fp32
// (ref:2357-2364).  The per-step bias corrections and the learning rate are folded on the host (in double,
// rounded once) into the two constants of the update's denominator:
//     lr * (m / bc1) / (sqrt(v / bc2) + eps)  ==  m / (sqrt(v) * den_scale + den_bias)
//     den_scale = bc1 / (lr * sqrt(bc2)),  den_bias = eps * bc1 / lr
struct AdamHyper {
    float b1, one_m_b1, one_m_b2, wd, one_m_wd;
    float sqrt_b2_over_255;  // dequantised sqrt(v_old * b2) = code * scale * sqrt(b2) / 255
    float b2;                // unquantised states only
    float den_scale, den_bias;
};

// What a lane holds between issuing its loads and consuming them.
template <int DT, int ECCB, bool QUANT> struct AdamRaw {
    static constexpr int EPL = DTypeInfo<DT>::epl;
    Pack<DTypeInfo<DT>::bytes, EPL> p, g;
    Pack<ECCB, EPL> e;
    Pack<QUANT ? 1 : DTypeInfo<DT>::bytes, EPL> m, v;
    uint16_t sm, sv;
};

template <int DT, int ECCB, bool QUANT, int FAST>
__device__ __forceinline__ void adam_load(const TensorPtrs& t, int64_t first, AdamRaw<DT, ECCB, QUANT>& r) {
    constexpr int EPL = DTypeInfo<DT>::epl;
    constexpr int PB = DTypeInfo<DT>::bytes;
    constexpr int SB = QUANT ? 1 : PB;  // state bytes per element
    const int64_t n = t.n;
    load_lane<PB, EPL, FAST>(r.g, t.grad, first, n);
    load_lane<PB, EPL, FAST>(r.p, t.param, first, n);
    load_lane<ECCB, EPL, FAST>(r.e, t.ecc, first, n);
    load_lane<SB, EPL, FAST>(r.m, t.mom, first, n);
    load_lane<SB, EPL, FAST>(r.v, t.var, first, n);
    r.sm = r.sv = 0x3c00;  // masked scales read 1.0 (ref:2318-2323)
    if constexpr (QUANT) {
        if (FAST == kVector || first < n) {
            r.sm = t.mom_scales[first >> 5];
            r.sv = t.var_scales[first >> 5];
        }
    }
}

template <int DT, int ECCB, bool QUANT, bool DECOUPLED, int FAST>
__device__ __forceinline__ void adam_finish(const TensorPtrs& t, int64_t first, AdamRaw<DT, ECCB, QUANT>& raw,
                                            const AdamHyper& h, const float* lut_lane) {
    constexpr int EPL = DTypeInfo<DT>::epl;
    constexpr int PB = DTypeInfo<DT>::bytes;
    constexpr int SB = QUANT ? 1 : PB;
    const int64_t n = t.n;
    const bool live_group = FAST == kVector || first < n;  // the lane owns at least one real element
    const int64_t group = first >> 5;
    // the EMA decay is folded into the group scale: one multiply per lane instead of one per element
    const float sm_b1 = f16_bits_to_f32(raw.sm) * h.b1;
    const float sv_b2 = f16_bits_to_f32(raw.sv) * h.sqrt_b2_over_255;

    float p[EPL], m[EPL], r[EPL], v[EPL];
    read_master<DT, ECCB, EPL>(p, raw.p, raw.e);

    float am = 0.0f, vm = 0.0f;
#pragma unroll
    for (int k = 0; k < EPL; ++k) {
        float g = widen<DT, EPL>(raw.g, k);
        if constexpr (!DECOUPLED) g = g + p[k] * h.wd;                              // ref:2310-2311
        float mn, vn;
        if constexpr (QUANT) {
            // m = dequant(m) * b1 + g * (1 - b1)   (ref:2332-2343, 2357)
            mn = fmaf(StepLut::lookup(lut_lane, byte_of<EPL>(raw.m, k)), sm_b1, g * h.one_m_b1);
            // v = dequant(v) * b2 + g^2 * (1 - b2), dequant(v) = (code/255 * scale)^2   (ref:2333-2348, 2360)
            const float s = (float)byte_of<EPL>(raw.v, k) * sv_b2;
            vn = fmaf(s, s, (g * g) * h.one_m_b2);
        } else {
            // unquantised states: operation by operation as written in the reference, no contraction
            mn = widen<DT, EPL>(raw.m, k) * h.b1 + g * h.one_m_b1;                   // ref:2351-2357
            vn = widen<DT, EPL>(raw.v, k) * h.b2 + (g * g) * h.one_m_b2;             // ref:2360
        }
        float pk = p[k];
        if constexpr (DECOUPLED) pk = pk * h.one_m_wd;                              // ref:2363-2364
        // p -= lr * (m/bc1) / (sqrt(v/bc2) + eps)  (ref:2368-2375); sqrt(v) is shared with the requantiser
        const float rk = __builtin_amdgcn_sqrtf(vn);
        const float den = fmaf(rk, h.den_scale, h.den_bias);
        pk = fmaf(-mn, __builtin_amdgcn_rcpf(den), pk);
        p[k] = pk; m[k] = mn; r[k] = rk; v[k] = vn;
    }
#pragma unroll
    for (int k = 0; k < EPL; k += 2) {  // pairs, so that each step is one three-operand max
        am = fmaxf(fmaxf(am, fabsf(m[k])), fabsf(m[k + 1]));
        vm = fmaxf(fmaxf(vm, v[k]), v[k + 1]);
    }

    Pack<ECCB, EPL> eout;
    write_master<DT, ECCB, EPL>(p, raw.p, eout);
    store_lane<PB, EPL, FAST>(raw.p, t.param, first, n);
    store_lane<ECCB, EPL, FAST>(eout, t.ecc, first, n);

    if constexpr (QUANT) {
        // group absmax (ref:2399-2404); sqrt is monotone, so the absmax of sqrt(v) is the correctly rounded
        // root of max(v)
        am = fmaxf(group_max<EPL>(am), 1e-12f);
        const float av = fmaxf(sqrt_rn(group_max<EPL>(vm)), 1e-12f);
        quantize_mom<EPL>(m, am, raw.m);
        quantize_var<EPL>(r, av, raw.v);
        store_lane<1, EPL, FAST>(raw.m, t.mom, first, n);
        store_lane<1, EPL, FAST>(raw.v, t.var, first, n);
        if (live_group && (threadIdx.x & (32 / EPL - 1)) == 0) {                    // ref:2424-2434
            store_scale(t.mom_scales, group, f32_to_f16_bits(am));
            store_scale(t.var_scales, group, f32_to_f16_bits(av));
        }
    } else {
        narrow_all<DT, EPL>(m, raw.m);                                              // ref:2435-2438
        narrow_all<DT, EPL>(v, raw.v);
        store_lane<SB, EPL, FAST>(raw.m, t.mom, first, n);
        store_lane<SB, EPL, FAST>(raw.v, t.var, first, n);
    }
}

template <int DT, int ECCB, bool QUANT, bool DECOUPLED> struct AdamOp {
    using Hyper = AdamHyper;
    static constexpr bool kNeedsLut = QUANT;
    // measured on MI355X with the 8B-parameter step: 14-15 resident workgroups per compute unit for 2-byte
    // parameters with no or a 1-byte ECC (3.6-4.1 KiB of loads per wavefront), 13 with a 2-byte ECC (4.6 KiB),
    // 16-20 for fp32 parameters (2.5 KiB)
    static constexpr int kLdsBytes = DT == DT_F32 ? 9216 : (ECCB == 2 ? 12288 : 11008);
    static constexpr int kEpl = DTypeInfo<DT>::epl;
    using Raw = AdamRaw<DT, ECCB, QUANT>;
    template <int FAST> __device__ __forceinline__ static void load(const TensorPtrs& t, int64_t first, Raw& r) {
        adam_load<DT, ECCB, QUANT, FAST>(t, first, r);
    }
    template <int FAST>
    __device__ __forceinline__ static void finish(const TensorPtrs& t, int64_t first, Raw& r, const Hyper& h, const float* lut) {
        adam_finish<DT, ECCB, QUANT, DECOUPLED, FAST>(t, first, r, h, lut);
    }
};

}  // namespace fo

namespace {
using namespace fo_host;

template <int DT, int EB, bool Q> using AdamL2Op = fo::AdamOp<DT, EB, Q, false>;  // FlashAdam: decay folded into the gradient
template <int DT, int EB, bool Q> using AdamWOp = fo::AdamOp<DT, EB, Q, true>;    // FlashAdamW: decay applied to the weights

fo::AdamHyper make_adam_hyper(float lr, float beta1, float beta2, float eps, float wd, int step) {
    fo::AdamHyper h;
    h.b1 = beta1; h.one_m_b1 = 1.0f - beta1;
    h.b2 = beta2; h.one_m_b2 = 1.0f - beta2;
    h.wd = wd; h.one_m_wd = 1.0f - wd;
    h.sqrt_b2_over_255 = (float)(std::sqrt((double)beta2) / 255.0);
    // beta^step is the correctly rounded fp32 power, 1 - that is formed in fp32 (ref:2368-2369)
    const double bc1 = (double)(1.0f - (float)std::pow((double)beta1, (double)step));
    const double bc2 = (double)(1.0f - (float)std::pow((double)beta2, (double)step));
    if (lr != 0.0f) {
        h.den_scale = (float)(bc1 / ((double)lr * std::sqrt(bc2)));
        h.den_bias = (float)((double)eps * bc1 / (double)lr);
    } else {  // no update: the denominator is infinite whatever sqrt(v) is
        h.den_scale = 0.0f;
        h.den_bias = std::numeric_limits<float>::infinity();
    }
    return h;
}

}  // namespace

extern "C" {

int fo_adam_step(void* mom, void* mom_scales, void* var, void* var_scales, void* param, const void* grad, void* ecc,
                 int64_t n, int dtype, int ecc_bytes, int quantized, float lr, float beta1, float beta2, float eps,
                 float weight_decay, int decoupled, int step, void* stream) {
    if (int rc = validate_common(param, grad, ecc, n, dtype, ecc_bytes)) return rc;
    if (n == 0) return 0;  // ref:2221-2223
    if (step < 1) return fail(FO_ERR_INVALID_ARGUMENT, "step must be >= 1 (got %d)", step);
    if (int rc = validate_state(mom, mom_scales, quantized, dtype, "mom")) return rc;
    if (int rc = validate_state(var, var_scales, quantized, dtype, "var")) return rc;
    fo::TensorPtrs t{param, grad, ecc_bytes ? ecc : nullptr, mom, (uint16_t*)mom_scales, var, (uint16_t*)var_scales, n};
    SingleLauncher<fo::AdamHyper> L{t, make_adam_hyper(lr, beta1, beta2, eps, weight_decay, step), (hipStream_t)stream};
    return decoupled ? dispatch<AdamWOp>(dtype, ecc_bytes, quantized, L) : dispatch<AdamL2Op>(dtype, ecc_bytes, quantized, L);
}

int fo_multi_adam_step(const fo_tensor_desc* descs, int64_t n_tensors, const fo_chunk* chunks, int64_t n_chunks, int dtype,
                       int ecc_bytes, int quantized, float lr, float beta1, float beta2, float eps, float weight_decay,
                       int decoupled, int step, void* stream) {
    if (int rc = validate_multi(descs, n_tensors, chunks, n_chunks, dtype, ecc_bytes)) return rc;
    if (n_chunks == 0) return 0;
    if (step < 1) return fail(FO_ERR_INVALID_ARGUMENT, "step must be >= 1 (got %d)", step);
    MultiLauncher<fo::AdamHyper> L{descs, chunks, n_chunks, make_adam_hyper(lr, beta1, beta2, eps, weight_decay, step), (hipStream_t)stream};
    return decoupled ? dispatch<AdamWOp>(dtype, ecc_bytes, quantized, L) : dispatch<AdamL2Op>(dtype, ecc_bytes, quantized, L);
}

}  // extern "C"
