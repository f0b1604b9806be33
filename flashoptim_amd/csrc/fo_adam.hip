// Fused Adam / AdamW step kernel for gfx950 and its C entry points (ref: /root/reference/flashoptim/
// optimizers.py:2203-2438, cited as "ref:").
#include "fo_step.h"

#include <cmath>

namespace fo {

// ------------------------------------------------------------------------------------------------
// Adam / AdamW (ref:2255-2438)
// ------------------------------------------------------------------------------------------------
struct AdamHyper {
    float b1, one_m_b1, b2, one_m_b2, wd, one_m_wd;
    float lr_over_bc1;   // lr / (1 - b1^step)
    float rsqrt_bc2;     // 1 / sqrt(1 - b2^step)
    float eps;
};

template <int DT, int ECCB, bool QUANT, bool DECOUPLED, bool FAST>
__device__ __forceinline__ void adam_lane(const TensorPtrs& t, int64_t first, const AdamHyper& h,
                                          const float* lut_lane) {
    constexpr int PB = DTypeInfo<DT>::bytes;
    constexpr int SB = QUANT ? 1 : PB;  // state bytes per element
    const int64_t n = t.n;

    Pack<PB> praw, graw;
    Pack<ECCB> eraw;
    Pack<SB> mraw, vraw;
    load_lane<PB, FAST>(graw, t.grad, first, n);
    load_lane<PB, FAST>(praw, t.param, first, n);
    load_lane<ECCB, FAST>(eraw, t.ecc, first, n);
    load_lane<SB, FAST>(mraw, t.mom, first, n);
    load_lane<SB, FAST>(vraw, t.var, first, n);
    const bool live_group = FAST || first < n;  // the lane owns at least one real element
    const int64_t group = first >> 5;
    float sm = 1.0f, sv = 1.0f;  // masked scales read 1.0 (ref:2318-2323)
    if constexpr (QUANT) {
        if (live_group) {
            sm = f16_bits_to_f32(t.mom_scales[group]);
            sv = f16_bits_to_f32(t.var_scales[group]);
        }
    }

    float p[kLaneElems], m[kLaneElems], r[kLaneElems], v[kLaneElems];
    read_master<DT, ECCB>(p, praw, eraw);

    float am = 0.0f, vm = 0.0f;
#pragma unroll
    for (int k = 0; k < kLaneElems; ++k) {
        float g = widen<DT>(graw, k);
        if constexpr (!DECOUPLED) g = g + p[k] * h.wd;                                   // ref:2310-2311
        float mo, vo;
        if constexpr (QUANT) {
            mo = lut_lane[byte_of(mraw, k) * 32] * sm;                           // ref:2332-2343
            const float s = code255_to_unit((float)byte_of(vraw, k)) * sv;       // ref:2333-2346
            vo = s * s;                                                          // ref:2348
        } else {
            mo = widen<DT>(mraw, k);                                             // ref:2351-2354
            vo = widen<DT>(vraw, k);
        }
        const float mn = mo * h.b1 + g * h.one_m_b1;                             // ref:2357
        const float vn = vo * h.b2 + (g * g) * h.one_m_b2;                       // ref:2360
        float pk = p[k];
        if constexpr (DECOUPLED) pk = pk * h.one_m_wd;                                   // ref:2363-2364
        // p -= lr * (m/bc1) / (sqrt(v/bc2) + eps)  (ref:2368-2375), with sqrt(v) shared with the requantiser
        const float rk = __builtin_amdgcn_sqrtf(vn);
        const float den = fmaf(rk, h.rsqrt_bc2, h.eps);
        pk = fmaf(-(h.lr_over_bc1 * mn), __builtin_amdgcn_rcpf(den), pk);
        p[k] = pk; m[k] = mn; r[k] = rk; v[k] = vn;
        am = fmaxf(am, fabsf(mn));
        vm = fmaxf(vm, vn);
    }

    Pack<ECCB> eout;
    write_master<DT, ECCB>(p, praw, eout);
    store_lane<PB, FAST>(praw, t.param, first, n);
    store_lane<ECCB, FAST>(eout, t.ecc, first, n);

    if constexpr (QUANT) {
        // group absmax over the lane pair (ref:2399-2404); sqrt is monotone, so the absmax of sqrt(v) is the
        // correctly rounded root of max(v)
        am = fmaxf(fmaxf(am, pair_swap(am)), 1e-12f);
        vm = fmaxf(vm, pair_swap(vm));
        const float av = fmaxf(sqrt_rn(vm), 1e-12f);
        quantize_mom(m, am, mraw);
        quantize_var(r, av, vraw);
        store_lane<1, FAST>(mraw, t.mom, first, n);
        store_lane<1, FAST>(vraw, t.var, first, n);
        if (live_group && (threadIdx.x & 1) == 0) {                              // ref:2424-2434
            t.mom_scales[group] = f32_to_f16_bits(am);
            t.var_scales[group] = f32_to_f16_bits(av);
        }
    } else {
        narrow_all<DT>(m, mraw);                                                 // ref:2435-2438
        narrow_all<DT>(v, vraw);
        store_lane<SB, FAST>(mraw, t.mom, first, n);
        store_lane<SB, FAST>(vraw, t.var, first, n);
    }
}


template <int DT, int ECCB, bool QUANT, bool DECOUPLED> struct AdamOp {
    using Hyper = AdamHyper;
    static constexpr bool kNeedsLut = QUANT;
    template <bool FAST>
    __device__ __forceinline__ static void lane(const TensorPtrs& t, int64_t first, const Hyper& h, const float* lut) {
        adam_lane<DT, ECCB, QUANT, DECOUPLED, FAST>(t, first, h, lut);
    }
};

}  // namespace fo

namespace {
using namespace fo_host;

template <int DT, int EB, bool Q> using AdamL2Op = fo::AdamOp<DT, EB, Q, false>;  // FlashAdam: decay folded into the gradient
template <int DT, int EB, bool Q> using AdamWOp = fo::AdamOp<DT, EB, Q, true>;    // FlashAdamW: decay applied to the weights

fo::AdamHyper make_adam_hyper(float lr, float beta1, float beta2, float eps, float wd, int step) {
    // Scalars arrive as fp32 like the reference's kernel arguments; 1 - x is formed in fp32 (ref:2357-2364).
    // beta^step is the correctly rounded fp32 power; the bias corrections are folded into two per-launch
    // factors in double and rounded once.
    fo::AdamHyper h;
    h.b1 = beta1; h.one_m_b1 = 1.0f - beta1;
    h.b2 = beta2; h.one_m_b2 = 1.0f - beta2;
    h.wd = wd; h.one_m_wd = 1.0f - wd;
    const float bc1 = 1.0f - (float)std::pow((double)beta1, (double)step);
    const float bc2 = 1.0f - (float)std::pow((double)beta2, (double)step);
    h.lr_over_bc1 = (float)((double)lr / (double)bc1);
    h.rsqrt_bc2 = (float)(1.0 / std::sqrt((double)bc2));
    h.eps = eps;
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
