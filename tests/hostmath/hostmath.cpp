// CPU build of the step kernels' arithmetic, for tests only.
//
// This file compiles flashoptim_amd/csrc/fo_math.h -- the very functions the gfx950 kernels call per element --
// for the host and wraps them in loops that mirror the kernels' structure (quantisation groups of 32 elements,
// masked tail elements read as zero, group maxima, code packing).  The instructions the kernels take from the
// hardware (reciprocal, reciprocal root, ldexp, floor-convert, the narrowing conversions) are stand-ins with the
// same contract; fo_math_host_noise != 0 makes the approximate ones err by an ulp.  The tests compare the
// output with the independent IEEE restatement of the reference in oracle/, without a GPU.
//
// Not part of the product: nothing in flashoptim_amd loads this library.
#define FO_MATH_HOST 1
#include "../../flashoptim_amd/csrc/fo_math.h"

#include <stdint.h>
#include <string.h>

extern "C" {
int fo_math_host_noise = 0;
}

namespace {
using namespace fo;

// ---- stand-ins for the conversion instructions (round to nearest even) ----
float bf16_to_f32(uint16_t h) { return as_f32((u32)h << 16); }
uint16_t f32_to_bf16(float f) {
    u32 u = as_u32(f);
    if ((u & 0x7fffffffu) > 0x7f800000u) return (uint16_t)((u >> 16) | 0x0040u);
    u += 0x7fffu + ((u >> 16) & 1u);
    return (uint16_t)(u >> 16);
}
float f16_to_f32(uint16_t h) {
    const u32 sign = (u32)(h & 0x8000u) << 16, e = (h >> 10) & 0x1fu, m = h & 0x3ffu;
    if (e == 0) return as_f32(as_u32((float)m * 0x1p-24f) | sign);
    if (e == 31) return as_f32(sign | 0x7f800000u | (m << 13));
    return as_f32(sign | ((e + 112u) << 23) | (m << 13));
}
uint16_t f32_to_f16(float f) {
    const u32 u = as_u32(f), a = u & 0x7fffffffu;
    const uint16_t sign = (uint16_t)((u >> 16) & 0x8000u);
    if (a > 0x7f800000u) return (uint16_t)(sign | 0x7e00u);
    if (a >= 0x47800000u) return (uint16_t)(sign | 0x7c00u);
    if (a < 0x38800000u) return (uint16_t)(sign | (uint16_t)(as_u32(as_f32(a) + 0.5f) - 0x3f000000u));
    u32 r = a + 0xfffu + ((a >> 13) & 1u);
    return (uint16_t)(sign | (uint16_t)((r - 0x38000000u) >> 13));
}

template <int DT> float load_elem(const void* p, int64_t i) {
    if constexpr (DT == DT_F32) return ((const float*)p)[i];
    if constexpr (DT == DT_BF16) return bf16_to_f32(((const uint16_t*)p)[i]);
    if constexpr (DT == DT_F16) return f16_to_f32(((const uint16_t*)p)[i]);
}
// narrows, stores, returns the stored value widened back
template <int DT> float store_elem(void* p, int64_t i, float v) {
    if constexpr (DT == DT_F32) { ((float*)p)[i] = v; return v; }
    if constexpr (DT == DT_BF16) { const uint16_t h = f32_to_bf16(v); ((uint16_t*)p)[i] = h; return bf16_to_f32(h); }
    if constexpr (DT == DT_F16) { const uint16_t h = f32_to_f16(v); ((uint16_t*)p)[i] = h; return f16_to_f32(h); }
}
template <int ECCB> float load_ecc(const void* e, int64_t i) {
    if constexpr (ECCB == 1) return (float)((const int8_t*)e)[i];
    if constexpr (ECCB == 2) return (float)((const int16_t*)e)[i];
    return 0.0f;
}
template <int ECCB> void store_ecc(void* e, int64_t i, u32 bits) {
    if constexpr (ECCB == 1) ((uint8_t*)e)[i] = (uint8_t)bits;
    if constexpr (ECCB == 2) ((uint16_t*)e)[i] = (uint16_t)bits;
}

constexpr SoftsignTable kTable = SoftsignTable();
template <int DT> constexpr StepTables<DT> kTables = StepTables<DT>();

// as read_master in fo_step.h: int8 codes through the fraction table, int16 codes arithmetically
template <int DT, int ECCB> float read_master(const void* param, const void* ecc, int64_t i) {
    const float w = load_elem<DT>(param, i);
    if constexpr (ECCB == 1) return ecc_join_fraction<DT>(w, kTables<DT>.v[256 * kTableEcc + ((const uint8_t*)ecc)[i]]);
    if constexpr (ECCB == 2) return ecc_join<DT, ECCB>(w, load_ecc<ECCB>(ecc, i));
    return w;
}
template <int DT, int ECCB> void write_master(void* param, void* ecc, int64_t i, float p) {
    const float w = store_elem<DT>(param, i, p);
    if constexpr (ECCB > 0) store_ecc<ECCB>(ecc, i, ecc_split_bits<DT, ECCB, false>(p, w));
}

// the structure of adam_finish (fo_adam.hip), one quantisation group at a time.  `flagged` (may be null) counts the
// elements whose folded update was redone operation by operation.
template <int DT, int ECCB, bool QUANT, bool DECOUPLED, bool EXACT>
void adam_tensor(void* mom, uint16_t* mom_scales, void* var, uint16_t* var_scales, void* param, const void* grad, void* ecc,
                 int64_t n, const AdamHyper& h, int64_t* flagged) {
    for (int64_t g0 = 0; g0 < n; g0 += kGroup) {
        const int cnt = (int)((n - g0) < kGroup ? (n - g0) : kGroup);
        const int64_t group = g0 >> 5;
        float sm = 1.0f, sv = 1.0f;
        if (QUANT) { sm = f16_to_f32(mom_scales[group]); sv = f16_to_f32(var_scales[group]); }
        float m[kGroup], v[kGroup];
        float am = 0.0f, vmax = 0.0f;
        for (int k = 0; k < cnt; ++k) {
            const int64_t i = g0 + k;
            const float p0 = read_master<DT, ECCB>(param, ecc, i);
            float gr = load_elem<DT>(grad, i);
            if (!DECOUPLED) gr = gr + p0 * h.wd;
            float mn, vn;
            if (QUANT) {
                adam_moments_quantized(gr, kTable.v[256 * kTableMom + ((const uint8_t*)mom)[i]], sm, (float)((const uint8_t*)var)[i], sv, h, mn, vn);
            } else {
                adam_moments_plain(gr, load_elem<DT>(mom, i), load_elem<DT>(var, i), h, mn, vn);
            }
            float p;
            if constexpr (EXACT) {
                p = adam_apply_exact(DECOUPLED ? p0 * h.one_m_wd : p0, mn, vn, h);
            } else {
                float slack;
                p = adam_apply_folded<DECOUPLED>(p0, mn, hw::sqrt(vn), h, AdamFoldedGuard<DT, ECCB>::value, slack);
                if (adam_folded_is_flagged(slack)) {
                    p = adam_apply_exact(DECOUPLED ? p0 * h.one_m_wd : p0, mn, vn, h);
                    if (flagged) ++*flagged;
                }
            }
            write_master<DT, ECCB>(param, ecc, i, p);
            m[k] = mn; v[k] = vn;
            am = fmaxf(am, fabsf(mn));
            vmax = fmaxf(vmax, vn);
        }
        if (QUANT) {
            // quick forms, each value verified and redone exactly if it fails (fo_math.h)
            am = fmaxf(am, 1e-12f);
            const float av_quick = fmaxf(hw::sqrt(vmax), 1e-12f);
            const float av = fmaxf(sqrt_corrected(vmax), 1e-12f);
            for (int k = 0; k < cnt; ++k) {
                ((uint8_t*)mom)[g0 + k] = (uint8_t)quantize_mom_code_verified(m[k], am);
                ((uint8_t*)var)[g0 + k] = (uint8_t)quantize_var_code_verified(v[k], av_quick, av);
            }
            mom_scales[group] = f32_to_f16(am);
            var_scales[group] = f32_to_f16(av);
        } else {
            for (int k = 0; k < cnt; ++k) {
                store_elem<DT>(mom, g0 + k, m[k]);
                store_elem<DT>(var, g0 + k, v[k]);
            }
        }
    }
}

// the structure of momentum_finish (fo_momentum.hip)
template <int DT, int ECCB, bool QUANT, int KIND>
void momentum_tensor(void* mom, uint16_t* mom_scales, void* param, const void* grad, void* ecc, int64_t n, const MomentumHyper& h) {
    for (int64_t g0 = 0; g0 < n; g0 += kGroup) {
        const int cnt = (int)((n - g0) < kGroup ? (n - g0) : kGroup);
        const int64_t group = g0 >> 5;
        float sm = 1.0f;
        if (QUANT && KIND != KIND_PLAIN) sm = f16_to_f32(mom_scales[group]);
        float m[kGroup];
        float am = 0.0f;
        for (int k = 0; k < cnt; ++k) {
            const int64_t i = g0 + k;
            float p = read_master<DT, ECCB>(param, ecc, i);
            const float gr = load_elem<DT>(grad, i);
            float mo = 0.0f;
            if (KIND != KIND_PLAIN) mo = QUANT ? kTable.v[256 * kTableMom + ((const uint8_t*)mom)[i]] * sm : load_elem<DT>(mom, i);
            momentum_element<KIND>(gr, p, mo, h, m[k]);
            write_master<DT, ECCB>(param, ecc, i, p);
            am = fmaxf(am, fabsf(m[k]));
        }
        if (KIND == KIND_PLAIN) continue;
        if (QUANT) {
            am = fmaxf(am, 1e-12f);
            const float ram = hw::rcp(am);
            for (int k = 0; k < cnt; ++k)  // as momentum_finish: 2-byte parameters go through the verified quick forms
                ((uint8_t*)mom)[g0 + k] = (uint8_t)(DT == DT_F32 ? quantize_mom_code(m[k], am, ram) : quantize_mom_code_verified(m[k], am));
            mom_scales[group] = f32_to_f16(am);
        } else {
            for (int k = 0; k < cnt; ++k) store_elem<DT>(mom, g0 + k, m[k]);
        }
    }
}

template <template <int, int, bool> class F, class... A> int dispatch(int dtype, int ecc_bytes, int quantized, A... a) {
#define HM_CASE(DT, EB)                                                                        \
    if (dtype == DT && ecc_bytes == EB) {                                                      \
        if (quantized) F<DT, EB, true>::run(a...); else F<DT, EB, false>::run(a...);           \
        return 0;                                                                              \
    }
    HM_CASE(DT_F32, 0)
    HM_CASE(DT_BF16, 0) HM_CASE(DT_BF16, 1) HM_CASE(DT_BF16, 2)
    HM_CASE(DT_F16, 0) HM_CASE(DT_F16, 1) HM_CASE(DT_F16, 2)
#undef HM_CASE
    return -2;
}

template <int DT, int EB, bool Q> struct AdamRun {
    static void run(void* mom, void* ms, void* var, void* vs, void* param, const void* grad, void* ecc, int64_t n,
                    const AdamHyper& h, int decoupled, int exact, int64_t* flagged) {
        // the folded update exists only for the variants that can vouch for it (AdamExact names the others)
        const bool ex = AdamExact<DT, EB>::value || exact > 0 || !h.folded_ok;
        uint16_t* ms16 = (uint16_t*)ms;
        uint16_t* vs16 = (uint16_t*)vs;
        if constexpr (AdamExact<DT, EB>::value) {
            if (decoupled) adam_tensor<DT, EB, Q, true, true>(mom, ms16, var, vs16, param, grad, ecc, n, h, flagged);
            else adam_tensor<DT, EB, Q, false, true>(mom, ms16, var, vs16, param, grad, ecc, n, h, flagged);
        } else {
            if (decoupled) {
                if (ex) adam_tensor<DT, EB, Q, true, true>(mom, ms16, var, vs16, param, grad, ecc, n, h, flagged);
                else adam_tensor<DT, EB, Q, true, false>(mom, ms16, var, vs16, param, grad, ecc, n, h, flagged);
            } else {
                if (ex) adam_tensor<DT, EB, Q, false, true>(mom, ms16, var, vs16, param, grad, ecc, n, h, flagged);
                else adam_tensor<DT, EB, Q, false, false>(mom, ms16, var, vs16, param, grad, ecc, n, h, flagged);
            }
        }
    }
};
template <int DT, int EB, bool Q> struct MomentumRun {
    static void run(void* mom, void* ms, void* param, const void* grad, void* ecc, int64_t n, const MomentumHyper& h, int kind) {
        if (kind == KIND_LION) momentum_tensor<DT, EB, Q, KIND_LION>(mom, (uint16_t*)ms, param, grad, ecc, n, h);
        else if (kind == KIND_PLAIN) momentum_tensor<DT, EB, Q, KIND_PLAIN>(mom, (uint16_t*)ms, param, grad, ecc, n, h);
        else momentum_tensor<DT, EB, Q, KIND_SGD>(mom, (uint16_t*)ms, param, grad, ecc, n, h);
    }
};

}  // namespace

extern "C" {

void hm_set_noise(int v) { fo_math_host_noise = v; }

// Arguments as fo_adam_step (include/flashoptim_hip.h) without the stream; host pointers.
// exact: <= 0 = the choice the kernels make for this variant (fo_adam_step), 1 = operation by operation on every
// element (fo_adam_step_exact).  flagged (may be null): receives the number of elements whose folded update was
// redone operation by operation.
int hm_adam_step(void* mom, void* mom_scales, void* var, void* var_scales, void* param, const void* grad, void* ecc,
                 int64_t n, int dtype, int ecc_bytes, int quantized, float lr, float beta1, float beta2, float eps,
                 float weight_decay, int decoupled, int step, int exact, int64_t* flagged) {
    const AdamHyper h = make_adam_hyper(lr, beta1, beta2, eps, weight_decay, step);
    if (flagged) *flagged = 0;
    return dispatch<AdamRun>(dtype, ecc_bytes, quantized, mom, mom_scales, var, var_scales, param, grad, ecc, n, h, decoupled, exact, flagged);
}
// The folded update of bf16 parameters with a 1-byte ECC and quantised states WITHOUT the repair: the fp32 results
// and which elements the guard flags.  Changes nothing in place.
void hm_adam_folded_update(const void* mom, const void* mom_scales, const void* var, const void* var_scales, const void* param,
                           const void* grad, const void* ecc, int64_t n, float lr, float beta1, float beta2, float eps,
                           float weight_decay, int decoupled, int step, float* p_out, uint8_t* redo_out) {
    const AdamHyper h = make_adam_hyper(lr, beta1, beta2, eps, weight_decay, step);
    for (int64_t i = 0; i < n; ++i) {
        const float sm = f16_to_f32(((const uint16_t*)mom_scales)[i >> 5]), sv = f16_to_f32(((const uint16_t*)var_scales)[i >> 5]);
        const float p0 = read_master<DT_BF16, 1>(param, ecc, i);
        float gr = load_elem<DT_BF16>(grad, i);
        if (!decoupled) gr = gr + p0 * h.wd;
        float mn, vn;
        adam_moments_quantized(gr, kTable.v[256 * kTableMom + ((const uint8_t*)mom)[i]], sm, (float)((const uint8_t*)var)[i], sv, h, mn, vn);
        float slack;
        p_out[i] = decoupled ? adam_apply_folded<true>(p0, mn, hw::sqrt(vn), h, AdamFoldedGuard<DT_BF16, 1>::value, slack)
                             : adam_apply_folded<false>(p0, mn, hw::sqrt(vn), h, AdamFoldedGuard<DT_BF16, 1>::value, slack);
        redo_out[i] = adam_folded_is_flagged(slack) ? 1 : 0;
    }
}
void hm_code_over_255(float* out) { for (int q = 0; q < 256; ++q) out[q] = code_over_255((float)q); }

// Arguments as fo_momentum_step without the stream.
int hm_momentum_step(void* mom, void* mom_scales, void* param, const void* grad, void* ecc, int64_t n, int dtype,
                     int ecc_bytes, int quantized, float lr, float mom_coef, float update_coef, float weight_decay,
                     int decoupled, int nesterov, int do_lion) {
    const MomentumHyper h = make_momentum_hyper(lr, mom_coef, update_coef, weight_decay, decoupled, nesterov);
    return dispatch<MomentumRun>(dtype, ecc_bytes, quantized, mom, mom_scales, param, grad, ecc, n, h, do_lion ? KIND_LION : KIND_SGD);
}

int hm_sgd_plain_step(void* param, const void* grad, void* ecc, int64_t n, int dtype, int ecc_bytes, float lr,
                      float weight_decay, int decoupled) {
    const MomentumHyper h = make_momentum_hyper(lr, 0.0f, 1.0f, weight_decay, decoupled, 0);
    return dispatch<MomentumRun>(dtype, ecc_bytes, 0, (void*)nullptr, (void*)nullptr, param, grad, ecc, n, h, (int)KIND_PLAIN);
}

// element-wise helpers, for direct tests of the correction steps
void hm_div_corrected(const float* a, const float* b, float* out, int64_t n) {
    for (int64_t i = 0; i < n; ++i) out[i] = div_corrected(a[i], b[i], hw::rcp(b[i]));
}
void hm_sqrt_corrected(const float* x, float* out, int64_t n) {
    for (int64_t i = 0; i < n; ++i) out[i] = sqrt_corrected(x[i]);
}
void hm_quantize_group(const float* m, const float* r, uint8_t* qm, uint8_t* qv, int64_t n) {  // n values = one group each way
    float am = 0.0f, av = 0.0f;
    for (int64_t i = 0; i < n; ++i) { am = fmaxf(am, fabsf(m[i])); av = fmaxf(av, r[i]); }
    am = fmaxf(am, 1e-12f); av = fmaxf(av, 1e-12f);
    const float ram = hw::rcp(am), rav = hw::rcp(av);
    for (int64_t i = 0; i < n; ++i) { qm[i] = (uint8_t)quantize_mom_code(m[i], am, ram); qv[i] = (uint8_t)quantize_var_code(r[i], av, rav); }
}
// table [256 + b] against the arithmetic form, for every byte
void hm_ecc_fraction_table(int dtype, float* table_out, float* arithmetic_out) {
    for (int b = 0; b < 256; ++b) {
        const float q = (float)(int8_t)b;
        if (dtype == DT_BF16) { table_out[b] = kTables<DT_BF16>.v[256 * kTableEcc + b]; arithmetic_out[b] = ecc_fraction<DT_BF16, 1>(q); }
        else { table_out[b] = kTables<DT_F16>.v[256 * kTableEcc + b]; arithmetic_out[b] = ecc_fraction<DT_F16, 1>(q); }
    }
}
// codes of one group from its first-moment values m and second-moment values v: through the quick forms with
// verification (quick != 0) or through the exact forms alone; also how many values failed the margin test
int64_t hm_quantize_group_from_moments(const float* m, const float* v, int8_t* qm, uint8_t* qv, int64_t n, int quick) {
    float am = 0.0f, vmax = 0.0f;
    for (int64_t i = 0; i < n; ++i) { am = fmaxf(am, fabsf(m[i])); vmax = fmaxf(vmax, v[i]); }
    am = fmaxf(am, 1e-12f);
    const float av_quick = fmaxf(hw::sqrt(vmax), 1e-12f), av = fmaxf(sqrt_corrected(vmax), 1e-12f);
    const float ram = hw::rcp(am), rav = hw::rcp(av);
    int64_t failed = 0;
    for (int64_t i = 0; i < n; ++i) {
        if (quick) {
            qm[i] = (int8_t)quantize_mom_code_verified(m[i], am);
            qv[i] = (uint8_t)quantize_var_code_verified(v[i], av_quick, av);
            failed += !quick_value_is_safe(quantize_mom_quick(m[i], am), kQuickMarginMom);
            failed += !quick_value_is_safe(quantize_var_quick(hw::sqrt(v[i]), hw::rcp(av_quick) * 255.0f), kQuickMarginVar);
        } else {
            qm[i] = (int8_t)quantize_mom_code(m[i], am, ram);
            qv[i] = (uint8_t)quantize_var_code(sqrt_corrected(v[i]), av, rav);
        }
    }
    return failed;
}
void hm_softsign_table(float* out) { for (int b = 0; b < 256; ++b) out[b] = kTable.v[256 * kTableMom + b]; }

int hm_ecc_join(const void* narrow, int narrow_dtype, const void* ecc, int ecc_bytes, float* out, int64_t n) {
    for (int64_t i = 0; i < n; ++i) {
        if (narrow_dtype == DT_BF16 && ecc_bytes == 1) out[i] = read_master<DT_BF16, 1>(narrow, ecc, i);
        else if (narrow_dtype == DT_BF16 && ecc_bytes == 2) out[i] = read_master<DT_BF16, 2>(narrow, ecc, i);
        else if (narrow_dtype == DT_F16 && ecc_bytes == 1) out[i] = read_master<DT_F16, 1>(narrow, ecc, i);
        else if (narrow_dtype == DT_F16 && ecc_bytes == 2) out[i] = read_master<DT_F16, 2>(narrow, ecc, i);
        else return -2;
    }
    return 0;
}
// clamp != 0: the standalone form (any narrow value); 0: the fused kernels' form (narrow is the rounding of x)
int hm_ecc_split(const float* x, const void* narrow, int narrow_dtype, void* ecc, int ecc_bytes, int64_t n, int clamp) {
    for (int64_t i = 0; i < n; ++i) {
        u32 b;
        if (narrow_dtype == DT_BF16) {
            const float w = load_elem<DT_BF16>(narrow, i);
            if (ecc_bytes == 1) b = clamp ? ecc_split_bits<DT_BF16, 1, true>(x[i], w) : ecc_split_bits<DT_BF16, 1, false>(x[i], w);
            else b = clamp ? ecc_split_bits<DT_BF16, 2, true>(x[i], w) : ecc_split_bits<DT_BF16, 2, false>(x[i], w);
        } else if (narrow_dtype == DT_F16) {
            const float w = load_elem<DT_F16>(narrow, i);
            if (ecc_bytes == 1) b = clamp ? ecc_split_bits<DT_F16, 1, true>(x[i], w) : ecc_split_bits<DT_F16, 1, false>(x[i], w);
            else b = clamp ? ecc_split_bits<DT_F16, 2, true>(x[i], w) : ecc_split_bits<DT_F16, 2, false>(x[i], w);
        } else return -2;
        if (ecc_bytes == 1) ((uint8_t*)ecc)[i] = (uint8_t)b; else ((uint16_t*)ecc)[i] = (uint16_t)b;
    }
    return 0;
}

}  // extern "C"
