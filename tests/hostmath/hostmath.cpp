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

// ------------------------------------------------------------------------------------------------
// a simulated wavefront: 64 lane states, the flows of fo_math.h run over it unchanged
// ------------------------------------------------------------------------------------------------
constexpr int kLanes = 64;

struct FlowStats {   // what the flows did, for the tests
    int64_t waves = 0;            // wavefronts stepped
    int64_t questions = 0;        // wave.any() calls: one per flow and wavefront, plus one per position once a flow repairs
    int64_t yes = 0;              // those answered with yes
    int64_t codes_replaced = 0;   // set_*_code calls
};
FlowStats g_stats;

template <class Lane> struct SimWave {
    Lane* lanes;
    template <class F> void each(F&& f) { for (int i = 0; i < kLanes; ++i) f(lanes[i]); }
    // every lane evaluates the predicate (no short circuit), as under a ballot
    template <class P> bool any(P&& p) {
        bool r = false;
        for (int i = 0; i < kLanes; ++i) r = p(const_cast<const Lane&>(lanes[i])) || r;
        ++g_stats.questions;
        g_stats.yes += r;
        return r;
    }
};

// lane states with the members the flows ask for; codes as plain integers (the kernels keep them packed)
template <int N> struct MomLane {
    float m[N], am = 1e-12f, x[N], slack[N], least = 0.0f, ram = 0.0f;
    u32 code[N];
    void convert_mom(const float (&q)[N]) { for (int k = 0; k < N; ++k) code[k] = (u32)hw::floor_to_int(q[k]) & 0xffu; }
    void set_mom_code(int k, u32 c) { code[k] = c & 0xffu; ++g_stats.codes_replaced; }
};
template <int N> struct VarLane {
    float v[N], r[N], av_quick = 1e-12f, av = 1e-12f, x[N], slack[N], least = 0.0f, rav = 0.0f;
    u32 code[N];
    void convert_var(const float (&q)[N]) { for (int k = 0; k < N; ++k) code[k] = (u32)(int)q[k] & 0xffu; }
    void set_var_code(int k, u32 c) { code[k] = c & 0xffu; ++g_stats.codes_replaced; }
};
template <int N> struct BothLane {
    float m[N], am = 1e-12f, v[N], r[N], av_quick = 1e-12f, av = 1e-12f;
    float xm[N], xv[N], slack_m[N], slack_v[N], least_m = 0.0f, least_v = 0.0f, ram = 0.0f, rav = 0.0f;
    u32 mcode[N], vcode[N];
    void convert_both(const float (&qm)[N], const float (&qv)[N]) {
        for (int k = 0; k < N; ++k) { mcode[k] = (u32)hw::floor_to_int(qm[k]) & 0xffu; vcode[k] = (u32)(int)qv[k] & 0xffu; }
    }
    void set_mom_code(int k, u32 c) { mcode[k] = c & 0xffu; ++g_stats.codes_replaced; }
    void set_var_code(int k, u32 c) { vcode[k] = c & 0xffu; ++g_stats.codes_replaced; }
};
template <int N> struct RedoLane {
    float p[N], slack[N], m[N], v[N], p_old[N], least = 0.0f;
    float old_master(int k) const { return p_old[k]; }
};

// One moment's requantisation for a wavefront of lanes that hold N values each; lanes_per_group lanes share a
// quantisation group.  m / v: kLanes * N values in lane order; live[l]: the lane owns at least one real element.
// Writes the codes and (for lanes that lead a group) the fp16 scales.
template <int N> void group_scales(const float* lane_am, const float* lane_vmax, float* am, float* av_quick, float* av) {
    constexpr int per_group = kGroup / N;
    for (int g0 = 0; g0 < kLanes; g0 += per_group) {
        float a = 0.0f, vm = 0.0f;
        for (int l = g0; l < g0 + per_group; ++l) { a = fmaxf(a, lane_am[l]); vm = fmaxf(vm, lane_vmax[l]); }
        for (int l = g0; l < g0 + per_group; ++l) {
            am[l] = fmaxf(a, 1e-12f);
            av_quick[l] = fmaxf(hw::sqrt(vm), 1e-12f);
            av[l] = fmaxf(sqrt_corrected(vm), 1e-12f);
        }
    }
}

// The structure of adam_finish (fo_adam.hip): one wavefront = kLanes lanes x EPL consecutive elements; lane l owns
// elements [l * EPL, (l + 1) * EPL) of the span, elements past the end read as zero (scales as 1.0) and are never
// stored.  `flagged` (may be null) counts the elements whose folded update was redone operation by operation.
template <int DT, int ECCB, bool QUANT, bool DECOUPLED, bool EXACT>
void adam_tensor(void* mom, uint16_t* mom_scales, void* var, uint16_t* var_scales, void* param, const void* grad, void* ecc,
                 int64_t n, const AdamHyper& h, int64_t* flagged) {
    constexpr int EPL = DTypeInfo<DT>::epl;
    constexpr int kSpan = kLanes * EPL;
    static RedoLane<EPL> redo[kLanes];
    static MomLane<EPL> ml[kLanes];
    static VarLane<EPL> vl[kLanes];
    static BothLane<EPL> bl[kLanes];
    for (int64_t base = 0; base < n; base += kSpan) {
        ++g_stats.waves;
        float lane_am[kLanes], lane_vmax[kLanes], r[kLanes][EPL];
        for (int l = 0; l < kLanes; ++l) {
            const int64_t first = base + (int64_t)l * EPL;
            const bool live = first < n;
            float sm = 1.0f, sv = 1.0f;                                       // masked scales read 1.0 (ref:2318-2323)
            if (QUANT && live) { sm = f16_to_f32(mom_scales[first >> 5]); sv = f16_to_f32(var_scales[first >> 5]); }
            lane_am[l] = lane_vmax[l] = 0.0f;
            for (int k = 0; k < EPL; ++k) {
                const int64_t i = first + k;
                const bool in = i < n;
                const float p0 = in ? read_master<DT, ECCB>(param, ecc, i) : 0.0f;
                float gr = in ? load_elem<DT>(grad, i) : 0.0f;
                if (!DECOUPLED) gr = gr + p0 * h.wd;
                float mn, vn;
                if (QUANT) {
                    adam_moments_quantized(gr, kTable.v[256 * kTableMom + (in ? ((const uint8_t*)mom)[i] : 0)], sm,
                                           in ? (float)((const uint8_t*)var)[i] : 0.0f, sv, h, mn, vn);
                } else {
                    adam_moments_plain(gr, in ? load_elem<DT>(mom, i) : 0.0f, in ? load_elem<DT>(var, i) : 0.0f, h, mn, vn);
                }
                const float rk = (QUANT || !EXACT) ? hw::sqrt(vn) : 0.0f;
                RedoLane<EPL>& R = redo[l];
                R.p_old[k] = p0; R.m[k] = mn; R.v[k] = vn; r[l][k] = rk;
                if constexpr (EXACT) {
                    R.p[k] = adam_apply_exact(DECOUPLED ? p0 * h.one_m_wd : p0, mn, vn, h);
                    R.slack[k] = 0.0f;
                } else {
                    R.p[k] = adam_apply_folded<DECOUPLED>(p0, mn, rk, h, AdamFoldedGuard<DT, ECCB>::value, R.slack[k]);
                    if (flagged && in && adam_folded_is_flagged(R.slack[k])) ++*flagged;
                }
                lane_am[l] = fmaxf(lane_am[l], fabsf(mn));
                lane_vmax[l] = fmaxf(lane_vmax[l], vn);
            }
        }
        if constexpr (!EXACT) {
            SimWave<RedoLane<EPL>> wave{redo};
            adam_redo_flagged<EPL, DECOUPLED>(wave, h);
        }
        for (int l = 0; l < kLanes; ++l)
            for (int k = 0; k < EPL; ++k) {
                const int64_t i = base + (int64_t)l * EPL + k;
                if (i < n) write_master<DT, ECCB>(param, ecc, i, redo[l].p[k]);
            }
        if (QUANT) {
            float am[kLanes], av_quick[kLanes], av[kLanes];
            group_scales<EPL>(lane_am, lane_vmax, am, av_quick, av);
            if constexpr (EPL == 8) {
                for (int l = 0; l < kLanes; ++l) {
                    ml[l].am = am[l]; vl[l].av_quick = av_quick[l]; vl[l].av = av[l];
                    for (int k = 0; k < EPL; ++k) { ml[l].m[k] = redo[l].m[k]; vl[l].v[k] = redo[l].v[k]; vl[l].r[k] = r[l][k]; }
                }
                SimWave<MomLane<EPL>> mw{ml};
                SimWave<VarLane<EPL>> vw{vl};
                requantize_mom_verified<EPL>(mw);
                requantize_var_verified<EPL>(vw);
            } else {
                for (int l = 0; l < kLanes; ++l) {
                    bl[l].am = am[l]; bl[l].av_quick = av_quick[l]; bl[l].av = av[l];
                    for (int k = 0; k < EPL; ++k) { bl[l].m[k] = redo[l].m[k]; bl[l].v[k] = redo[l].v[k]; bl[l].r[k] = r[l][k]; }
                }
                SimWave<BothLane<EPL>> bw{bl};
                requantize_both_verified<EPL>(bw);
            }
            for (int l = 0; l < kLanes; ++l) {
                const int64_t first = base + (int64_t)l * EPL;
                for (int k = 0; k < EPL; ++k) {
                    if (first + k >= n) break;
                    ((uint8_t*)mom)[first + k] = (uint8_t)(EPL == 8 ? ml[l].code[k] : bl[l].mcode[k]);
                    ((uint8_t*)var)[first + k] = (uint8_t)(EPL == 8 ? vl[l].code[k] : bl[l].vcode[k]);
                }
                if (first < n && (l & (kGroup / EPL - 1)) == 0) {                    // ref:2424-2434
                    mom_scales[first >> 5] = f32_to_f16(am[l]);
                    var_scales[first >> 5] = f32_to_f16(av[l]);
                }
            }
        } else {
            for (int l = 0; l < kLanes; ++l)
                for (int k = 0; k < EPL; ++k) {
                    const int64_t i = base + (int64_t)l * EPL + k;
                    if (i < n) { store_elem<DT>(mom, i, redo[l].m[k]); store_elem<DT>(var, i, redo[l].v[k]); }
                }
        }
    }
}

// the structure of momentum_finish (fo_momentum.hip), wavefront by wavefront
template <int DT, int ECCB, bool QUANT, int KIND>
void momentum_tensor(void* mom, uint16_t* mom_scales, void* param, const void* grad, void* ecc, int64_t n, const MomentumHyper& h) {
    constexpr int EPL = DTypeInfo<DT>::epl;
    constexpr int kSpan = kLanes * EPL;
    static MomLane<EPL> ml[kLanes];
    for (int64_t base = 0; base < n; base += kSpan) {
        ++g_stats.waves;
        float lane_am[kLanes], lane_zero[kLanes];
        for (int l = 0; l < kLanes; ++l) {
            const int64_t first = base + (int64_t)l * EPL;
            float sm = 1.0f;
            if (QUANT && KIND != KIND_PLAIN && first < n) sm = f16_to_f32(mom_scales[first >> 5]);
            lane_am[l] = lane_zero[l] = 0.0f;
            for (int k = 0; k < EPL; ++k) {
                const int64_t i = first + k;
                const bool in = i < n;
                float p = in ? read_master<DT, ECCB>(param, ecc, i) : 0.0f;
                const float gr = in ? load_elem<DT>(grad, i) : 0.0f;
                float mo = 0.0f;
                if (KIND != KIND_PLAIN && in) mo = QUANT ? kTable.v[256 * kTableMom + ((const uint8_t*)mom)[i]] * sm : load_elem<DT>(mom, i);
                momentum_element<KIND>(gr, p, mo, h, ml[l].m[k]);
                if (in) write_master<DT, ECCB>(param, ecc, i, p);
                lane_am[l] = fmaxf(lane_am[l], fabsf(ml[l].m[k]));
            }
        }
        if (KIND == KIND_PLAIN) continue;
        if (QUANT) {
            float am[kLanes], unused_q[kLanes], unused_e[kLanes];
            group_scales<EPL>(lane_am, lane_zero, am, unused_q, unused_e);
            for (int l = 0; l < kLanes; ++l) ml[l].am = am[l];
            if constexpr (EPL == 8) {   // 2-byte parameters go through the verified quick forms
                SimWave<MomLane<EPL>> mw{ml};
                requantize_mom_verified<EPL>(mw);
            } else {                    // fp32 parameters: the exact form on every value (fo_step.h: quantize_mom)
                for (int l = 0; l < kLanes; ++l) {
                    const float ram = hw::rcp(ml[l].am);
                    for (int k = 0; k < EPL; ++k) ml[l].code[k] = quantize_mom_code(ml[l].m[k], ml[l].am, ram) & 0xffu;
                }
            }
            for (int l = 0; l < kLanes; ++l) {
                const int64_t first = base + (int64_t)l * EPL;
                for (int k = 0; k < EPL && first + k < n; ++k) ((uint8_t*)mom)[first + k] = (uint8_t)ml[l].code[k];
                if (first < n && (l & (kGroup / EPL - 1)) == 0) mom_scales[first >> 5] = f32_to_f16(am[l]);
            }
        } else {
            for (int l = 0; l < kLanes; ++l)
                for (int k = 0; k < EPL; ++k) {
                    const int64_t i = base + (int64_t)l * EPL + k;
                    if (i < n) store_elem<DT>(mom, i, ml[l].m[k]);
                }
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

// Counters of the simulated wavefronts since the last reset: {waves, questions, yes, codes_replaced}.
void hm_flow_stats(int64_t* out, int reset) {
    out[0] = g_stats.waves; out[1] = g_stats.questions; out[2] = g_stats.yes; out[3] = g_stats.codes_replaced;
    if (reset) g_stats = FlowStats();
}

// One wavefront (64 lanes x 8 values) through requantize_mom_verified / requantize_var_verified: m, v in lane order,
// one group per 4 lanes.  The codes the flows deliver and, next to them, the exact forms' codes value by value.
void hm_requantize_wave(const float* m, const float* v, uint8_t* qm, uint8_t* qv, uint8_t* qm_exact, uint8_t* qv_exact) {
    static MomLane<8> ml[kLanes];
    static VarLane<8> vl[kLanes];
    float lane_am[kLanes], lane_vmax[kLanes], am[kLanes], av_quick[kLanes], av[kLanes];
    for (int l = 0; l < kLanes; ++l) {
        lane_am[l] = lane_vmax[l] = 0.0f;
        for (int k = 0; k < 8; ++k) {
            ml[l].m[k] = m[l * 8 + k]; vl[l].v[k] = v[l * 8 + k]; vl[l].r[k] = hw::sqrt(v[l * 8 + k]);
            lane_am[l] = fmaxf(lane_am[l], fabsf(m[l * 8 + k])); lane_vmax[l] = fmaxf(lane_vmax[l], v[l * 8 + k]);
        }
    }
    group_scales<8>(lane_am, lane_vmax, am, av_quick, av);
    for (int l = 0; l < kLanes; ++l) { ml[l].am = am[l]; vl[l].av_quick = av_quick[l]; vl[l].av = av[l]; }
    SimWave<MomLane<8>> mw{ml};
    SimWave<VarLane<8>> vw{vl};
    requantize_mom_verified<8>(mw);
    requantize_var_verified<8>(vw);
    for (int l = 0; l < kLanes; ++l)
        for (int k = 0; k < 8; ++k) {
            qm[l * 8 + k] = (uint8_t)ml[l].code[k];
            qv[l * 8 + k] = (uint8_t)vl[l].code[k];
            qm_exact[l * 8 + k] = (uint8_t)quantize_mom_code(m[l * 8 + k], am[l], hw::rcp(am[l]));
            qv_exact[l * 8 + k] = (uint8_t)quantize_var_code(sqrt_corrected(v[l * 8 + k]), av[l], hw::rcp(av[l]));
        }
}

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
