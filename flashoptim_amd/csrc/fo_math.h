// Per-element arithmetic of the gfx950 step kernels, in one place and in a form that also compiles for the
// host: the ECC join/split, the moment requantiser and the Adam / SGD / Lion element updates.  The kernels
// (fo_adam.hip, fo_momentum.hip, fo_codec.hip) call exactly these functions; a CPU build of the same text
// (FO_MATH_HOST defined, any C++17 compiler) lets the arithmetic be compared element for element with an IEEE
// evaluation of the reference formulas on a machine without a GPU.
//
// Nothing here touches memory, lanes or LDS.  fp32 throughout; the translation units are compiled with
// -ffp-contract=off, so a fused multiply-add happens only where fmaf() is written.
//
// The kernels lean on four hardware approximations (v_rcp_f32, v_rsq_f32, v_sqrt_f32: within one ulp, correctly
// rounded for 85-90 % of inputs on MI355X) and on a few exact instructions (v_ldexp_f32, v_med3, v_cvt_flr).
// In the host build they are stand-ins with the same contract; `fo_math_host_noise` != 0 makes the approximate
// ones err by an ulp in a pseudo-random direction, which is how the CPU tests show that every result that
// is meant to be correctly rounded stays so whatever the hardware returns inside its error bound.
//
// "ref:" cites /root/reference/flashoptim/optimizers.py.
#pragma once

#include <stdint.h>

#include <cmath>
#include <limits>

#ifdef FO_MATH_HOST
#include <math.h>
#define FO_FN static inline
#define FO_LANE_FN inline
#define FO_LANE_ATTR
#define FO_UNROLL
#else
#include <hip/hip_runtime.h>
#define FO_FN __device__ __forceinline__
#define FO_LANE_FN __device__ __forceinline__
#define FO_LANE_ATTR __attribute__((always_inline))
#define FO_UNROLL _Pragma("unroll")
#endif

namespace fo {

typedef uint32_t u32;

constexpr int kGroup = 32;             // ref:1549, 2219: quantisation group
constexpr float kMagic = 12582912.0f;  // 1.5 * 2^23: x + kMagic leaves rne(x) in the low mantissa bits

enum { DT_F32 = 0, DT_BF16 = 1, DT_F16 = 2 };

template <int DT> struct DTypeInfo;
template <> struct DTypeInfo<DT_F32> { static constexpr int bytes = 4, mant = 23, epl = 4; };
template <> struct DTypeInfo<DT_BF16> { static constexpr int bytes = 2, mant = 7, epl = 8; };
template <> struct DTypeInfo<DT_F16> { static constexpr int bytes = 2, mant = 10, epl = 8; };

FO_FN float as_f32(u32 u) { return __builtin_bit_cast(float, u); }
FO_FN u32 as_u32(float f) { return __builtin_bit_cast(u32, f); }

// ------------------------------------------------------------------------------------------------
// the instructions the kernels rely on
// ------------------------------------------------------------------------------------------------
namespace hw {
#ifdef FO_MATH_HOST
extern "C" int fo_math_host_noise;
// Moves an approximate result one ulp up or down for about a quarter of the inputs each.
static inline float nudge(float exact, float x) {
    if (!fo_math_host_noise || !(exact == exact) || exact == 0.0f || __builtin_isinf(exact)) return exact;
    u32 h = as_u32(x) * 2654435761u + (u32)fo_math_host_noise * 40503u;
    h ^= h >> 15; h *= 2246822519u; h ^= h >> 13;
    const u32 pick = h & 3u;
    if (pick == 0) return as_f32(as_u32(exact) + 1u);
    if (pick == 1) return as_f32(as_u32(exact) - 1u);
    return exact;
}
static inline float rcp(float x) { return nudge((float)(1.0 / (double)x), x); }
static inline float rsq(float x) { return nudge((float)(1.0 / sqrt((double)x)), x); }
static inline float sqrt(float x) { return nudge(sqrtf(x), x); }
static inline float fract(float x) { return x - floorf(x); }
static inline float ldexp(float x, int e) { return ldexpf(x, e); }
static inline float med3(float x, float lo, float hi) { return fminf(fmaxf(x, lo), hi); }
static inline int floor_to_int(float x) { return (int)floorf(x); }
static inline float fma(float a, float b, float c) { return __builtin_fmaf(a, b, c); }
#else
FO_FN float rcp(float x) { return __builtin_amdgcn_rcpf(x); }
FO_FN float rsq(float x) { return __builtin_amdgcn_rsqf(x); }
FO_FN float sqrt(float x) { return __builtin_amdgcn_sqrtf(x); }
FO_FN float fract(float x) { return __builtin_amdgcn_fractf(x); }  // x - floor(x)
FO_FN float ldexp(float x, int e) { return __builtin_amdgcn_ldexpf(x, e); }
FO_FN float med3(float x, float lo, float hi) { return __builtin_amdgcn_fmed3f(x, lo, hi); }
// (int)floor(x) in one instruction
FO_FN int floor_to_int(float x) {
    int r;
    asm("v_cvt_flr_i32_f32 %0, %1" : "=v"(r) : "v"(x));
    return r;
}
FO_FN float fma(float a, float b, float c) { return __builtin_fmaf(a, b, c); }
#endif
FO_FN u32 clamp_u32(u32 x, u32 lo, u32 hi) {  // one v_med3_u32
    const u32 t = x > lo ? x : lo;
    return t < hi ? t : hi;
}
}  // namespace hw

// ------------------------------------------------------------------------------------------------
// correctly rounded quotients and roots from the approximate instructions
// ------------------------------------------------------------------------------------------------

// RN(a / b) given r within an ulp of 1/b: one residual correction of the quotient estimate.  q + rem * r equals
// a/b to about 2^-22 ulp before the final rounding of the fma, so the result is the correctly rounded quotient
// except when a/b lies that close to a rounding boundary (about one quotient in a million); with r = RN(1/b)
// it is correctly rounded always (Markstein).  No scaling: callers keep b well inside the normal range.
FO_FN float div_corrected(float a, float b, float r) {
    const float q = a * r;
    const float rem = hw::fma(-b, q, a);
    return hw::fma(rem, r, q);
}

// RN(sqrt(x)) for x >= 0 from the reciprocal-root instruction: s = x * y, one Newton correction with the exact
// residual x - s*s.  x == 0 gives 0 (the clamp keeps y finite), subnormal x gives a value below 2^-63.
FO_FN float sqrt_corrected(float x) {
    const float y = hw::rsq(fmaxf(x, 1.17549435e-38f));
    const float s = x * y;
    const float h = 0.5f * y;
    const float rem = hw::fma(-s, s, x);
    return hw::fma(rem, h, s);
}

// RN(q / 255) for an integer q in 0..255 (ref:2333): the product with 1/255 held as a two-term constant,
// fma(q, k_hi, q * k_lo) with k_hi + k_lo = 1/255 to 2^-50.  The correctly rounded quotient for each of the 256
// codes (checked exhaustively on the host); q * RN(1/255) alone misses it for 126 of them.
FO_FN float code_over_255(float q) {
    constexpr double k = 1.0 / 255.0;
    constexpr float k_hi = (float)k;
    constexpr float k_lo = (float)(k - (double)k_hi);
    return hw::fma(q, k_hi, q * k_lo);
}

// ------------------------------------------------------------------------------------------------
// ECC: narrow value + signed integer fraction of half its ulp (ref:2682-2776)
// ------------------------------------------------------------------------------------------------
template <int ECCB> struct EccInfo;
template <> struct EccInfo<1> { static constexpr float max_val = 127.0f; };      // ref:1521
template <> struct EccInfo<2> { static constexpr float max_val = 32767.0f; };    // ref:1523

// fp32 bit pattern of 2^E, E = unbiased exponent of the narrow value with zero/subnormal mapped to the
// smallest normal exponent (ref:2704-2712), given the value widened to fp32.  bf16 shares fp32's exponent
// field; an fp16 subnormal widens to an fp32 normal below 2^-14, which the lower clamp maps back to -14.
// The upper clamp keeps inf/NaN inputs from producing an infinite scale.
template <int DT> FO_FN u32 pow2_of_exponent_bits(float widened) {
    constexpr u32 lo = (DT == DT_F16) ? ((127u - 14u) << 23) : (1u << 23);
    const u32 e = as_u32(widened) & 0x7f800000u;
    return hw::clamp_u32(e, lo, 254u << 23);
}

// x_narrow + (ecc / MAX) * 2^(E - mant - 1) with the product and the sum fused (ref:2767-2776; the reference
// compiles with FP fusion, and its invariants test only passes with the fused form).
//   ecc_fraction: (ecc / MAX) * 2^-(mant+1), the division correctly rounded, formed as fma(e, K_hi, e * K_lo) with
//   K_hi + K_lo = 2^-(mant+1) / MAX to well beyond fp32 precision (checked exhaustively over every int8 / int16
//   value on the host).  For int8 codes the kernels read the same values from a 256-entry table (EccFractionTable).
template <int DT, int ECCB> FO_FN float ecc_fraction(float ecc) {
    constexpr double k = 1.0 / ((double)EccInfo<ECCB>::max_val * (double)(1 << (DTypeInfo<DT>::mant + 1)));
    constexpr float k_hi = (float)k;
    constexpr float k_lo = (float)(k - (double)k_hi);
    return hw::fma(ecc, k_hi, ecc * k_lo);
}
template <int DT> FO_FN float ecc_join_fraction(float widened, float fraction) {
    return hw::fma(fraction, as_f32(pow2_of_exponent_bits<DT>(widened)), widened);
}
template <int DT, int ECCB> FO_FN float ecc_join(float widened, float ecc) {
    return ecc_join_fraction<DT>(widened, ecc_fraction<DT, ECCB>(ecc));
}

// Signed fraction of half an ulp of the NEW narrow value, scaled to +-MAX and rounded half away from zero
// (ref:2735-2756).  Returns a word whose low byte / half is the two's-complement code.
//   General form: sc = clamp(en) * MAX rounded to fp32 as in the reference, then trunc(sc + copysign(0.5, sc)),
//   which equals copysign(floor(|sc| + 0.5), sc) including the fp32 rounding of the sum.
//   bf16 with an int8 code: p - narrow is exact and a multiple of 2^-16 half-ulps, so en * 127 fits 24 bits and
//   is exact; the only tie that can occur is +-63.5, where half-even and half-away agree.  One fma against
//   1.5 * 2^23 then leaves the rounded integer in the low mantissa bits.
//   CLAMP = false is for callers whose narrow value IS the round-to-nearest of p (|en| <= 1 by construction).
//   For them the bf16/int8 case folds the scaling into the fma: with eb the biased exponent field of the narrow
//   value (1..254), en * 127 = err * 127 * 2^(135 - eb).  That factor can exceed the fp32 range, so both fma
//   operands carry an extra 2^-13: S = 127 * 2^(122 - eb) is a normal number for every eb (bit pattern
//   0x7ffe0000 - (eb << 23)) and 1.5 * 2^10 + en * 127 * 2^-13 has the same mantissa bits as
//   1.5 * 2^23 + en * 127, rounded at the same place.
template <int DT, int ECCB, bool CLAMP> FO_FN u32 ecc_split_bits(float p, float widened) {
    const float err = p - widened;
    if constexpr (DT == DT_BF16 && ECCB == 1 && !CLAMP) {
        const float s = as_f32(0x7ffe0000u - pow2_of_exponent_bits<DT>(widened));
        return as_u32(hw::fma(err, s, 1536.0f));
    } else {
        const int nls = (DTypeInfo<DT>::mant + 1 + 127) - (int)(pow2_of_exponent_bits<DT>(widened) >> 23);
        float en = hw::ldexp(err, nls);
        if constexpr (CLAMP) en = hw::med3(en, -1.0f, 1.0f);
        if constexpr (DT == DT_BF16 && ECCB == 1) {
            return as_u32(hw::fma(en, EccInfo<ECCB>::max_val, kMagic));
        } else {
            const float sc = en * EccInfo<ECCB>::max_val;
            return (u32)(int)(sc + __builtin_copysignf(0.5f, sc));
        }
    }
}

// ------------------------------------------------------------------------------------------------
// 8-bit group codec
// ------------------------------------------------------------------------------------------------

// The two code tables of the step kernels, evaluated by the compiler (IEEE, round to nearest), 256 entries each,
// indexed by the code byte:
//   kTableMom   first-moment value of signed code byte b before the group scale, (q/127) / (2 - |q/127|) with
//               each operation correctly rounded (ref:2332-2336);
//   kTableEcc   (q/127) * 2^-(mant+1) for an int8 ECC byte b, the division correctly rounded (ref:2772): the
//               factor that multiplies 2^E in ecc_join_fraction.  The scaling by a power of two is exact.
// (The second-moment value q / 255 is formed arithmetically, code_over_255: a third table saved two instructions
// per element and cost a lookup, with no gain in step time.)
enum { kTableMom = 0, kTableEcc = 1, kTableCount = 2 };
template <int DT> struct StepTables {
    float v[256 * kTableCount];
    constexpr StepTables() : v() {
        for (int b = 0; b < 256; ++b) {
            const int q = b < 128 ? b : b - 256;
            const float y = (float)q / 127.0f;
            const float a = y < 0.0f ? -y : y;
            v[256 * kTableMom + b] = y / (2.0f - a);
            v[256 * kTableEcc + b] = y * (1.0f / (float)(1 << (DTypeInfo<DT>::mant + 1)));
        }
    }
};
typedef StepTables<DT_BF16> SoftsignTable;  // first 256 entries: the same for every parameter dtype

// Requantisation of a moment value against its group's absmax, rounding exactly as the reference's formula does
// when every operation is evaluated in IEEE fp32 (ref:2405-2419, 1703-1710):
//     nm = m / am;  t = (2 nm) / (1 + |nm|);  code = floor(t * 127 + 0.5)          first moment
//     code = floor((r / av) * 255 + 0.5),  r = sqrt(v)                             second moment
// Each quotient is the correctly rounded one (div_corrected), the product and the sum round separately, and the
// floor is taken of the rounded sum.  Doubling is exact, so RN(2nm / d) * 127 is formed as RN(nm / d) * 254.
// ram / rav: the reciprocal instruction applied to the group absmax (shared by the lanes of the group).
// Returns a word whose low byte is the code.
// The *_rounded functions return the rounded sum fl(x + 0.5) whose floor is the code (the kernels convert and pack
// four of them at a time); the *_code functions finish the job for one value.
FO_FN float quantize_mom_rounded(float m, float am, float ram) {
    const float nm = div_corrected(m, am, ram);
    const float d = 1.0f + fabsf(nm);
    const float t = div_corrected(nm, d, hw::rcp(d));
    return t * 254.0f + 0.5f;
}
FO_FN float quantize_var_rounded(float r, float av, float rav) {
    const float q = div_corrected(r, av, rav);
    return q * 255.0f + 0.5f;  // non-negative: truncation is the floor
}
FO_FN u32 quantize_mom_code(float m, float am, float ram) { return (u32)hw::floor_to_int(quantize_mom_rounded(m, am, ram)); }
FO_FN u32 quantize_var_code(float r, float av, float rav) { return (u32)(int)quantize_var_rounded(r, av, rav); }
// The quick forms.  The exact requantiser above costs two corrected quotients per first-moment value and a corrected
// quotient plus a corrected square root per second-moment value.  The quick forms evaluate the same real-number
// formulas with the quotients merged and approximate, and say whether their result can be trusted:
//     first moment   x = 254 m / (am + |m|) + 0.5            as  fma(m * rcp(am + |m|), 254, 0.5 + margin)
//     second moment  x = 255 r / av + 0.5                     as  fma(r, 255 * rcp(av), 0.5 + margin), r, av from hw::sqrt
// Either form and the exact one stay within a known distance of the real-number value x (each rounding contributes
// 2^-24 relative, each approximate instruction at most an ulp; in code units, with |x| <= 128 resp. 256):
//     first moment   exact 3.8e-5, quick 3.8e-5   ->  they can differ by 7.6e-5   ->  margin 2^-13 = 1.2e-4
//     second moment  exact 7.6e-5, quick 1.2e-4   ->  they can differ by 2.0e-4   ->  margin 2^-12 = 2.4e-4
// so when the quick value lies farther than the margin from every integer, floor() of it IS the exact form's code.
// Precondition: am + |m| and av stay below 2^126 (beyond that the reciprocal instruction returns a subnormal, flushed
// to zero).  The group scale is stored as fp16 and overflows at 65504, forty orders of magnitude earlier, so a state
// that large is already lost; the bound is stated, not enforced.
// The margin is added up front (so the test is one fract and one compare: fract(x + margin) >= 2 margin) and a value
// that fails the test is requantised with the exact form.  About 2.4e-4 of the first-moment and 4.9e-4 of the
// second-moment values of a continuous distribution fail it; values that sit on a rounding boundary to the last bit
// (first steps from a zero state, sparse or lattice-valued gradients) always fail it.  The codes are therefore those
// of the exact requantiser on any data, by construction; the stored scales are always formed from the correctly
// rounded maximum.
// Used by the Adam kernels (all but the folded update with a 2-byte ECC, AdamQuickRequant) and by the momentum
// kernels on 2-byte parameters; the other kernels evaluate the exact forms only.
constexpr float kQuickMarginMom = 0x1p-13f;
constexpr float kQuickMarginVar = 0x1p-12f;
// Quick pre-floor values (margin included).  rav255 = 255 * rcp(av), av = hw::sqrt of the group's largest v.
FO_FN float quantize_mom_quick(float m, float am) {
    const float t = m * hw::rcp(am + fabsf(m));  // = nm / (1 + |nm|), nm = m / am
    return hw::fma(t, 254.0f, 0.5f + kQuickMarginMom);
}
FO_FN float quantize_var_quick(float r, float rav255) { return hw::fma(r, rav255, 0.5f + kQuickMarginVar); }
// floor(x) is the exact form's code unless x (a quick value, margin included) lies within the margin of an integer:
// the value is safe when fract(x) >= 2 margin.  quick_value_slack is that fractional part; callers that hold several
// values compare the smallest slack once and look at the single values only when that fails.
FO_FN float quick_value_slack(float x) { return hw::fract(x); }
FO_FN bool quick_slack_is_safe(float slack, float margin) { return slack >= 2.0f * margin; }
FO_FN bool quick_value_is_safe(float x, float margin) { return quick_slack_is_safe(quick_value_slack(x), margin); }
// One value through quick form, test and, if need be, exact form (what the kernels do, element by element).
//   av_quick / av_exact: hw::sqrt and sqrt_corrected of the group's largest v; v: the element's second moment.
FO_FN u32 quantize_mom_code_verified(float m, float am) {
    const float x = quantize_mom_quick(m, am);
    return quick_value_is_safe(x, kQuickMarginMom) ? (u32)hw::floor_to_int(x) : quantize_mom_code(m, am, hw::rcp(am));
}
FO_FN u32 quantize_var_code_verified(float v, float av_quick, float av_exact) {
    const float x = quantize_var_quick(hw::sqrt(v), hw::rcp(av_quick) * 255.0f);
    return quick_value_is_safe(x, kQuickMarginVar) ? (u32)(int)x : quantize_var_code(sqrt_corrected(v), av_exact, hw::rcp(av_exact));
}

// ------------------------------------------------------------------------------------------------
// Adam / AdamW element update (ref:2296-2375)
// ------------------------------------------------------------------------------------------------

// Per-launch constants.  Scalars arrive as fp32 like the reference's kernel arguments; 1 - x is formed in fp32
// (ref:2357-2364).
struct AdamHyper {
    float b1, one_m_b1, b2, one_m_b2, wd, one_m_wd;
    // folded form: the per-step bias corrections and the learning rate are folded on the host (in double, rounded
    // once) into the two constants of the update's denominator, negated so that the update is one fma:
    //     lr * (m / bc1) / (sqrt(v / bc2) + eps)  ==  m / (sqrt(v) * den_scale + den_bias)
    //     den_scale = bc1 / (lr * sqrt(bc2)),  den_bias = eps * bc1 / lr
    float neg_den_scale, neg_den_bias;
    // host only: the folded constants are ordinary numbers (see make_adam_hyper); otherwise the launch takes the
    // operation-by-operation kernel
    int folded_ok;
    // operation-by-operation form (EXACT): the reference's own sequence with correctly rounded quotients
    float lr, eps, bc1, rcp_bc1, bc2, rcp_bc2;  // rcp_*: correctly rounded reciprocals, formed on the host
};

// Host side: the constants of one launch from the reference's kernel arguments (ref:2264-2270).
inline AdamHyper make_adam_hyper(float lr, float beta1, float beta2, float eps, float wd, int step) {
    AdamHyper h;
    h.b1 = beta1; h.one_m_b1 = 1.0f - beta1;
    h.b2 = beta2; h.one_m_b2 = 1.0f - beta2;
    h.wd = wd; h.one_m_wd = 1.0f - wd;
    // beta^step is the correctly rounded fp32 power, 1 - that is formed in fp32 (ref:2368-2369)
    h.bc1 = 1.0f - (float)std::pow((double)beta1, (double)step);
    h.bc2 = 1.0f - (float)std::pow((double)beta2, (double)step);
    h.rcp_bc1 = (float)(1.0 / (double)h.bc1);
    h.rcp_bc2 = (float)(1.0 / (double)h.bc2);
    h.lr = lr; h.eps = eps;
    const double bc1 = (double)h.bc1, bc2 = (double)h.bc2;
    if (lr != 0.0f) {
        h.neg_den_scale = -(float)(bc1 / ((double)lr * std::sqrt(bc2)));
        h.neg_den_bias = -(float)((double)eps * bc1 / (double)lr);
    } else {  // no update: the denominator is infinite whatever sqrt(v) is
        h.neg_den_scale = 0.0f;
        h.neg_den_bias = -std::numeric_limits<float>::infinity();
    }
    // The folded update's error bound (adam_apply_folded) assumes that both constants carry a full fp32 mantissa and
    // that sqrt(v) * den_scale neither overflows nor turns subnormal for any fp32 v: den_scale within 2^-40 .. 2^60
    // (lr between about 1e-18 and 1e12) and den_bias zero or a normal number.  lr == 0 is exact as it stands.
    const double ds = std::fabs((double)h.neg_den_scale), db = std::fabs((double)h.neg_den_bias);
    h.folded_ok = lr == 0.0f || (lr > 0.0f && ds >= 0x1p-40 && ds <= 0x1p60 && (db == 0.0 || (db >= 0x1p-126 && db <= 0x1p100)));
    return h;
}

// Which variants follow the reference's update operation by operation on every element (EXACT): those whose unit
// of master precision is about one fp32 ulp or finer, so that nothing but the reference's own sequence of
// roundings meets it -- fp32 parameters, 2-byte parameters with a 2-byte ECC (32-bit masters: the unit is
// 32768/32767 fp32 ulps), fp16 parameters with a 1-byte ECC (unit 2^-19 of the weight).  bf16 parameters with a
// 1-byte ECC (24-bit masters, unit 2^-16 of the weight) and 2-byte parameters without ECC (unit = one ulp of the
// narrow type) take the folded update and redo operation by operation only the elements it cannot vouch for
// (adam_apply_folded below).
template <int DT, int ECCB> struct AdamExact {
    static constexpr bool value = DT == DT_F32 || ECCB == 2 || (DT == DT_F16 && ECCB == 1);
};
// Variants that use the quick requantiser forms (verified value by value, see above; the codes are the exact
// forms' either way): every one.
template <int DT, int ECCB> struct AdamQuickRequant { static constexpr bool value = true; };

// New moments from the dequantised pieces, every operation of ref:2332-2360 rounded on its own.
//   table_m: (q/127) / (2 - |q/127|) of the first-moment code (StepTables); qv: the second-moment code as a float.
FO_FN void adam_moments_quantized(float g, float table_m, float sm, float qv, float sv, const AdamHyper& h, float& mn,
                                  float& vn) {
    const float mo = table_m * sm;                                              // ref:2332-2343
    const float s = code_over_255(qv) * sv;                                     // ref:2333-2347
    const float vo = s * s;                                                     // ref:2348
    mn = mo * h.b1 + g * h.one_m_b1;                                            // ref:2357
    vn = vo * h.b2 + (g * g) * h.one_m_b2;                                      // ref:2360
}
// Unquantised states: operation by operation as written in the reference, no contraction (ref:2351-2360).
FO_FN void adam_moments_plain(float g, float mo, float vo, const AdamHyper& h, float& mn, float& vn) {
    mn = mo * h.b1 + g * h.one_m_b1;
    vn = vo * h.b2 + (g * g) * h.one_m_b2;
}

// p -= lr * (m/bc1) / (sqrt(v/bc2) + eps), operation by operation (ref:2368-2375): every quotient and the root
// correctly rounded.  p: the weight after the decoupled decay, if any.
FO_FN float adam_apply_exact(float p, float mn, float vn, const AdamHyper& h) {
    const float cm = div_corrected(mn, h.bc1, h.rcp_bc1);
    const float cv = div_corrected(vn, h.bc2, h.rcp_bc2);
    const float den = sqrt_corrected(cv) + h.eps;
    float rd = hw::rcp(den);
    rd = hw::fma(hw::fma(-den, rd, 1.0f), rd, rd);  // reciprocal refined to well below an ulp
    return p - div_corrected(h.lr * cm, den, rd);
}

// The folded update and its guard.
//   Folded: u = m * rcp(-(r c1 + c2)) with r = hw::sqrt(v) and c1, c2 the host-folded constants (AdamHyper), then
//   p_new = fma(p, 1 - wd, u) (decoupled decay) or p + u: four instructions, where the reference's sequence costs
//   about twenty.  With u = 2^-24 (half an ulp, relative) the two evaluations of the update differ by at most
//       reference   lr*cm: 2u;  cv: u -> root u/2, rounding of the root u, of the sum with eps u;  quotient u    = 5.5u
//       folded      r: one ulp = 2u, c1: u, fma: u, rcp: one ulp = 2u, product: u                                = 7u
//   i.e. by 12.5u |update| from identical m and v (the moments are formed operation by operation in both), and
//   the fused decay rounds p(1 - wd) once less than the reference: u |p(1 - wd)| <= u (|p_new| + |update|).  With
//   the final rounding of either side (u |p_new| each) the two fp32 results are at most
//       13.5u |update| + 3u |p_new|
//   apart.  They are split into the same narrow value and a correction code that differs by at most one -- the
//   master weights agree to within one unit of master precision -- whenever that distance is below one unit,
//   and a unit is at least G |p_new| with G = 2^-16 for bf16 + 1-byte ECC (2^(E-8)/127 against |p_new| <
//   2^(E+1)), 2^-8 for bf16 without ECC (one bf16 ulp) and 2^-11 for fp16 without ECC:
//       13.5u |update| < (G - 3u) |p_new|   <=>   |update| < (2^24 G - 3) / 13.5 |p_new|
//   = 18.7, 4854 and 606 times |p_new|.  kGuard is the power of two below (16, 4096, 512); an element whose
//   folded update exceeds kGuard |p_new| -- a weight that its own update all but cancels: 1e-3 of the elements on a
//   first step with weights ~N(0, 0.02) and lr 1e-3, fewer later -- is flagged and the caller redoes it with
//   adam_apply_exact, whose result is the reference's bit for bit.  Every other element is within one unit by
//   the bound above, whatever the data.
template <int DT, int ECCB> struct AdamFoldedGuard {
    static_assert(!AdamExact<DT, ECCB>::value, "the folded update is not offered for this variant");
    static constexpr float value = ECCB == 1 ? 16.0f : (DT == DT_BF16 ? 4096.0f : 512.0f);
};
// Returns the new weight; `slack` receives guard * |p_new| - |update|, negative for a flagged element (callers that
// hold several elements take the smallest slack, test it once and look at the single ones only when that fails).
template <bool DECOUPLED>
FO_FN float adam_apply_folded(float p, float mn, float r, const AdamHyper& h, float guard, float& slack) {
    const float neg_den = hw::fma(r, h.neg_den_scale, h.neg_den_bias);
    const float u = mn * hw::rcp(neg_den);
    const float pn = DECOUPLED ? hw::fma(p, h.one_m_wd, u) : p + u;
    slack = hw::fma(fabsf(pn), guard, -fabsf(u));
    return pn;
}
FO_FN bool adam_folded_is_flagged(float slack) { return slack < 0.0f; }

// ------------------------------------------------------------------------------------------------
// wave-level control flow of the verified forms
// ------------------------------------------------------------------------------------------------
// The verified forms act on a whole wavefront.  Every lane converts its values from the quick forms and keeps each
// value's slack; the wavefront asks once whether any lane holds a value that failed its test (most wavefronts branch
// past the repair there), and only then looks at the element positions one by one: a position is recomputed with
// the exact form -- by every lane, the result kept by the lanes in which it failed -- only if it failed in some lane.
// The flows are written once, over a `Wave`:
//     wave.each(f)   runs f(lane) for every lane of the wavefront,
//     wave.any(p)    tells whether p(lane) holds in some lane,
// with `lane` the lane's own state (the structs named below).  In the kernels a Wave is the hardware wavefront seen
// from one of its lanes (each: one call; any: a ballot; fo_step.h) and the lane state lives in registers; in the CPU
// build used by the tests it is an array of 64 lane states (each: a loop; any: a logical or), so the same text runs
// with a chosen lane and position failing.

// Requantisation of a lane's N first-moment values.  Lane members:
//   m[N], am            the values and the group absmax (clamped at 1e-12)
//   x[N], slack[N], least, ram    scratch of the flow
//   convert_mom(x)      codes of all N values from their quick values (floor)
//   set_mom_code(k, c)  replaces the code of position k
template <int N, class Wave> FO_FN void requantize_mom_verified(Wave& wave) {
    wave.each([](auto& L) FO_LANE_ATTR {
        FO_UNROLL for (int k = 0; k < N; ++k) {
            L.x[k] = quantize_mom_quick(L.m[k], L.am);
            L.slack[k] = quick_value_slack(L.x[k]);
        }
        L.least = L.slack[0];
        FO_UNROLL for (int k = 1; k < N; ++k) L.least = fminf(L.least, L.slack[k]);
        L.convert_mom(L.x);
    });
    if (wave.any([](const auto& L) FO_LANE_ATTR { return !quick_slack_is_safe(L.least, kQuickMarginMom); })) {
        wave.each([](auto& L) FO_LANE_ATTR { L.ram = hw::rcp(L.am); });
        FO_UNROLL for (int k = 0; k < N; ++k) {
            if (wave.any([k](const auto& L) FO_LANE_ATTR { return !quick_slack_is_safe(L.slack[k], kQuickMarginMom); })) {
                wave.each([k](auto& L) FO_LANE_ATTR {
                    const u32 code = quantize_mom_code(L.m[k], L.am, L.ram);
                    if (!quick_slack_is_safe(L.slack[k], kQuickMarginMom)) L.set_mom_code(k, code);
                });
            }
        }
    }
}

// Requantisation of a lane's N second-moment values.  Lane members:
//   v[N], r[N]          the values and hw::sqrt of them
//   av_quick, av        hw::sqrt and sqrt_corrected of the group's largest v (clamped at 1e-12)
//   x[N], slack[N], least, rav    scratch of the flow
//   convert_var(x), set_var_code(k, c)
template <int N, class Wave> FO_FN void requantize_var_verified(Wave& wave) {
    wave.each([](auto& L) FO_LANE_ATTR {
        const float rav255 = hw::rcp(L.av_quick) * 255.0f;
        FO_UNROLL for (int k = 0; k < N; ++k) {
            L.x[k] = quantize_var_quick(L.r[k], rav255);
            L.slack[k] = quick_value_slack(L.x[k]);
        }
        L.least = L.slack[0];
        FO_UNROLL for (int k = 1; k < N; ++k) L.least = fminf(L.least, L.slack[k]);
        L.convert_var(L.x);
    });
    if (wave.any([](const auto& L) FO_LANE_ATTR { return !quick_slack_is_safe(L.least, kQuickMarginVar); })) {
        wave.each([](auto& L) FO_LANE_ATTR { L.rav = hw::rcp(L.av); });
        FO_UNROLL for (int k = 0; k < N; ++k) {
            if (wave.any([k](const auto& L) FO_LANE_ATTR { return !quick_slack_is_safe(L.slack[k], kQuickMarginVar); })) {
                wave.each([k](auto& L) FO_LANE_ATTR {
                    const u32 code = quantize_var_code(sqrt_corrected(L.v[k]), L.av, L.rav);
                    if (!quick_slack_is_safe(L.slack[k], kQuickMarginVar)) L.set_var_code(k, code);
                });
            }
        }
    }
}

// Both moments of a lane that holds N values of each (fp32 parameters, N = 4): one conversion, one repair branch.
// Lane members: those of the two flows above with the scratch doubled (xm, xv, slack_m, slack_v, least_m, least_v)
// and convert_both(xm, xv).
template <int N, class Wave> FO_FN void requantize_both_verified(Wave& wave) {
    wave.each([](auto& L) FO_LANE_ATTR {
        const float rav255 = hw::rcp(L.av_quick) * 255.0f;
        FO_UNROLL for (int k = 0; k < N; ++k) {
            L.xm[k] = quantize_mom_quick(L.m[k], L.am);
            L.xv[k] = quantize_var_quick(L.r[k], rav255);
            L.slack_m[k] = quick_value_slack(L.xm[k]);
            L.slack_v[k] = quick_value_slack(L.xv[k]);
        }
        L.least_m = L.slack_m[0];
        L.least_v = L.slack_v[0];
        FO_UNROLL for (int k = 1; k < N; ++k) {
            L.least_m = fminf(L.least_m, L.slack_m[k]);
            L.least_v = fminf(L.least_v, L.slack_v[k]);
        }
        L.convert_both(L.xm, L.xv);
    });
    if (wave.any([](const auto& L) FO_LANE_ATTR {
            return !quick_slack_is_safe(L.least_m, kQuickMarginMom) || !quick_slack_is_safe(L.least_v, kQuickMarginVar);
        })) {
        wave.each([](auto& L) FO_LANE_ATTR { L.ram = hw::rcp(L.am); L.rav = hw::rcp(L.av); });
        FO_UNROLL for (int k = 0; k < N; ++k) {
            if (wave.any([k](const auto& L) FO_LANE_ATTR { return !quick_slack_is_safe(L.slack_m[k], kQuickMarginMom); })) {
                wave.each([k](auto& L) FO_LANE_ATTR {
                    const u32 code = quantize_mom_code(L.m[k], L.am, L.ram);
                    if (!quick_slack_is_safe(L.slack_m[k], kQuickMarginMom)) L.set_mom_code(k, code);
                });
            }
            if (wave.any([k](const auto& L) FO_LANE_ATTR { return !quick_slack_is_safe(L.slack_v[k], kQuickMarginVar); })) {
                wave.each([k](auto& L) FO_LANE_ATTR {
                    const u32 code = quantize_var_code(sqrt_corrected(L.v[k]), L.av, L.rav);
                    if (!quick_slack_is_safe(L.slack_v[k], kQuickMarginVar)) L.set_var_code(k, code);
                });
            }
        }
    }
}

// The repair of the guarded folded Adam update: the positions flagged in some lane again, operation by operation.
// Lane members:
//   p[N]                the folded results, overwritten where flagged
//   slack[N]            from adam_apply_folded (negative = flagged); least: scratch
//   m[N], v[N]          the new moments
//   old_master(k)       the weight before the step (fp32 master, before the decoupled decay)
template <int N, bool DECOUPLED, class Wave> FO_FN void adam_redo_flagged(Wave& wave, const AdamHyper& h) {
    wave.each([](auto& L) FO_LANE_ATTR {
        L.least = L.slack[0];
        FO_UNROLL for (int k = 1; k < N; ++k) L.least = fminf(L.least, L.slack[k]);
    });
    if (wave.any([](const auto& L) FO_LANE_ATTR { return adam_folded_is_flagged(L.least); })) {
        FO_UNROLL for (int k = 0; k < N; ++k) {
            if (wave.any([k](const auto& L) FO_LANE_ATTR { return adam_folded_is_flagged(L.slack[k]); })) {
                wave.each([k, &h](auto& L) FO_LANE_ATTR {
                    float pk = L.old_master(k);
                    if (DECOUPLED) pk = pk * h.one_m_wd;                                // ref:2363-2364
                    const float pe = adam_apply_exact(pk, L.m[k], L.v[k], h);           // ref:2368-2375
                    if (adam_folded_is_flagged(L.slack[k])) L.p[k] = pe;
                });
            }
        }
    }
}

// ------------------------------------------------------------------------------------------------
// SGD / SGDW / Nesterov / Lion element update (ref:1624-1683, 1447-1465)
// ------------------------------------------------------------------------------------------------
enum { KIND_SGD = 0, KIND_LION = 1, KIND_PLAIN = 2 };

struct MomentumHyper {
    float lr, mom_coef, update_coef, one_m_mom_coef, one_m_update_coef, wd, one_m_wd;
    int decoupled, nesterov;
    int apply_decay;  // momentum-free branch only: the reference skips both decays when weight_decay == 0
};

inline MomentumHyper make_momentum_hyper(float lr, float mom_coef, float update_coef, float wd, int decoupled, int nesterov) {
    MomentumHyper h;
    h.lr = lr; h.mom_coef = mom_coef; h.update_coef = update_coef;
    h.one_m_mom_coef = 1.0f - mom_coef; h.one_m_update_coef = 1.0f - update_coef;
    h.wd = wd; h.one_m_wd = 1.0f - wd;
    h.decoupled = decoupled ? 1 : 0; h.nesterov = nesterov ? 1 : 0;
    h.apply_decay = wd > 0.0f ? 1 : 0;
    return h;
}

// g, p: gradient and master weight; mo: the dequantised (or plain) momentum.  Writes the new weight and momentum.
template <int KIND> FO_FN void momentum_element(float g, float& p, float mo, const MomentumHyper& h, float& mn) {
    float pk = p;
    if constexpr (KIND == KIND_PLAIN) {
        if (h.apply_decay && !h.decoupled) g = g + pk * h.wd;                       // ref:1452-1453
        if (h.apply_decay && h.decoupled) pk = pk * h.one_m_wd;                     // ref:1454-1455
        pk = pk - g * h.lr;                                                         // ref:1456
        mn = 0.0f;
    } else if constexpr (KIND == KIND_LION) {
        const float u = (mo * h.update_coef) + (g * h.one_m_update_coef);           // ref:1667
        const float sgn = (u > 0.0f) ? 1.0f : ((u < 0.0f) ? -1.0f : 0.0f);          // ref:1668
        mn = (mo * h.mom_coef) + (g * h.one_m_mom_coef);                            // ref:1669
        pk = pk * h.one_m_wd;                                                       // ref:1675
        pk = pk - sgn * h.lr;                                                       // ref:1676
    } else {
        if (!h.decoupled) g = g + pk * h.wd;                                        // ref:1639-1640
        mn = mo * h.mom_coef + g * h.update_coef;                                   // ref:1671
        if (h.decoupled) pk = pk * h.one_m_wd;                                      // ref:1678-1679
        if (h.nesterov) pk = pk - (g + h.mom_coef * mn) * h.lr;                     // ref:1680-1681
        else pk = pk - mn * h.lr;                                                   // ref:1682-1683
    }
    p = pk;
}

}  // namespace fo
