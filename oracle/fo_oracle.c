/*
 * Scalar C restatement of FlashOptim's fused step math (IEEE fp32, one rounding per operation).
 *
 * TEST INFRASTRUCTURE ONLY.  Built into oracle/libfo_oracle.so by oracle/Makefile with
 * -ffp-contract=off and loaded by tests/, __graft_entry__.smoke() and bench.py's cpu_baseline
 * leg through oracle/c_oracle.py.  The product library never links or loads it.
 *
 * "ref:" cites /root/reference/flashoptim/optimizers.py.  The file is written independently of
 * oracle/torch_oracle.py (element-at-a-time instead of tensor-at-a-time) so that the two can be
 * checked against each other bit for bit; see the parity notes in torch_oracle.py's header, which
 * apply here unchanged (bit-level parity with the Triton kernels is unpinned; the bias-correction
 * power is the correctly rounded fp32 power).
 */
#include <math.h>
#include <stdint.h>
#include <string.h>

#define FO_GROUP 32 /* ref:1549, 2219, 2451, 2506 */

enum { FO_F32 = 0, FO_BF16 = 1, FO_F16 = 2 };

/* ---------------------------------------------------------------- scalar format helpers --- */

static inline uint32_t f2u(float f) { uint32_t u; memcpy(&u, &f, 4); return u; }
static inline float u2f(uint32_t u) { float f; memcpy(&f, &u, 4); return f; }

static float bf16_to_f32(uint16_t h) { return u2f((uint32_t)h << 16); }

static uint16_t f32_to_bf16(float f) { /* round to nearest even; NaN stays NaN */
    uint32_t u = f2u(f);
    if ((u & 0x7fffffffu) > 0x7f800000u) return (uint16_t)((u >> 16) | 0x0040u);
    u += 0x7fffu + ((u >> 16) & 1u);
    return (uint16_t)(u >> 16);
}

static float f16_to_f32(uint16_t h) {
    uint32_t sign = (uint32_t)(h & 0x8000u) << 16;
    uint32_t e = (h >> 10) & 0x1fu, m = h & 0x3ffu;
    if (e == 0) { /* zero / subnormal: m * 2^-24 is exact in fp32 */
        float v = (float)m * 0x1p-24f;
        return u2f(f2u(v) | sign);
    }
    if (e == 31) return u2f(sign | 0x7f800000u | (m << 13));
    return u2f(sign | ((e + 112u) << 23) | (m << 13));
}

static uint16_t f32_to_f16(float f) { /* round to nearest even, subnormals kept, overflow -> inf */
    uint32_t u = f2u(f);
    uint16_t sign = (uint16_t)((u >> 16) & 0x8000u);
    uint32_t a = u & 0x7fffffffu;
    if (a > 0x7f800000u) return (uint16_t)(sign | 0x7e00u);
    if (a >= 0x47800000u) return (uint16_t)(sign | 0x7c00u); /* >= 65536 (incl. inf) -> inf */
    if (a < 0x38800000u) { /* below the smallest fp16 normal 2^-14: result is k * 2^-24 */
        /* adding 0.5 makes the fp32 adder round |f| to a multiple of 2^-24 (ulp of [0.5,1)) with RNE */
        float r = u2f(a) + 0.5f;
        return (uint16_t)(sign | (uint16_t)(f2u(r) - 0x3f000000u));
    }
    uint32_t r = a + 0xfffu + ((a >> 13) & 1u); /* RNE at bit 13 */
    r = (r - 0x38000000u) >> 13;                 /* rebias 127 -> 15; may carry into inf (65520+) */
    return (uint16_t)(sign | (uint16_t)r);
}

static float load_as_f32(const void *p, int dtype, int64_t i) {
    switch (dtype) {
        case FO_F32: return ((const float *)p)[i];
        case FO_BF16: return bf16_to_f32(((const uint16_t *)p)[i]);
        default: return f16_to_f32(((const uint16_t *)p)[i]);
    }
}

/* rounds v to the narrow dtype, stores it, returns the stored value widened back to fp32 */
static float store_narrow(void *p, int dtype, int64_t i, float v) {
    switch (dtype) {
        case FO_F32: ((float *)p)[i] = v; return v;
        case FO_BF16: { uint16_t h = f32_to_bf16(v); ((uint16_t *)p)[i] = h; return bf16_to_f32(h); }
        default: { uint16_t h = f32_to_f16(v); ((uint16_t *)p)[i] = h; return f16_to_f32(h); }
    }
}

/* -------------------------------------------------------------------------- ECC (ref:2682-2776) */

static int mantissa_bits(int dtype) { return dtype == FO_F32 ? 23 : dtype == FO_BF16 ? 7 : 10; }

/* ref:2682-2712 on the raw narrow bits */
static int unbiased_exponent_bits(uint32_t abs_bits, int dtype) {
    int mant = mantissa_bits(dtype);
    int bias = dtype == FO_F16 ? 15 : 127;
    int e = (int)(abs_bits >> mant);
    return e == 0 ? 1 - bias : e - bias;
}

static uint32_t narrow_abs_bits(const void *p, int dtype, int64_t i) {
    if (dtype == FO_F32) return ((const uint32_t *)p)[i] & 0x7fffffffu;
    return ((const uint16_t *)p)[i] & 0x7fffu;
}

static int floordiv2(int x) { return (x >= 0) ? x / 2 : -((-x + 1) / 2); }

/* ref:2759-2776.  The last product and the sum are one fused multiply-add: the reference compiles with
 * FP fusion on, and only the fused form stays inside the exception budgets its own invariants test
 * records for the binades 2^-125 .. 2^-113, where c * 2^log_scale is an fp32 subnormal
 * (/root/reference/test/test_ecc_invariants.py:257-262; an unfused sum has 8192 exceptions there, the
 * budget is 32). */
static float ecc_join_one(float narrow_f32, int log_scale, float ecc, float max_val) {
    float c = ecc / max_val;
    int h = floordiv2(log_scale);
    return fmaf(c * ldexpf(1.0f, h), ldexpf(1.0f, log_scale - h), narrow_f32);
}

/* ref:2726-2756 */
static int32_t ecc_split_one(float x, float narrow_f32, int log_scale, float max_val) {
    float err = x - narrow_f32;
    int nls = -log_scale;
    int h = floordiv2(nls);
    float en = (err * ldexpf(1.0f, h)) * ldexpf(1.0f, nls - h);
    float cl = en < -1.0f ? -1.0f : (en > 1.0f ? 1.0f : en);
    float sc = cl * max_val;
    float r = copysignf(floorf(fabsf(sc) + 0.5f), sc);
    return (int32_t)r;
}

static float ecc_load(const void *ecc, int ecc_bytes, int64_t i) {
    return ecc_bytes == 1 ? (float)((const int8_t *)ecc)[i] : (float)((const int16_t *)ecc)[i];
}
static void ecc_store(void *ecc, int ecc_bytes, int64_t i, int32_t v) {
    if (ecc_bytes == 1) ((int8_t *)ecc)[i] = (int8_t)v; else ((int16_t *)ecc)[i] = (int16_t)v;
}
static float ecc_max(int ecc_bytes) { return ecc_bytes == 1 ? 127.0f : 32767.0f; } /* ref:1519-1523 */

static float read_master(const void *param, int dtype, const void *ecc, int ecc_bytes, int64_t i) {
    float pn = load_as_f32(param, dtype, i);
    if (!ecc_bytes) return pn;
    int ls = unbiased_exponent_bits(narrow_abs_bits(param, dtype, i), dtype) - mantissa_bits(dtype) - 1;
    return ecc_join_one(pn, ls, ecc_load(ecc, ecc_bytes, i), ecc_max(ecc_bytes));
}

static void write_master(void *param, int dtype, void *ecc, int ecc_bytes, int64_t i, float p) {
    float pn = store_narrow(param, dtype, i, p);
    if (!ecc_bytes) return;
    int ls = unbiased_exponent_bits(narrow_abs_bits(param, dtype, i), dtype) - mantissa_bits(dtype) - 1;
    ecc_store(ecc, ecc_bytes, i, ecc_split_one(p, pn, ls, ecc_max(ecc_bytes)));
}

void fo_oracle_ecc_join(const void *narrow, int dtype, const void *ecc, int ecc_bytes, float *out, int64_t n) {
    for (int64_t i = 0; i < n; ++i) out[i] = read_master(narrow, dtype, ecc, ecc_bytes, i);
}

void fo_oracle_ecc_split(const float *x, const void *narrow, int dtype, void *ecc, int ecc_bytes, int64_t n) {
    for (int64_t i = 0; i < n; ++i) {
        int ls = unbiased_exponent_bits(narrow_abs_bits(narrow, dtype, i), dtype) - mantissa_bits(dtype) - 1;
        ecc_store(ecc, ecc_bytes, i, ecc_split_one(x[i], load_as_f32(narrow, dtype, i), ls, ecc_max(ecc_bytes)));
    }
}

/* ------------------------------------------------------------ group codec (ref:2541-2676) --- */

static float dequant_one(float q, float in_max, int softsign, float scale, int sq) {
    float t = q / in_max;                                   /* ref:2591 */
    float nrm = softsign ? t / (2.0f - fabsf(t)) : t;       /* ref:2594-2597 */
    float x = nrm * scale;                                  /* ref:2600 */
    return sq ? x * x : x;                                  /* ref:2603-2604 */
}

/* Quantises one group held in vals[0..cnt) (already sqrt-ed when the codec wants it); returns the
 * fp32 absmax.  ref:2656-2671 */
static float quant_group(const float *vals, int cnt, int is_signed, int softsign, int32_t *codes) {
    float amax = 0.0f;
    for (int k = 0; k < cnt; ++k) { float a = fabsf(vals[k]); if (a > amax) amax = a; }
    if (amax < 1e-12f) amax = 1e-12f;
    float out_max = is_signed ? 127.0f : 255.0f;
    for (int k = 0; k < cnt; ++k) {
        float nrm = vals[k] / amax;
        float t = softsign ? (2.0f * nrm) / (1.0f + fabsf(nrm)) : nrm;
        codes[k] = (int32_t)floorf(t * out_max + 0.5f);
    }
    return amax;
}

void fo_oracle_quantize(const void *x, int dtype, void *codes, uint16_t *scales_f16, int64_t n,
                        int is_signed, int do_sqrt, int softsign) {
    float vals[FO_GROUP]; int32_t q[FO_GROUP];
    for (int64_t base = 0; base < n; base += FO_GROUP) {
        int cnt = (int)((n - base) < FO_GROUP ? (n - base) : FO_GROUP);
        for (int k = 0; k < cnt; ++k) {
            float v = load_as_f32(x, dtype, base + k);
            vals[k] = do_sqrt ? sqrtf(v) : v;               /* ref:2650-2651 */
        }
        float amax = quant_group(vals, cnt, is_signed, softsign, q);
        for (int k = 0; k < cnt; ++k) {
            if (is_signed) ((int8_t *)codes)[base + k] = (int8_t)q[k];
            else ((uint8_t *)codes)[base + k] = (uint8_t)q[k];
        }
        scales_f16[base / FO_GROUP] = f32_to_f16(amax);     /* ref:2676 */
    }
}

void fo_oracle_dequantize(const void *codes, const uint16_t *scales_f16, float *out, int64_t n,
                          int is_signed, int do_sqrt, int softsign) {
    float in_max = is_signed ? 127.0f : 255.0f;
    for (int64_t i = 0; i < n; ++i) {
        float q = is_signed ? (float)((const int8_t *)codes)[i] : (float)((const uint8_t *)codes)[i];
        out[i] = dequant_one(q, in_max, softsign, f16_to_f32(scales_f16[i / FO_GROUP]), do_sqrt);
    }
}

/* ------------------------------------------------------------------- state load / store --- */

/* quantized: state = codes (int8 if is_signed else uint8) + fp16 scales; else state = param-dtype array */
static float state_load(const void *state, const uint16_t *scales, int quantized, int dtype, int64_t i,
                        int is_signed, int do_sqrt, int softsign) {
    if (!quantized) return load_as_f32(state, dtype, i);     /* ref:2351-2354 */
    float q = is_signed ? (float)((const int8_t *)state)[i] : (float)((const uint8_t *)state)[i];
    return dequant_one(q, is_signed ? 127.0f : 255.0f, softsign, f16_to_f32(scales[i / FO_GROUP]), do_sqrt);
}

static void state_store_group(void *state, uint16_t *scales, int quantized, int dtype, int64_t base, int cnt,
                              const float *vals, int is_signed, int do_sqrt, int softsign) {
    if (!quantized) {                                        /* ref:2435-2438 */
        for (int k = 0; k < cnt; ++k) store_narrow(state, dtype, base + k, vals[k]);
        return;
    }
    float tmp[FO_GROUP] = {0.0f}; int32_t q[FO_GROUP];
    for (int k = 0; k < cnt; ++k) tmp[k] = do_sqrt ? sqrtf(vals[k]) : vals[k];   /* ref:2393 */
    float amax = quant_group(tmp, cnt, is_signed, softsign, q);
    for (int k = 0; k < cnt; ++k) {
        if (is_signed) ((int8_t *)state)[base + k] = (int8_t)q[k];
        else ((uint8_t *)state)[base + k] = (uint8_t)q[k];
    }
    scales[base / FO_GROUP] = f32_to_f16(amax);
}

static float pow_f32(float base, int step) { return (float)pow((double)base, (double)step); }

/* ------------------------------------------------------------- Adam (ref:2255-2438) --- */

void fo_oracle_adam_step(void *mom, uint16_t *mom_scales, void *var, uint16_t *var_scales, void *param,
                         const void *grad, void *ecc, int64_t n, int dtype, int ecc_bytes, int quantized,
                         float lr, float beta1, float beta2, float eps, float wd, int decoupled, int step) {
    const float one_m_b1 = 1.0f - beta1, one_m_b2 = 1.0f - beta2, one_m_wd = 1.0f - wd;
    const float bc1 = 1.0f - pow_f32(beta1, step), bc2 = 1.0f - pow_f32(beta2, step);
    float mbuf[FO_GROUP], vbuf[FO_GROUP];
    for (int64_t base = 0; base < n; base += FO_GROUP) {
        int cnt = (int)((n - base) < FO_GROUP ? (n - base) : FO_GROUP);
        for (int k = 0; k < cnt; ++k) {
            int64_t i = base + k;
            float g = load_as_f32(grad, dtype, i);
            float p = read_master(param, dtype, ecc, ecc_bytes, i);
            if (!decoupled) { float t = p * wd; g = g + t; }                   /* ref:2311 */
            float m = state_load(mom, mom_scales, quantized, dtype, i, 1, 0, 1);
            float v = state_load(var, var_scales, quantized, dtype, i, 0, 1, 0);
            { float a = m * beta1, b = g * one_m_b1; m = a + b; }               /* ref:2357 */
            { float a = v * beta2, gg = g * g, b = gg * one_m_b2; v = a + b; }   /* ref:2360 */
            if (decoupled) p = p * one_m_wd;                                    /* ref:2364 */
            float cm = m / bc1, cv = v / bc2;                                   /* ref:2370-2371 */
            float den = sqrtf(cv) + eps;                                        /* ref:2374 */
            float num = lr * cm;
            p = p - num / den;                                                  /* ref:2375 */
            write_master(param, dtype, ecc, ecc_bytes, i, p);
            mbuf[k] = m; vbuf[k] = v;
        }
        state_store_group(mom, mom_scales, quantized, dtype, base, cnt, mbuf, 1, 0, 1);
        state_store_group(var, var_scales, quantized, dtype, base, cnt, vbuf, 0, 1, 0);
    }
}

/* ---------------------------------------------- SGD / SGDW / Nesterov / Lion (ref:1586-1719) --- */

void fo_oracle_momentum_step(void *mom, uint16_t *scales, void *param, const void *grad, void *ecc, int64_t n,
                             int dtype, int ecc_bytes, int quantized, float lr, float mom_coef,
                             float update_coef, float wd, int decoupled, int nesterov, int do_lion) {
    const float one_m_wd = 1.0f - wd, one_m_uc = 1.0f - update_coef, one_m_mc = 1.0f - mom_coef;
    float mbuf[FO_GROUP];
    for (int64_t base = 0; base < n; base += FO_GROUP) {
        int cnt = (int)((n - base) < FO_GROUP ? (n - base) : FO_GROUP);
        for (int k = 0; k < cnt; ++k) {
            int64_t i = base + k;
            float g = load_as_f32(grad, dtype, i);
            float p = read_master(param, dtype, ecc, ecc_bytes, i);
            if (!do_lion && !decoupled) { float t = p * wd; g = g + t; }       /* ref:1639-1640 */
            float m = state_load(mom, scales, quantized, dtype, i, 1, 0, 1);
            if (do_lion) {
                float a = m * update_coef, b = g * one_m_uc, u = a + b;         /* ref:1667 */
                u = u > 0.0f ? 1.0f : (u < 0.0f ? -1.0f : 0.0f);                /* ref:1668 */
                float c = m * mom_coef, d = g * one_m_mc; m = c + d;            /* ref:1669 */
                p = p * one_m_wd;                                               /* ref:1675 */
                float ul = u * lr; p = p - ul;                                  /* ref:1676 */
            } else {
                float a = m * mom_coef, b = g * update_coef; m = a + b;         /* ref:1671 */
                if (decoupled) p = p * one_m_wd;                                /* ref:1679 */
                if (nesterov) { float t = mom_coef * m, s = g + t, sl = s * lr; p = p - sl; } /* ref:1681 */
                else { float ml = m * lr; p = p - ml; }                          /* ref:1683 */
            }
            write_master(param, dtype, ecc, ecc_bytes, i, p);
            mbuf[k] = m;
        }
        state_store_group(mom, scales, quantized, dtype, base, cnt, mbuf, 1, 0, 1);
    }
}

/* Momentum-free SGD: the branch the reference runs in eager PyTorch (ref:1447-1465). */
void fo_oracle_sgd_plain_step(void *param, const void *grad, void *ecc, int64_t n, int dtype, int ecc_bytes,
                              float lr, float wd, int decoupled) {
    const float one_m_wd = 1.0f - wd;
    for (int64_t i = 0; i < n; ++i) {
        float g = load_as_f32(grad, dtype, i);
        float p = read_master(param, dtype, ecc, ecc_bytes, i);
        if (!decoupled && wd > 0.0f) { float t = p * wd; g = g + t; }
        if (decoupled && wd > 0.0f) p = p * one_m_wd;
        float gl = g * lr; p = p - gl;
        write_master(param, dtype, ecc, ecc_bytes, i, p);
    }
}

/* format conversions exported for the conversion tests */
uint16_t fo_oracle_f32_to_f16(float f) { return f32_to_f16(f); }
float fo_oracle_f16_to_f32(uint16_t h) { return f16_to_f32(h); }
uint16_t fo_oracle_f32_to_bf16(float f) { return f32_to_bf16(f); }

/* ECC invariant sweep over all 2^23 fp32 mantissas of one (sign, exponent), following the
 * seven invariants of /root/reference/test/test_ecc_invariants.py:39-47,105-148.
 * exponent == -127 means the fp32 subnormal binade.  counts[0..6] receive the exception counts. */
void fo_oracle_ecc_invariants(int sign, int exponent, int dtype, int64_t *counts) {
    for (int k = 0; k < 7; ++k) counts[k] = 0;
    for (uint32_t mant = 0; mant < (1u << 23); ++mant) {
        uint32_t bits = (exponent == -127) ? mant : (((uint32_t)(exponent + 127) << 23) | mant);
        if (sign < 0) bits |= 0x80000000u;
        float x = u2f(bits);
        uint16_t nb = dtype == FO_BF16 ? f32_to_bf16(x) : f32_to_f16(x);
        float nf = dtype == FO_BF16 ? bf16_to_f32(nb) : f16_to_f32(nb);
        if (isinf(nf)) continue;
        int ls = unbiased_exponent_bits(nb & 0x7fffu, dtype) - mantissa_bits(dtype) - 1;
        int32_t e8 = ecc_split_one(x, nf, ls, 127.0f), e16 = ecc_split_one(x, nf, ls, 32767.0f);
        float r8 = ecc_join_one(nf, ls, (float)(int8_t)e8, 127.0f);
        float r16 = ecc_join_one(nf, ls, (float)(int16_t)e16, 32767.0f);
        double xd = (double)x, err0 = fabs((double)nf - xd), err8 = fabs((double)r8 - xd), err16 = fabs((double)r16 - xd);
        double ax = fabs(xd), den = ax > 0.0 ? ax : 1.0;
        double rel0 = err0 / den, rel8 = err8 / den, rel16 = err16 / den;
        const double t8 = 1.0 / 127.0, t16 = 1.0 / 32767.0;
        if (err0 == 0.0 && err8 > 0.0) counts[0]++;
        if (err0 == 0.0 && err16 > 0.0) counts[1]++;
        if (err8 == 0.0 && err16 > 0.0) counts[2]++;
        if (err16 > err8) counts[3]++;
        if (rel0 >= t8 && rel8 >= t8) counts[4]++;
        if (rel0 >= t16 && rel16 >= t16) counts[5]++;
        if (rel0 >= t16 && !(rel0 >= t8) && err16 >= err8) counts[6]++;
    }
}
