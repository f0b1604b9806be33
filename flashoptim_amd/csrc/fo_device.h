// Device-side building blocks for the gfx950 step kernels: lane-private packed I/O, dtype widening and
// narrowing, the ECC join/split and the 8-bit group codec.  Everything here is wave64 CDNA code; the file is
// compiled with -ffp-contract=off, so a fused multiply-add happens only where fmaf() is written.
//
// "ref:" cites /root/reference/flashoptim/optimizers.py.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

namespace fo {

typedef uint32_t u32;
typedef u32 u32x4 __attribute__((ext_vector_type(4)));
typedef float f32x2 __attribute__((ext_vector_type(2)));
typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
typedef _Float16 f16x2 __attribute__((ext_vector_type(2)));

constexpr int kGroup = 32;                               // ref:1549, 2219: quantisation group
constexpr int kLaneElems = 16;                           // contiguous elements owned by one lane
constexpr int kBlockThreads = 256;                       // 4 wavefronts
constexpr int kTileElems = kLaneElems * kBlockThreads;   // 4096 elements = 128 groups per block iteration
constexpr float kMagic = 12582912.0f;                    // 1.5 * 2^23: x + kMagic leaves rne(x) in the low mantissa bits

enum { DT_F32 = 0, DT_BF16 = 1, DT_F16 = 2 };

// Correctly rounded division and square root: the plain operators, which hipcc lowers to the IEEE sequences
// by default (the __fsqrt_rn intrinsic is NOT correctly rounded on this toolchain: it maps to the native
// approximate root).
__device__ __forceinline__ float div_rn(float a, float b) { return a / b; }
__device__ __forceinline__ float sqrt_rn(float a) { return __builtin_sqrtf(a); }

__device__ __forceinline__ float as_f32(u32 u) { return __builtin_bit_cast(float, u); }
__device__ __forceinline__ u32 as_u32(float f) { return __builtin_bit_cast(u32, f); }

template <int DT> struct DTypeInfo;
template <> struct DTypeInfo<DT_F32> { static constexpr int bytes = 4, mant = 23; };
template <> struct DTypeInfo<DT_BF16> { static constexpr int bytes = 2, mant = 7; };
template <> struct DTypeInfo<DT_F16> { static constexpr int bytes = 2, mant = 10; };

// ------------------------------------------------------------------------------------------------
// Lane-private packed storage: 16 elements of EB bytes each, kept as the dwords that travel to memory.
// ------------------------------------------------------------------------------------------------
template <int EB> struct Pack {
    static constexpr int kDwords = EB * kLaneElems / 4;  // 4, 8 or 16
    u32 w[kDwords];
};
template <> struct Pack<0> {
    static constexpr int kDwords = 0;
    u32 w[1];
};

// Fast path: the lane's 16 elements are in range and the base pointer is 16-byte aligned, so the lane moves
// 16*EB contiguous bytes with 128-bit accesses.  The streams are touched once per step: non-temporal hint.
template <int EB>
__device__ __forceinline__ void load_vec(Pack<EB>& d, const void* base, int64_t first) {
    const u32x4* p = reinterpret_cast<const u32x4*>(static_cast<const char*>(base) + first * EB);
#pragma unroll
    for (int i = 0; i < Pack<EB>::kDwords / 4; ++i) {
        u32x4 v = __builtin_nontemporal_load(p + i);
        d.w[4 * i + 0] = v.x; d.w[4 * i + 1] = v.y; d.w[4 * i + 2] = v.z; d.w[4 * i + 3] = v.w;
    }
}
template <int EB>
__device__ __forceinline__ void store_vec(const Pack<EB>& d, void* base, int64_t first) {
    u32x4* p = reinterpret_cast<u32x4*>(static_cast<char*>(base) + first * EB);
#pragma unroll
    for (int i = 0; i < Pack<EB>::kDwords / 4; ++i) {
        u32x4 v;
        v.x = d.w[4 * i + 0]; v.y = d.w[4 * i + 1]; v.z = d.w[4 * i + 2]; v.w = d.w[4 * i + 3];
        __builtin_nontemporal_store(v, p + i);
    }
}

// Guarded path (tensor tails, unaligned views): element-wise accesses, out-of-range elements read as zero and
// are never written (ref:1625-1630, 2296-2301 masked loads with other=0).
template <int EB>
__device__ __forceinline__ void load_guarded(Pack<EB>& d, const void* base, int64_t first, int64_t n) {
#pragma unroll
    for (int i = 0; i < Pack<EB>::kDwords; ++i) d.w[i] = 0;
#pragma unroll
    for (int k = 0; k < kLaneElems; ++k) {
        const int64_t idx = first + k;
        if (idx < n) {
            if constexpr (EB == 1) d.w[k / 4] |= (u32) static_cast<const uint8_t*>(base)[idx] << (8 * (k % 4));
            if constexpr (EB == 2) d.w[k / 2] |= (u32) static_cast<const uint16_t*>(base)[idx] << (16 * (k % 2));
            if constexpr (EB == 4) d.w[k] = static_cast<const u32*>(base)[idx];
        }
    }
}
template <int EB>
__device__ __forceinline__ void store_guarded(const Pack<EB>& d, void* base, int64_t first, int64_t n) {
#pragma unroll
    for (int k = 0; k < kLaneElems; ++k) {
        const int64_t idx = first + k;
        if (idx < n) {
            if constexpr (EB == 1) static_cast<uint8_t*>(base)[idx] = (uint8_t)(d.w[k / 4] >> (8 * (k % 4)));
            if constexpr (EB == 2) static_cast<uint16_t*>(base)[idx] = (uint16_t)(d.w[k / 2] >> (16 * (k % 2)));
            if constexpr (EB == 4) static_cast<u32*>(base)[idx] = d.w[k];
        }
    }
}
template <int EB, bool FAST>
__device__ __forceinline__ void load_lane(Pack<EB>& d, const void* base, int64_t first, int64_t n) {
    if constexpr (EB > 0) {
        if constexpr (FAST) load_vec<EB>(d, base, first); else load_guarded<EB>(d, base, first, n);
    }
}
template <int EB, bool FAST>
__device__ __forceinline__ void store_lane(const Pack<EB>& d, void* base, int64_t first, int64_t n) {
    if constexpr (EB > 0) {
        if constexpr (FAST) store_vec<EB>(d, base, first); else store_guarded<EB>(d, base, first, n);
    }
}

// ------------------------------------------------------------------------------------------------
// widening / narrowing of the parameter dtype
// ------------------------------------------------------------------------------------------------
template <int DT> __device__ __forceinline__ float widen(const Pack<DTypeInfo<DT>::bytes>& d, int k) {
    if constexpr (DT == DT_F32) return as_f32(d.w[k]);
    if constexpr (DT == DT_BF16) return as_f32((k & 1) ? (d.w[k / 2] & 0xffff0000u) : (d.w[k / 2] << 16));
    if constexpr (DT == DT_F16) {
        f16x2 h = __builtin_bit_cast(f16x2, d.w[k / 2]);
        return (float)((k & 1) ? h.y : h.x);
    }
}

// Round to nearest even into the parameter dtype (ref:2377 param.to(PARAM_DTYPE)); writes elements k, k+1
// and returns them widened back.  bf16 pairs use the gfx950 packed convert.
template <int DT>
__device__ __forceinline__ void narrow_pair(Pack<DTypeInfo<DT>::bytes>& d, int k, float a, float b, float& wa, float& wb) {
    if constexpr (DT == DT_F32) {
        d.w[k] = as_u32(a); d.w[k + 1] = as_u32(b); wa = a; wb = b;
    }
    if constexpr (DT == DT_BF16) {
        f32x2 f = {a, b};
        u32 w = __builtin_bit_cast(u32, __builtin_convertvector(f, bf16x2));
        d.w[k / 2] = w; wa = as_f32(w << 16); wb = as_f32(w & 0xffff0000u);
    }
    if constexpr (DT == DT_F16) {
        f16x2 h = {(_Float16)a, (_Float16)b};
        d.w[k / 2] = __builtin_bit_cast(u32, h); wa = (float)h.x; wb = (float)h.y;
    }
}

// ------------------------------------------------------------------------------------------------
// ECC: narrow value + signed integer fraction of half its ulp (ref:2682-2776)
// ------------------------------------------------------------------------------------------------
template <int ECCB> struct EccInfo;
template <> struct EccInfo<1> { static constexpr float max_val = 127.0f; };      // ref:1521
template <> struct EccInfo<2> { static constexpr float max_val = 32767.0f; };    // ref:1523

// Biased exponent field of the narrow value given its widened fp32 bits, with zero/subnormal mapped to the
// smallest normal exponent (ref:2704-2712).  bf16 shares fp32's field; fp16's is recovered from the fp32 one
// (an fp16 subnormal widens to an fp32 normal with exponent < -14, which the max() maps back to -14).
template <int DT> __device__ __forceinline__ int narrow_exp_field(float widened) {
    const int e = (int)((as_u32(widened) >> 23) & 0xffu);
    if constexpr (DT == DT_F16) return max(e, 127 - 14);
    return max(e, 1);
}

template <int ECCB> __device__ __forceinline__ float ecc_to_float(const Pack<ECCB>& d, int k) {
    if constexpr (ECCB == 1) return (float)(int8_t)(d.w[k / 4] >> (8 * (k % 4)));
    if constexpr (ECCB == 2) return (float)(int16_t)(d.w[k / 2] >> (16 * (k % 2)));
    return 0.0f;
}

// x_narrow + (ecc / MAX) * 2^(E - mant - 1) with the product and the sum fused (ref:2767-2776; the reference
// compiles with FP fusion, and its invariants test only passes with the fused form).
//   ecc / MAX is formed exactly rounded as fma(e, K_hi, e * K_lo) with K_hi + K_lo = 2^-(mant+1) / MAX to
//   well beyond fp32 precision (checked exhaustively over every int8 / int16 value on the host);
//   2^E comes straight from the exponent field; inf/NaN inputs (field 255) are clamped to 254.
template <int DT, int ECCB> __device__ __forceinline__ float ecc_join(float widened, float ecc) {
    constexpr double k = 1.0 / ((double)EccInfo<ECCB>::max_val * (double)(1 << (DTypeInfo<DT>::mant + 1)));
    constexpr float k_hi = (float)k;
    constexpr float k_lo = (float)(k - (double)k_hi);
    const float c = fmaf(ecc, k_hi, ecc * k_lo);
    const int e = min(narrow_exp_field<DT>(widened), 254);
    return fmaf(c, as_f32((u32)e << 23), widened);
}

// Signed fraction of half an ulp of the NEW narrow value, scaled to +-MAX and rounded half away from zero
// (ref:2735-2756).  Returns a word whose low byte / half is the two's-complement code.
//   General form: sc = clamp(en) * MAX rounded to fp32 as in the reference, then trunc(sc + copysign(0.5, sc)),
//   which equals copysign(floor(|sc| + 0.5), sc) including the fp32 rounding of the sum.
//   bf16 with an int8 code: p - narrow is exact and a multiple of 2^-16 half-ulps, so en * 127 fits 24 bits and
//   is exact; the only tie that can occur is +-63.5, where half-even and half-away agree.  One fma against
//   1.5 * 2^23 then leaves the rounded integer in the low mantissa bits.
template <int DT, int ECCB> __device__ __forceinline__ u32 ecc_split_bits(float p, float widened) {
    const float err = p - widened;
    const int nls = (DTypeInfo<DT>::mant + 1 + 127) - narrow_exp_field<DT>(widened);
    const float en = __builtin_amdgcn_ldexpf(err, nls);
    const float cl = __builtin_amdgcn_fmed3f(en, -1.0f, 1.0f);
    if constexpr (DT == DT_BF16 && ECCB == 1) {
        return as_u32(fmaf(cl, EccInfo<ECCB>::max_val, kMagic));
    } else {
        const float sc = cl * EccInfo<ECCB>::max_val;
        return (u32)(int)(sc + __builtin_copysignf(0.5f, sc));
    }
}

// Gathers the low byte (or low half) of consecutive magic-rounded words into packed storage.
__device__ __forceinline__ u32 pack_bytes4(u32 a, u32 b, u32 c, u32 d) {
    const u32 lo = __builtin_amdgcn_perm(b, a, 0x0c0c0400u);  // a.b0 | b.b0 << 8
    const u32 hi = __builtin_amdgcn_perm(d, c, 0x04000c0cu);  // c.b0 << 16 | d.b0 << 24
    return lo | hi;
}
__device__ __forceinline__ u32 pack_halves2(u32 a, u32 b) { return __builtin_amdgcn_perm(b, a, 0x05040100u); }

// ------------------------------------------------------------------------------------------------
// 8-bit group codec pieces used by the fused kernels
// ------------------------------------------------------------------------------------------------

// value of lane (id ^ 1): the two lanes that share a 32-element group are neighbours
__device__ __forceinline__ float pair_swap(float x) {
    return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, x), 0xB1, 0xf, 0xf, true));
}

// rn(q / 255) for q in 0..255, exact: fma(q, hi, q*lo) with hi+lo = 1/255 (checked exhaustively on the host)
__device__ __forceinline__ float code255_to_unit(float q) {
    constexpr float hi = (float)(1.0 / 255.0);
    constexpr float lo = (float)(1.0 / 255.0 - (double)hi);
    return fmaf(q, hi, q * lo);
}

// Dequantised first-moment magnitude for signed code byte b, before the scale: (q/127) / (2 - |q/127|)
// (ref:2332-2336), IEEE-rounded at each step.  Filled once per block into a bank-replicated LDS table.
__device__ __forceinline__ float softsign_inverse_of_code(int q) {
    const float y = div_rn((float)q, 127.0f);
    return div_rn(y, 2.0f - fabsf(y));
}

constexpr int kLutFloats = 256 * 32;  // 32 KiB: entry for code byte b and lane l lives at [b*32 + (l & 31)]

// One thread per code value writes its 32 bank copies, so later lookups never conflict: lane l always reads
// bank l & 31 whatever its code is.
__device__ __forceinline__ void build_softsign_lut(float* lut) {
    const int b = threadIdx.x;  // blockDim.x == 256
    const float v = softsign_inverse_of_code((int)(int8_t)b);
    float4 v4 = make_float4(v, v, v, v);
    float4* row = reinterpret_cast<float4*>(lut + b * 32);
#pragma unroll
    for (int i = 0; i < 8; ++i) row[i] = v4;
    __syncthreads();
}

__device__ __forceinline__ float f16_bits_to_f32(uint16_t h) { return (float)__builtin_bit_cast(_Float16, h); }
__device__ __forceinline__ uint16_t f32_to_f16_bits(float f) { return __builtin_bit_cast(uint16_t, (_Float16)f); }  // RTNE

__device__ __forceinline__ u32 byte_of(const Pack<1>& d, int k) { return (d.w[k / 4] >> (8 * (k % 4))) & 0xffu; }

}  // namespace fo
