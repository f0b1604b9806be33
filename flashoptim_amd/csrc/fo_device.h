// Device-side building blocks for the gfx950 step kernels: lane-private packed I/O, dtype widening and
// narrowing, the ECC join/split and the 8-bit group codec.  Everything here is wave64 CDNA code; the file is
// compiled with -ffp-contract=off, so a fused multiply-add happens only where fmaf() is written.
//
// Access shape.  A wavefront works on one "sub-tile" at a time: 64 lanes x EPL consecutive elements, where
// EPL = 16 bytes / sizeof(parameter element) (8 for bf16/fp16, 4 for fp32).  Lane l owns elements
// [l*EPL, (l+1)*EPL) of the sub-tile, so every parameter/gradient access is one 128-bit load or store per
// lane and consecutive lanes touch consecutive 16-byte pieces: each wave-level instruction covers 1 KiB of
// contiguous memory.  The 1-byte streams (codes, int8 ECC) move EPL bytes per lane (64- or 32-bit accesses,
// again contiguous across the wave).  A 32-element quantisation group is 32/EPL neighbouring lanes (a DPP
// quad for bf16/fp16), so the group absmax needs no LDS.
//
// "ref:" cites /root/reference/flashoptim/optimizers.py.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include "../../include/flashoptim_hip.h"

namespace fo {

typedef uint32_t u32;
typedef u32 u32x2 __attribute__((ext_vector_type(2)));
typedef u32 u32x4 __attribute__((ext_vector_type(4)));
typedef float f32x2 __attribute__((ext_vector_type(2)));
typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
typedef _Float16 f16x2 __attribute__((ext_vector_type(2)));

constexpr int kGroup = 32;             // ref:1549, 2219: quantisation group
constexpr int kTileElems = FO_TILE_ELEMS;  // unit of scheduling and of the multi-tensor chunk table (4096)
constexpr float kMagic = 12582912.0f;  // 1.5 * 2^23: x + kMagic leaves rne(x) in the low mantissa bits

enum { DT_F32 = 0, DT_BF16 = 1, DT_F16 = 2 };

// Correctly rounded division and square root: the plain operators, which hipcc lowers to the IEEE sequences
// by default (the __fsqrt_rn intrinsic is NOT correctly rounded on this toolchain: it maps to the native
// approximate root).
__device__ __forceinline__ float div_rn(float a, float b) { return a / b; }
__device__ __forceinline__ float sqrt_rn(float a) { return __builtin_sqrtf(a); }

__device__ __forceinline__ float as_f32(u32 u) { return __builtin_bit_cast(float, u); }
__device__ __forceinline__ u32 as_u32(float f) { return __builtin_bit_cast(u32, f); }

template <int DT> struct DTypeInfo;
template <> struct DTypeInfo<DT_F32> { static constexpr int bytes = 4, mant = 23, epl = 4; };
template <> struct DTypeInfo<DT_BF16> { static constexpr int bytes = 2, mant = 7, epl = 8; };
template <> struct DTypeInfo<DT_F16> { static constexpr int bytes = 2, mant = 10, epl = 8; };

// ------------------------------------------------------------------------------------------------
// Lane-private packed storage: EPL elements of EB bytes each (4, 8 or 16 bytes in total), kept as the
// dwords that travel to memory.  EB == 0 is an absent stream.
// ------------------------------------------------------------------------------------------------
template <int EB, int EPL> struct Pack {
    static constexpr int kBytes = EB * EPL;
    static constexpr int kDwords = kBytes / 4;
    static_assert(kBytes == 4 || kBytes == 8 || kBytes == 16, "a lane moves 4, 8 or 16 bytes per stream");
    u32 w[kDwords];
};
template <int EPL> struct Pack<0, EPL> {
    static constexpr int kBytes = 0;
    static constexpr int kDwords = 0;
    u32 w[1];
};

// Fast path: all EPL elements are in range and the address is aligned to the access size; one vector access
// per lane.  Every stream is touched exactly once per step, hence the non-temporal hint.
template <int EB, int EPL>
__device__ __forceinline__ void load_vec(Pack<EB, EPL>& d, const void* base, int64_t first) {
    const char* p = static_cast<const char*>(base) + first * EB;
    if constexpr (Pack<EB, EPL>::kBytes == 16) {
        const u32x4 v = __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(p));
        d.w[0] = v.x; d.w[1] = v.y; d.w[2] = v.z; d.w[3] = v.w;
    } else if constexpr (Pack<EB, EPL>::kBytes == 8) {
        const u32x2 v = __builtin_nontemporal_load(reinterpret_cast<const u32x2*>(p));
        d.w[0] = v.x; d.w[1] = v.y;
    } else {
        d.w[0] = __builtin_nontemporal_load(reinterpret_cast<const u32*>(p));
    }
}
// Stores carry the non-temporal hint and system-scope write-through (`sc0 sc1 nt`): a streamed line goes straight
// to memory instead of sitting dirty in L2 until it is evicted, which measures 1.5 points of HBM peak better than
// `nt` alone on MI355X.  The compiler has no builtin for this policy on plain global stores, hence the asm.
// (Raw buffer stores take the policy through their builtin, but buffer accesses measured 1 point slower for the
// stores and another point for the loads than global ones in these kernels.)
// The hazard recogniser does not look inside asm: a store of more than 64 bits must be followed by two wait
// states before a VALU instruction may overwrite its data registers, hence the `s_nop 1` after the 128-bit form.
#ifndef FO_STORE_WRITE_THROUGH
#define FO_STORE_WRITE_THROUGH 1
#endif
template <int EB, int EPL>
__device__ __forceinline__ void store_vec(const Pack<EB, EPL>& d, void* base, int64_t first) {
    char* p = static_cast<char*>(base) + first * EB;
    if constexpr (Pack<EB, EPL>::kBytes == 16) {
        u32x4 v; v.x = d.w[0]; v.y = d.w[1]; v.z = d.w[2]; v.w = d.w[3];
#if FO_STORE_WRITE_THROUGH
        asm volatile("global_store_dwordx4 %0, %1, off sc0 sc1 nt\n\ts_nop 1" : : "v"(p), "v"(v) : "memory");
#else
        __builtin_nontemporal_store(v, reinterpret_cast<u32x4*>(p));
#endif
    } else if constexpr (Pack<EB, EPL>::kBytes == 8) {
        u32x2 v; v.x = d.w[0]; v.y = d.w[1];
#if FO_STORE_WRITE_THROUGH
        asm volatile("global_store_dwordx2 %0, %1, off sc0 sc1 nt" : : "v"(p), "v"(v) : "memory");
#else
        __builtin_nontemporal_store(v, reinterpret_cast<u32x2*>(p));
#endif
    } else {
#if FO_STORE_WRITE_THROUGH
        asm volatile("global_store_dword %0, %1, off sc0 sc1 nt" : : "v"(p), "v"(d.w[0]) : "memory");
#else
        __builtin_nontemporal_store(d.w[0], reinterpret_cast<u32*>(p));
#endif
    }
}

// One fp16 group scale.  A wavefront writes 32 bytes of a 128-byte line here, so this store stays a cached
// write-back store and lets L2 merge the pieces: written through like the streams it costs 3 points of HBM peak.
__device__ __forceinline__ void store_scale(uint16_t* scales, int64_t group, uint16_t bits) { scales[group] = bits; }

// Guarded path (tensor tails, unaligned views): element-wise accesses, out-of-range elements read as zero and
// are never written (ref:1625-1630, 2296-2301 masked loads with other=0).
template <int EB, int EPL>
__device__ __forceinline__ void load_guarded(Pack<EB, EPL>& d, const void* base, int64_t first, int64_t n) {
#pragma unroll
    for (int i = 0; i < Pack<EB, EPL>::kDwords; ++i) d.w[i] = 0;
#pragma unroll
    for (int k = 0; k < EPL; ++k) {
        const int64_t idx = first + k;
        if (idx < n) {
            if constexpr (EB == 1) d.w[k / 4] |= (u32) static_cast<const uint8_t*>(base)[idx] << (8 * (k % 4));
            if constexpr (EB == 2) d.w[k / 2] |= (u32) static_cast<const uint16_t*>(base)[idx] << (16 * (k % 2));
            if constexpr (EB == 4) d.w[k] = static_cast<const u32*>(base)[idx];
        }
    }
}
template <int EB, int EPL>
__device__ __forceinline__ void store_guarded(const Pack<EB, EPL>& d, void* base, int64_t first, int64_t n) {
#pragma unroll
    for (int k = 0; k < EPL; ++k) {
        const int64_t idx = first + k;
        if (idx < n) {
            if constexpr (EB == 1) static_cast<uint8_t*>(base)[idx] = (uint8_t)(d.w[k / 4] >> (8 * (k % 4)));
            if constexpr (EB == 2) static_cast<uint16_t*>(base)[idx] = (uint16_t)(d.w[k / 2] >> (16 * (k % 2)));
            if constexpr (EB == 4) static_cast<u32*>(base)[idx] = d.w[k];
        }
    }
}
// How a lane reaches its EPL elements of a stream:
//   kVector   one vector access, no checks (the whole span is in range and every stream is 16-byte aligned);
//   kLane     aligned streams, span cut by the end of the tensor: lanes that are entirely in range still use the
//             vector access, only the lane that straddles the end goes element by element;
//   kGuarded  element by element (unaligned views).
enum { kGuarded = 0, kVector = 1, kLane = 2 };

template <int EB, int EPL, int MODE>
__device__ __forceinline__ void load_lane(Pack<EB, EPL>& d, const void* base, int64_t first, int64_t n) {
    if constexpr (EB > 0) {
        if constexpr (MODE == kVector) {
            load_vec<EB, EPL>(d, base, first);
        } else if constexpr (MODE == kLane) {
            if (first + EPL <= n) load_vec<EB, EPL>(d, base, first); else load_guarded<EB, EPL>(d, base, first, n);
        } else {
            load_guarded<EB, EPL>(d, base, first, n);
        }
    }
}
template <int EB, int EPL, int MODE>
__device__ __forceinline__ void store_lane(const Pack<EB, EPL>& d, void* base, int64_t first, int64_t n) {
    if constexpr (EB > 0) {
        if constexpr (MODE == kVector) {
            store_vec<EB, EPL>(d, base, first);
        } else if constexpr (MODE == kLane) {
            if (first + EPL <= n) store_vec<EB, EPL>(d, base, first); else store_guarded<EB, EPL>(d, base, first, n);
        } else {
            store_guarded<EB, EPL>(d, base, first, n);
        }
    }
}

// ------------------------------------------------------------------------------------------------
// widening / narrowing of the parameter dtype
// ------------------------------------------------------------------------------------------------
template <int DT, int EPL> __device__ __forceinline__ float widen(const Pack<DTypeInfo<DT>::bytes, EPL>& d, int k) {
    if constexpr (DT == DT_F32) return as_f32(d.w[k]);
    if constexpr (DT == DT_BF16) return as_f32((k & 1) ? (d.w[k / 2] & 0xffff0000u) : (d.w[k / 2] << 16));
    if constexpr (DT == DT_F16) {
        f16x2 h = __builtin_bit_cast(f16x2, d.w[k / 2]);
        return (float)((k & 1) ? h.y : h.x);
    }
}

// Round to nearest even into the parameter dtype (ref:2377 param.to(PARAM_DTYPE)); writes elements k, k+1
// and returns them widened back.  bf16 pairs use the gfx950 packed convert.
template <int DT, int EPL>
__device__ __forceinline__ void narrow_pair(Pack<DTypeInfo<DT>::bytes, EPL>& d, int k, float a, float b, float& wa, float& wb) {
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

// fp32 bit pattern of 2^E, E = unbiased exponent of the narrow value with zero/subnormal mapped to the
// smallest normal exponent (ref:2704-2712), given the value widened to fp32.  bf16 shares fp32's exponent
// field; an fp16 subnormal widens to an fp32 normal below 2^-14, which the lower clamp maps back to -14.
// The upper clamp keeps inf/NaN inputs from producing an infinite scale.
template <int DT> __device__ __forceinline__ u32 pow2_of_exponent_bits(float widened) {
    constexpr u32 lo = (DT == DT_F16) ? ((127u - 14u) << 23) : (1u << 23);
    const u32 e = as_u32(widened) & 0x7f800000u;
    return min(max(e, lo), 254u << 23);
}

template <int ECCB, int EPL> __device__ __forceinline__ float ecc_to_float(const Pack<ECCB, EPL>& d, int k) {
    if constexpr (ECCB == 1) return (float)(int8_t)(d.w[k / 4] >> (8 * (k % 4)));
    if constexpr (ECCB == 2) return (float)(int16_t)(d.w[k / 2] >> (16 * (k % 2)));
    return 0.0f;
}

// x_narrow + (ecc / MAX) * 2^(E - mant - 1) with the product and the sum fused (ref:2767-2776; the reference
// compiles with FP fusion, and its invariants test only passes with the fused form).
//   ecc / MAX is formed exactly rounded as fma(e, K_hi, e * K_lo) with K_hi + K_lo = 2^-(mant+1) / MAX to
//   well beyond fp32 precision (checked exhaustively over every int8 / int16 value on the host).
template <int DT, int ECCB> __device__ __forceinline__ float ecc_join(float widened, float ecc) {
    constexpr double k = 1.0 / ((double)EccInfo<ECCB>::max_val * (double)(1 << (DTypeInfo<DT>::mant + 1)));
    constexpr float k_hi = (float)k;
    constexpr float k_lo = (float)(k - (double)k_hi);
    const float c = fmaf(ecc, k_hi, ecc * k_lo);
    return fmaf(c, as_f32(pow2_of_exponent_bits<DT>(widened)), widened);
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
template <int DT, int ECCB, bool CLAMP> __device__ __forceinline__ u32 ecc_split_bits(float p, float widened) {
    const float err = p - widened;
    if constexpr (DT == DT_BF16 && ECCB == 1 && !CLAMP) {
        const float s = as_f32(0x7ffe0000u - pow2_of_exponent_bits<DT>(widened));
        return as_u32(fmaf(err, s, 1536.0f));
    } else {
        const int nls = (DTypeInfo<DT>::mant + 1 + 127) - (int)(pow2_of_exponent_bits<DT>(widened) >> 23);
        float en = __builtin_amdgcn_ldexpf(err, nls);
        if constexpr (CLAMP) en = __builtin_amdgcn_fmed3f(en, -1.0f, 1.0f);
        if constexpr (DT == DT_BF16 && ECCB == 1) {
            return as_u32(fmaf(en, EccInfo<ECCB>::max_val, kMagic));
        } else {
            const float sc = en * EccInfo<ECCB>::max_val;
            return (u32)(int)(sc + __builtin_copysignf(0.5f, sc));
        }
    }
}

// Gathers the low byte (or low half) of consecutive code words into packed storage.
__device__ __forceinline__ u32 pack_bytes4(u32 a, u32 b, u32 c, u32 d) {
    const u32 lo = __builtin_amdgcn_perm(b, a, 0x0c0c0400u);  // a.b0 | b.b0 << 8
    const u32 hi = __builtin_amdgcn_perm(d, c, 0x04000c0cu);  // c.b0 << 16 | d.b0 << 24
    return lo | hi;
}
__device__ __forceinline__ u32 pack_halves2(u32 a, u32 b) { return __builtin_amdgcn_perm(b, a, 0x05040100u); }

template <int EB, int EPL> __device__ __forceinline__ void pack_codes(const u32 (&c)[EPL], Pack<EB, EPL>& out) {
    if constexpr (EB == 1) {
#pragma unroll
        for (int i = 0; i < EPL / 4; ++i) out.w[i] = pack_bytes4(c[4 * i], c[4 * i + 1], c[4 * i + 2], c[4 * i + 3]);
    }
    if constexpr (EB == 2) {
#pragma unroll
        for (int i = 0; i < EPL / 2; ++i) out.w[i] = pack_halves2(c[2 * i], c[2 * i + 1]);
    }
}

// ------------------------------------------------------------------------------------------------
// 8-bit group codec pieces used by the fused kernels
// ------------------------------------------------------------------------------------------------

template <int CTRL> __device__ __forceinline__ float dpp_move(float x) {
    return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, x), CTRL, 0xf, 0xf, true));
}

// max over the 32/EPL neighbouring lanes that share one quantisation group; every lane gets the result
template <int EPL> __device__ __forceinline__ float group_max(float x) {
    x = fmaxf(x, dpp_move<0xB1>(x));  // quad_perm [1,0,3,2]
    x = fmaxf(x, dpp_move<0x4E>(x));  // quad_perm [2,3,0,1]: now the max of each aligned group of 4 lanes
    if constexpr (EPL == 4) x = fmaxf(x, dpp_move<0x141>(x));  // row_half_mirror: swaps the two quads of each 8 lanes
    return x;
}

// Dequantised first-moment magnitude for signed code byte b, before the scale:
// (q/127) / (2 - |q/127|) (ref:2332-2336), each operation correctly rounded.  Evaluated by the compiler.
struct SoftsignTable {
    float v[256];
    constexpr SoftsignTable() : v() {
        for (int b = 0; b < 256; ++b) {
            const int q = b < 128 ? b : b - 256;
            const float y = (float)q / 127.0f;
            const float a = y < 0.0f ? -y : y;
            v[b] = y / (2.0f - a);
        }
    }
};
__device__ const SoftsignTable kSoftsignTable = SoftsignTable();

// The table lives in LDS during a kernel.  REPL copies per entry; a lane uses copy (lane % REPL).
// REPL = 32 would give every lane its own bank; REPL = 1 (1 KiB) costs a few conflicted reads but fills with
// one store per thread, which matters because every short-lived workgroup fills its own copy.
// Filling is split so that the global read of the table is in flight together with the workgroup's streaming
// loads: fetch() first, commit() (LDS stores + barrier) just before the first lookup.  T = workgroup size.
template <int REPL, int T> struct Lut {
    static constexpr int kFloats = 256 * REPL;
    static constexpr int kPerThread = T >= 256 ? 1 : 256 / T;  // table entries a thread copies
    struct Frag { float v[kPerThread]; };
    __device__ __forceinline__ static Frag fetch() {
        Frag f;
        const float* src = kSoftsignTable.v + (threadIdx.x & (256 / kPerThread - 1)) * kPerThread;
#pragma unroll
        for (int j = 0; j < kPerThread; ++j) f.v[j] = src[j];
        return f;
    }
    __device__ __forceinline__ static void commit(float* lut, const Frag& f) {
        if (T <= 256 || threadIdx.x < 256) {
#pragma unroll
            for (int j = 0; j < kPerThread; ++j)
#pragma unroll
                for (int i = 0; i < REPL; ++i) lut[(threadIdx.x * kPerThread + j) * REPL + i] = f.v[j];
        }
        __syncthreads();  // a single-wavefront workgroup needs no hardware barrier; the compiler drops it
    }
    __device__ __forceinline__ static const float* lane_base(const float* lut) { return lut + (threadIdx.x & (REPL - 1)); }
    __device__ __forceinline__ static float lookup(const float* lane_lut, u32 byte) { return lane_lut[byte * REPL]; }
};

__device__ __forceinline__ float f16_bits_to_f32(uint16_t h) { return (float)__builtin_bit_cast(_Float16, h); }
__device__ __forceinline__ uint16_t f32_to_f16_bits(float f) { return __builtin_bit_cast(uint16_t, (_Float16)f); }  // RTNE

template <int EPL> __device__ __forceinline__ u32 byte_of(const Pack<1, EPL>& d, int k) { return (d.w[k / 4] >> (8 * (k % 4))) & 0xffu; }

}  // namespace fo
