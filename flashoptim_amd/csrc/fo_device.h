// Device-side building blocks for the gfx950 step kernels: lane-private packed I/O, dtype widening and
// narrowing, code packing, the DPP group maximum and the LDS code table (the per-element arithmetic is in fo_math.h).  Everything here is wave64 CDNA code; the file is
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
#include "fo_math.h"

namespace fo {

typedef u32 u32x2 __attribute__((ext_vector_type(2)));
typedef u32 u32x4 __attribute__((ext_vector_type(4)));
typedef float f32x2 __attribute__((ext_vector_type(2)));
typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
typedef _Float16 f16x2 __attribute__((ext_vector_type(2)));

constexpr int kTileElems = FO_TILE_ELEMS;  // unit of scheduling and of the multi-tensor chunk table (4096)

// Correctly rounded division and square root: the plain operators, which hipcc lowers to the IEEE sequences
// by default (the __fsqrt_rn intrinsic is NOT correctly rounded on this toolchain: it maps to the native
// approximate root).  Used by the cold codec kernels only.
__device__ __forceinline__ float div_rn(float a, float b) { return a / b; }
__device__ __forceinline__ float sqrt_rn(float a) { return __builtin_sqrtf(a); }

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

// Where a lane's EPL elements sit: `span` is the first element of the workgroup's span (workgroup-uniform, a
// multiple of 64 * EPL), `lane` the lane's offset inside the span in elements (lane id * EPL).
struct Where {
    int64_t span;
    int lane;
    __device__ __forceinline__ int64_t first() const { return span + lane; }
};

#define FO_GLOBAL __attribute__((address_space(1)))

// Fast path: all EPL elements are in range and the address is aligned to the access size; one vector access
// per lane.  Every stream is touched exactly once per step, hence the non-temporal hint.  The address is formed
// as a workgroup-uniform 64-bit base (scalar registers) plus a 32-bit lane offset, so a stream costs no
// 64-bit vector arithmetic, and the pointer is marked as global memory (tensor pointers read from a descriptor
// table would otherwise be accessed with the slower generic-address instructions).
template <int EB, int EPL>
__device__ __forceinline__ void load_vec(Pack<EB, EPL>& d, const void* base, Where w) {
    const FO_GLOBAL char* p = (const FO_GLOBAL char*)(static_cast<const char*>(base) + w.span * EB) + (unsigned)(w.lane * EB);
    if constexpr (Pack<EB, EPL>::kBytes == 16) {
        const u32x4 v = __builtin_nontemporal_load(reinterpret_cast<const FO_GLOBAL u32x4*>(p));
        d.w[0] = v.x; d.w[1] = v.y; d.w[2] = v.z; d.w[3] = v.w;
    } else if constexpr (Pack<EB, EPL>::kBytes == 8) {
        const u32x2 v = __builtin_nontemporal_load(reinterpret_cast<const FO_GLOBAL u32x2*>(p));
        d.w[0] = v.x; d.w[1] = v.y;
    } else {
        d.w[0] = __builtin_nontemporal_load(reinterpret_cast<const FO_GLOBAL u32*>(p));
    }
}
// Stores carry the non-temporal hint and system-scope write-through (`sc0 sc1 nt`): a streamed line goes straight
// to memory instead of sitting dirty in L2 until it is evicted, which measures 1.5 points of HBM peak better than
// `nt` alone on MI355X.  The compiler has no builtin for this policy on plain global stores, hence the asm.
// (Raw buffer stores take the policy through their builtin, but buffer accesses measured 1 point slower for the
// stores and another point for the loads than global ones in these kernels.)
// The hazard recogniser does not look inside asm: a store of more than 64 bits must be followed by two wait
// states before a VALU instruction may overwrite its data registers, hence the `s_nop 1` after the 128-bit form.
template <int EB, int EPL>
__device__ __forceinline__ void store_vec(const Pack<EB, EPL>& d, void* base, Where w) {
    char* p = static_cast<char*>(base) + w.span * EB;   // workgroup-uniform: lives in scalar registers
    const unsigned off = (unsigned)(w.lane * EB);
    if constexpr (Pack<EB, EPL>::kBytes == 16) {
        u32x4 v; v.x = d.w[0]; v.y = d.w[1]; v.z = d.w[2]; v.w = d.w[3];
        asm volatile("global_store_dwordx4 %0, %1, %2 sc0 sc1 nt\n\ts_nop 1" : : "v"(off), "v"(v), "s"(p) : "memory");
    } else if constexpr (Pack<EB, EPL>::kBytes == 8) {
        u32x2 v; v.x = d.w[0]; v.y = d.w[1];
        asm volatile("global_store_dwordx2 %0, %1, %2 sc0 sc1 nt" : : "v"(off), "v"(v), "s"(p) : "memory");
    } else {
        asm volatile("global_store_dword %0, %1, %2 sc0 sc1 nt" : : "v"(off), "v"(d.w[0]), "s"(p) : "memory");
    }
}

// The same accesses for callers whose position is a per-lane 64-bit element index (cold kernels).
template <int EB, int EPL>
__device__ __forceinline__ void load_vec(Pack<EB, EPL>& d, const void* base, int64_t first) {
    const FO_GLOBAL char* p = (const FO_GLOBAL char*)(static_cast<const char*>(base) + first * EB);
    if constexpr (Pack<EB, EPL>::kBytes == 16) {
        const u32x4 v = __builtin_nontemporal_load(reinterpret_cast<const FO_GLOBAL u32x4*>(p));
        d.w[0] = v.x; d.w[1] = v.y; d.w[2] = v.z; d.w[3] = v.w;
    } else if constexpr (Pack<EB, EPL>::kBytes == 8) {
        const u32x2 v = __builtin_nontemporal_load(reinterpret_cast<const FO_GLOBAL u32x2*>(p));
        d.w[0] = v.x; d.w[1] = v.y;
    } else {
        d.w[0] = __builtin_nontemporal_load(reinterpret_cast<const FO_GLOBAL u32*>(p));
    }
}
template <int EB, int EPL>
__device__ __forceinline__ void store_vec(const Pack<EB, EPL>& d, void* base, int64_t first) {
    char* p = static_cast<char*>(base) + first * EB;
    if constexpr (Pack<EB, EPL>::kBytes == 16) {
        u32x4 v; v.x = d.w[0]; v.y = d.w[1]; v.z = d.w[2]; v.w = d.w[3];
        asm volatile("global_store_dwordx4 %0, %1, off sc0 sc1 nt\n\ts_nop 1" : : "v"(p), "v"(v) : "memory");
    } else if constexpr (Pack<EB, EPL>::kBytes == 8) {
        u32x2 v; v.x = d.w[0]; v.y = d.w[1];
        asm volatile("global_store_dwordx2 %0, %1, off sc0 sc1 nt" : : "v"(p), "v"(v) : "memory");
    } else {
        asm volatile("global_store_dword %0, %1, off sc0 sc1 nt" : : "v"(p), "v"(d.w[0]) : "memory");
    }
}

// One fp16 group scale.  A wavefront writes 32 bytes of a 128-byte line here, so this store stays a cached
// write-back store and lets L2 merge the pieces: written through like the streams it costs 3 points of HBM peak.
__device__ __forceinline__ void store_scale(uint16_t* scales, Where w, uint16_t bits) {
    ((FO_GLOBAL uint16_t*)(scales + (w.span >> 5)))[(unsigned)(w.lane >> 5)] = bits;
}
__device__ __forceinline__ uint16_t load_scale(const uint16_t* scales, Where w) {
    return ((const FO_GLOBAL uint16_t*)(scales + (w.span >> 5)))[(unsigned)(w.lane >> 5)];
}
// per-lane 64-bit group index (cold kernels)
__device__ __forceinline__ void store_scale(uint16_t* scales, int64_t group, uint16_t bits) { ((FO_GLOBAL uint16_t*)scales)[group] = bits; }

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
__device__ __forceinline__ void load_lane(Pack<EB, EPL>& d, const void* base, Where w, int64_t n) {
    if constexpr (EB > 0) {
        if constexpr (MODE == kVector) {
            load_vec<EB, EPL>(d, base, w);
        } else if constexpr (MODE == kLane) {
            if (w.first() + EPL <= n) load_vec<EB, EPL>(d, base, w); else load_guarded<EB, EPL>(d, base, w.first(), n);
        } else {
            load_guarded<EB, EPL>(d, base, w.first(), n);
        }
    }
}
template <int EB, int EPL, int MODE>
__device__ __forceinline__ void store_lane(const Pack<EB, EPL>& d, void* base, Where w, int64_t n) {
    if constexpr (EB > 0) {
        if constexpr (MODE == kVector) {
            store_vec<EB, EPL>(d, base, w);
        } else if constexpr (MODE == kLane) {
            if (w.first() + EPL <= n) store_vec<EB, EPL>(d, base, w); else store_guarded<EB, EPL>(d, base, w.first(), n);
        } else {
            store_guarded<EB, EPL>(d, base, w.first(), n);
        }
    }
}

template <int EB, int EPL, int MODE>
__device__ __forceinline__ void load_lane(Pack<EB, EPL>& d, const void* base, int64_t first, int64_t n) {
    if constexpr (EB > 0) {
        if (MODE == kVector || (MODE == kLane && first + EPL <= n)) load_vec<EB, EPL>(d, base, first);
        else load_guarded<EB, EPL>(d, base, first, n);
    }
}
template <int EB, int EPL, int MODE>
__device__ __forceinline__ void store_lane(const Pack<EB, EPL>& d, void* base, int64_t first, int64_t n) {
    if constexpr (EB > 0) {
        if (MODE == kVector || (MODE == kLane && first + EPL <= n)) store_vec<EB, EPL>(d, base, first);
        else store_guarded<EB, EPL>(d, base, first, n);
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
// ECC streams (the arithmetic is in fo_math.h)
// ------------------------------------------------------------------------------------------------
template <int ECCB, int EPL> __device__ __forceinline__ float ecc_to_float(const Pack<ECCB, EPL>& d, int k) {
    if constexpr (ECCB == 1) return (float)(int8_t)(d.w[k / 4] >> (8 * (k % 4)));
    if constexpr (ECCB == 2) return (float)(int16_t)(d.w[k / 2] >> (16 * (k % 2)));
    return 0.0f;
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

// Converts eight floats to integers and packs the low byte of each into two dwords: a[0..3] -> lo, b[0..3] -> hi.
// KIND_A / KIND_B: kFloor = (int)floor(x) (signed first-moment codes), kTrunc = truncation (non-negative
// second-moment codes).  Each conversion writes its byte straight into the destination dword (sub-dword
// destination select), so no separate packing instructions are needed.
// The hazard recogniser does not look inside asm: on gfx940/gfx950 a VALU instruction that reads a register
// written by the preceding instruction with a sub-dword destination select needs one wait state, and a byte write
// that preserves the rest of the dword reads it.  The two chains are therefore interleaved (every dependent pair
// has an independent instruction between it) and the block ends with a wait state for whatever reads the result.
enum { kFloor = 0, kTrunc = 1 };
#define FO_CVT_FLOOR "v_cvt_flr_i32_f32_sdwa"
#define FO_CVT_TRUNC "v_cvt_i32_f32_sdwa"
#define FO_CONVERT_PACK8(OPA, OPB)                                                                          \
    asm(OPA " %0, %2 dst_sel:BYTE_0 dst_unused:UNUSED_PAD src0_sel:DWORD\n\t"                               \
        OPB " %1, %6 dst_sel:BYTE_0 dst_unused:UNUSED_PAD src0_sel:DWORD\n\t"                               \
        OPA " %0, %3 dst_sel:BYTE_1 dst_unused:UNUSED_PRESERVE src0_sel:DWORD\n\t"                          \
        OPB " %1, %7 dst_sel:BYTE_1 dst_unused:UNUSED_PRESERVE src0_sel:DWORD\n\t"                          \
        OPA " %0, %4 dst_sel:BYTE_2 dst_unused:UNUSED_PRESERVE src0_sel:DWORD\n\t"                          \
        OPB " %1, %8 dst_sel:BYTE_2 dst_unused:UNUSED_PRESERVE src0_sel:DWORD\n\t"                          \
        OPA " %0, %5 dst_sel:BYTE_3 dst_unused:UNUSED_PRESERVE src0_sel:DWORD\n\t"                          \
        OPB " %1, %9 dst_sel:BYTE_3 dst_unused:UNUSED_PRESERVE src0_sel:DWORD\n\t"                          \
        "s_nop 0"                                                                                           \
        : "=&v"(lo), "=&v"(hi)                                                                              \
        : "v"(a[0]), "v"(a[1]), "v"(a[2]), "v"(a[3]), "v"(b[0]), "v"(b[1]), "v"(b[2]), "v"(b[3]))
template <int KIND_A, int KIND_B>
__device__ __forceinline__ void convert_pack8(const float (&a)[4], const float (&b)[4], u32& lo, u32& hi) {
    if constexpr (KIND_A == kFloor && KIND_B == kFloor) FO_CONVERT_PACK8(FO_CVT_FLOOR, FO_CVT_FLOOR);
    else if constexpr (KIND_A == kTrunc && KIND_B == kTrunc) FO_CONVERT_PACK8(FO_CVT_TRUNC, FO_CVT_TRUNC);
    else if constexpr (KIND_A == kFloor && KIND_B == kTrunc) FO_CONVERT_PACK8(FO_CVT_FLOOR, FO_CVT_TRUNC);
    else FO_CONVERT_PACK8(FO_CVT_TRUNC, FO_CVT_FLOOR);
}
#undef FO_CONVERT_PACK8
#undef FO_CVT_FLOOR
#undef FO_CVT_TRUNC

// ------------------------------------------------------------------------------------------------
// 8-bit group codec pieces used by the fused kernels
// ------------------------------------------------------------------------------------------------

// max(x, x of the lane that the DPP control selects) in one instruction.  (Written as a DPP move followed by fmaxf
// the compiler emits the move, one or two canonicalising maxes and the max itself.)  v_max_f32 returns the other
// operand when one is a NaN, as fmaxf does.  A DPP source register written by the preceding VALU instruction
// needs two wait states, and the hazard recogniser does not look inside asm: hence the s_nop.
#define FO_DPP_MAX(CTRL)                                                                                           \
    asm("s_nop 1\n\tv_max_f32_dpp %0, %1, %1 " CTRL " row_mask:0xf bank_mask:0xf bound_ctrl:1" : "=&v"(r) : "v"(x))

// max over the 32/EPL neighbouring lanes that share one quantisation group; every lane gets the result
template <int EPL> __device__ __forceinline__ float group_max(float x) {
    float r;
    FO_DPP_MAX("quad_perm:[1,0,3,2]"); x = r;
    FO_DPP_MAX("quad_perm:[2,3,0,1]"); x = r;  // now the max of each aligned group of 4 lanes
    if constexpr (EPL == 4) { FO_DPP_MAX("row_half_mirror"); x = r; }  // swaps the two quads of each 8 lanes
    return x;
}
#undef FO_DPP_MAX

// The code tables (fo_math.h) in device memory, one instance per parameter dtype.
template <int DT> __device__ const StepTables<DT> kStepTables = StepTables<DT>();

// The tables a kernel uses live in LDS while it runs (1 KiB each at fixed places, no replication: a few conflicted
// reads cost less than filling a bank-replicated copy, because every short-lived workgroup fills its own).  A
// workgroup is one wavefront; it fills each table with one 128-bit load per lane that writes straight into LDS
// (lane l delivers entries 4l .. 4l+3; no registers, no ds_write).  The loads are issued before the workgroup's
// streaming loads and the first lookup only waits for them, not for the streams issued after them.
// MASK: bit t set = table t (kTableMom, kTableEcc) is used.
template <int MASK> struct StepLut {
    static constexpr int kTables = (MASK & 2) ? 2 : (MASK & 1);  // LDS reaches up to the last one used
    static constexpr int kFloats = kTables > 0 ? 256 * kTables : 4;
    __device__ __forceinline__ static void fill(float* lut, const float* table) {
#pragma unroll
        for (int t = 0; t < kTableCount; ++t)
            if ((MASK >> t) & 1)
                __builtin_amdgcn_global_load_lds((const FO_GLOBAL void*)(table + 256 * t + (threadIdx.x & 63) * 4),
                                                 (__attribute__((address_space(3))) void*)(lut + 256 * t), 16, 0, 0);
    }
};
__device__ __forceinline__ float lookup_mom(const float* lut, u32 byte) { return lut[256 * kTableMom + byte]; }
__device__ __forceinline__ float lookup_ecc(const float* lut, u32 byte) { return lut[256 * kTableEcc + byte]; }

__device__ __forceinline__ float f16_bits_to_f32(uint16_t h) { return (float)__builtin_bit_cast(_Float16, h); }
__device__ __forceinline__ uint16_t f32_to_f16_bits(float f) { return __builtin_bit_cast(uint16_t, (_Float16)f); }  // RTNE

template <int EPL> __device__ __forceinline__ u32 byte_of(const Pack<1, EPL>& d, int k) { return (d.w[k / 4] >> (8 * (k % 4))) & 0xffu; }

}  // namespace fo
