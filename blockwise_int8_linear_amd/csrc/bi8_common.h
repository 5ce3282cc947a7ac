// Shared device helpers for the gfx950 kernels of libbi8.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include "bi8.h"

#define BI8_WAVE 64

typedef int bi8_v4i __attribute__((ext_vector_type(4)));
typedef int bi8_v16i __attribute__((ext_vector_type(16)));
typedef uint32_t bi8_v4u __attribute__((ext_vector_type(4)));
typedef uint32_t bi8_v2u __attribute__((ext_vector_type(2)));
typedef float bi8_v4f __attribute__((ext_vector_type(4)));
typedef float bi8_v2f __attribute__((ext_vector_type(2)));

// Multi-dword accesses at addresses that are only aligned to the element (rows of odd length, e.g. the GPT-2
// vocabulary 50257): the amdhsa ABI runs with unaligned access enabled, so these are single instructions.
typedef bi8_v4u bi8_v4u_unaligned __attribute__((aligned(2)));
typedef bi8_v2u bi8_v2u_unaligned __attribute__((aligned(1)));
typedef uint32_t bi8_u32_unaligned __attribute__((aligned(1)));

static inline int bi8_hip_rc(hipError_t e) { return e == hipSuccess ? BI8_OK : BI8_ERR_HIP_BASE + (int)e; }
static inline int bi8_launch_rc() { return bi8_hip_rc(hipGetLastError()); }
static inline bool bi8_pow2(int64_t v) { return v > 0 && (v & (v - 1)) == 0; }
static inline bool bi8_aligned(const void *p, uintptr_t a) { return ((uintptr_t)p & (a - 1)) == 0; }
static inline size_t bi8_dtype_size(int dt) { return dt == BI8_F32 ? 4 : 2; }

// ---- element types ---------------------------------------------------------------------------
__device__ __forceinline__ float bi8_u2f(uint32_t u) { return __builtin_bit_cast(float, u); }
__device__ __forceinline__ uint32_t bi8_f2u(float f) { return __builtin_bit_cast(uint32_t, f); }

// fp32 -> bf16 bits, round to nearest even (NaN stays a quiet NaN)
__device__ __forceinline__ uint32_t bi8_bf16_bits(float f) {
    return (uint32_t)__builtin_bit_cast(uint16_t, (__bf16)f);
}
// The empty asm pins f as a rounded binary32 value: without it the backend may fold a preceding fp32
// multiply into a mixed-precision multiply-and-convert, which rounds once instead of twice.
__device__ __forceinline__ uint32_t bi8_f16_bits(float f) {
    asm volatile("" : "+v"(f));
    return (uint32_t)__builtin_bit_cast(uint16_t, (_Float16)f);
}
__device__ __forceinline__ float bi8_from_bf16_bits(uint32_t h) { return bi8_u2f(h << 16); }
__device__ __forceinline__ float bi8_from_f16_bits(uint32_t h) {
    return (float)__builtin_bit_cast(_Float16, (uint16_t)h);
}

// the value a store to `DT` followed by a load returns
template <int DT> __device__ __forceinline__ float bi8_round_to(float v) {
    if constexpr (DT == BI8_F32) return v;
    else if constexpr (DT == BI8_BF16) return bi8_from_bf16_bits(bi8_bf16_bits(v));
    else return bi8_from_f16_bits(bi8_f16_bits(v));
}

template <int DT> __device__ __forceinline__ float bi8_load_elem(const void *p, int64_t i) {
    if constexpr (DT == BI8_F32) return ((const float *)p)[i];
    else if constexpr (DT == BI8_BF16) return bi8_from_bf16_bits(((const uint16_t *)p)[i]);
    else return bi8_from_f16_bits(((const uint16_t *)p)[i]);
}

template <int DT> __device__ __forceinline__ void bi8_store_elem(void *p, int64_t i, float v) {
    if constexpr (DT == BI8_F32) ((float *)p)[i] = v;
    else if constexpr (DT == BI8_BF16) ((uint16_t *)p)[i] = (uint16_t)bi8_bf16_bits(v);
    else ((uint16_t *)p)[i] = (uint16_t)bi8_f16_bits(v);
}

// ---- 16-byte loads of floating-point elements -----------------------------------------------------
template <int DT> struct Bi8Vec {
    static constexpr int kElems = (DT == BI8_F32) ? 4 : 8;     // elements per 16-byte load
};

// 16 raw bytes -> kElems floats
template <int DT> __device__ __forceinline__ void bi8_unpack(const bi8_v4u &raw, float *f) {
    if constexpr (DT == BI8_F32) {
#pragma unroll
        for (int e = 0; e < 4; ++e) f[e] = bi8_u2f(raw[e]);
    } else if constexpr (DT == BI8_BF16) {
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            f[2 * e] = bi8_u2f(raw[e] << 16);
            f[2 * e + 1] = bi8_u2f(raw[e] & 0xffff0000u);
        }
    } else {
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            f[2 * e] = bi8_from_f16_bits(raw[e] & 0xffffu);
            f[2 * e + 1] = bi8_from_f16_bits(raw[e] >> 16);
        }
    }
}

// ---- cross-lane maximum over aligned groups of L lanes (L a power of two, 1..64) ---------------
// DPP moves for the steps inside a row of 16 lanes, ds_bpermute beyond.  max is idempotent, so the
// mirror patterns (lane i <-> 7-i, i <-> 15-i) finish the 8- and 16-lane reductions.
template <int CTRL> __device__ __forceinline__ float bi8_dpp(float v) {
    return bi8_u2f((uint32_t)__builtin_amdgcn_update_dpp(0, (int)bi8_f2u(v), CTRL, 0xf, 0xf, false));
}

template <int L> __device__ __forceinline__ float bi8_group_max(float m) {
    if constexpr (L >= 2) m = __builtin_fmaxf(m, bi8_dpp<0xB1>(m));   // quad_perm [1,0,3,2]
    if constexpr (L >= 4) m = __builtin_fmaxf(m, bi8_dpp<0x4E>(m));   // quad_perm [2,3,0,1]
    if constexpr (L >= 8) m = __builtin_fmaxf(m, bi8_dpp<0x141>(m));  // row_half_mirror
    if constexpr (L >= 16) m = __builtin_fmaxf(m, bi8_dpp<0x140>(m)); // row_mirror
    if constexpr (L >= 32) m = __builtin_fmaxf(m, __shfl_xor(m, 16, 64));
    if constexpr (L >= 64) m = __builtin_fmaxf(m, __shfl_xor(m, 32, 64));
    return m;
}

// ---- exact block quantization of one element ----------------------------------------------------
// code = rint_even( fl32( 127 * fl32( v / s ) ) ), the reference's llrint(127. * (x / max_val))
// (triton_functions.py:212).  Built with -ffp-contract=off, so the product and the magic add below
// are separate roundings.

#define BI8_MAGIC 12582912.0f      /* 1.5 * 2^23: adding it rounds to an integer, ties to even */
#define BI8_MAGIC_BITS 0x4B400000u

// Scales inside [2^-60, 2^100] take the reciprocal path; everything else (0, subnormal, huge, inf,
// NaN) takes the IEEE division.
__device__ __forceinline__ bool bi8_scale_is_ordinary(float s) {
    return s >= 8.6736173798840355e-19f && s <= 1.2676506002282294e+30f;
}

// Correctly rounded v / s from y = fl32(1/s), for |v| <= s and s ordinary: a rounded product and
// NCORR FMA corrections.  Two corrections are exact for any binary32 operands (Markstein: the first
// leaves a faithful quotient, and a faithful quotient corrected with the correctly rounded reciprocal
// is the correctly rounded quotient).  For operands widened from bf16/f16 one correction is already
// exact; that is established by exhaustion over every pair of 16-bit values on the CPU.
template <int NCORR> __device__ __forceinline__ float bi8_div_by_recip(float v, float s, float y) {
    float q = v * y;
#pragma unroll
    for (int i = 0; i < NCORR; ++i) {
        float r = __builtin_fmaf(-q, s, v);
        q = __builtin_fmaf(r, y, q);
    }
    return q;
}

// low byte of the result is the int8 code
template <int NCORR> __device__ __forceinline__ uint32_t bi8_code_fast(float v, float s, float y) {
    float t = 127.0f * bi8_div_by_recip<NCORR>(v, s, y);
    return bi8_f2u(t + BI8_MAGIC);
}

// any scale, any element: IEEE division; zero blocks and NaN elements give code 0
__device__ __forceinline__ uint32_t bi8_code_slow(float v, float s) {
    if (!(s > 0.0f) || v != v) return 0u;
    float t = 127.0f * (v / s);
    if (t != t) return 0u;                       // inf / inf
    t = __builtin_fminf(__builtin_fmaxf(t, -127.0f), 127.0f);
    return bi8_f2u(t + BI8_MAGIC);
}

__device__ __forceinline__ uint32_t bi8_pack4(uint32_t c0, uint32_t c1, uint32_t c2, uint32_t c3) {
    uint32_t lo = __builtin_amdgcn_perm(c1, c0, 0x0c0c0400u);   // byte0 = c0.b0, byte1 = c1.b0
    uint32_t hi = __builtin_amdgcn_perm(c3, c2, 0x0c0c0400u);
    return __builtin_amdgcn_perm(hi, lo, 0x05040100u);          // hi.b1 hi.b0 lo.b1 lo.b0
}
