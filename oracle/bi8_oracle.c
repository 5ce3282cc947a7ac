/*
 * TEST INFRASTRUCTURE -- NOT PRODUCT CODE.
 *
 * Scalar CPU restatement of the reference's blockwise int8 arithmetic.  It is
 * the checker the HIP kernels are compared against and the CPU baseline that
 * the benchmark times; nothing in the shipped package may call it.
 *
 * Every routine follows the reference's Triton kernels line by line, in IEEE
 * binary32 with no FMA contraction (build with -ffp-contract=off, no
 * -ffast-math):
 *
 *   bi8o_quantize_rowwise    triton_functions.py:207-216 (loop), :221-233 (layout)
 *   bi8o_dequantize_rowwise  triton_functions.py:483-490, :492-500
 *   bi8o_gemm_nt_partials    triton_functions.py:115 (tl.dot int8 -> int32)
 *   bi8o_gemm_nt_dequant     triton_functions.py:106-131, :142-168
 *   bi8o_quantize_transposed block_linear.py:93-94, :100-103
 *                            (x.t().contiguous() followed by the row quantizer)
 *
 * Pinned (see tests/test_oracle_*.py): hand known-answer vectors, exact
 * rational brute force on small inputs, closed-form invariants, int64 einsum
 * for the partials.  No routine here is "parity unpinned".
 *
 * Two cases the reference leaves undefined are defined here, and the HIP
 * kernels follow the same definition:
 *   - an all-zero block has scale 0 and codes 0 (the reference divides 0/0);
 *   - NaN elements do not contribute to the block maximum and get code 0.
 */
#include <math.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

#define BI8O_F32 0
#define BI8O_BF16 1
#define BI8O_F16 2

static inline float u2f(uint32_t u) { float f; memcpy(&f, &u, 4); return f; }
static inline uint32_t f2u(float f) { uint32_t u; memcpy(&u, &f, 4); return u; }

static inline float bf16_to_f32(uint16_t h) { return u2f((uint32_t)h << 16); }

/* round-to-nearest-even, NaN kept quiet */
static inline uint16_t f32_to_bf16(float f) {
    uint32_t u = f2u(f);
    if ((u & 0x7fffffffu) > 0x7f800000u) return (uint16_t)((u >> 16) | 0x0040u);
    u += 0x7fffu + ((u >> 16) & 1u);
    return (uint16_t)(u >> 16);
}

static inline float f16_to_f32(uint16_t h) {
    uint32_t sign = (uint32_t)(h & 0x8000u) << 16;
    uint32_t exp = (h >> 10) & 0x1fu;
    uint32_t man = h & 0x3ffu;
    if (exp == 0) {
        if (man == 0) return u2f(sign);
        /* subnormal half: man * 2^-24, exact in binary32 */
        float v = (float)man * 5.9604644775390625e-08f;
        return sign ? -v : v;
    }
    if (exp == 31) return u2f(sign | 0x7f800000u | (man << 13));
    return u2f(sign | ((exp + 112u) << 23) | (man << 13));
}

/* round-to-nearest-even binary32 -> binary16 */
static inline uint16_t f32_to_f16(float f) {
    uint32_t u = f2u(f);
    uint16_t sign = (uint16_t)((u >> 16) & 0x8000u);
    uint32_t a = u & 0x7fffffffu;
    if (a > 0x7f800000u) return (uint16_t)(sign | 0x7e00u);
    if (a >= 0x47800000u) return (uint16_t)(sign | 0x7c00u);          /* >= 65536 -> inf (65520 rounds up below) */
    if (a < 0x33000000u) return sign;                                   /* < 2^-25 -> 0 */
    int e = (int)(a >> 23) - 127;
    uint32_t m = (a & 0x7fffffu) | 0x800000u;
    int shift = (e < -14) ? (13 + (-14 - e)) : 13;
    uint32_t q = m >> shift;
    uint32_t rem = m & ((1u << shift) - 1u);
    uint32_t half = 1u << (shift - 1);
    if (rem > half || (rem == half && (q & 1u))) q++;
    uint32_t out;
    if (e < -14) out = q;                                               /* subnormal (q may carry into exp 1) */
    else out = ((uint32_t)(e + 15) << 10) + (q - 0x400u);               /* carry propagates into the exponent */
    if (out >= 0x7c00u) out = 0x7c00u;
    return (uint16_t)(sign | out);
}

static inline float load_as_f32(const void *p, int dtype, int64_t i) {
    switch (dtype) {
    case BI8O_F32: return ((const float *)p)[i];
    case BI8O_BF16: return bf16_to_f32(((const uint16_t *)p)[i]);
    default: return f16_to_f32(((const uint16_t *)p)[i]);
    }
}

static inline void store_from_f32(void *p, int dtype, int64_t i, float v) {
    switch (dtype) {
    case BI8O_F32: ((float *)p)[i] = v; break;
    case BI8O_BF16: ((uint16_t *)p)[i] = f32_to_bf16(v); break;
    default: ((uint16_t *)p)[i] = f32_to_f16(v); break;
    }
}

/* the value a store to `dtype` followed by a load would give back */
static inline float round_to_dtype(float v, int dtype) {
    switch (dtype) {
    case BI8O_F32: return v;
    case BI8O_BF16: return bf16_to_f32(f32_to_bf16(v));
    default: return f16_to_f32(f32_to_f16(v));
    }
}

static int bad_dtype(int d) { return d < 0 || d > 2; }

/* One block: triton_functions.py:208-216.
 *   max_val = max(|x|) over the valid elements          (:210-211)
 *   code    = llrint(127. * (x / max_val))              (:212)  two roundings: the
 *             quotient, then the product; llrint rounds half to even. */
static inline void quantize_block(const void *x, int dtype, int64_t base, int64_t stride, int64_t n,
                                  int8_t *q, int64_t qbase, int64_t qstride, float *scale) {
    float m = 0.0f;
    for (int64_t k = 0; k < n; ++k) {
        float a = fabsf(load_as_f32(x, dtype, base + k * stride));
        if (a > m) m = a;                       /* NaN compares false: ignored */
    }
    *scale = m;
    for (int64_t k = 0; k < n; ++k) {
        float v = load_as_f32(x, dtype, base + k * stride);
        int8_t c = 0;
        if (m > 0.0f && v == v) {
            volatile float quot = v / m;        /* volatile: forbid re-association into v*(127/m) */
            volatile float t = 127.0f * quot;
            float r = nearbyintf(t);            /* default rounding mode: ties to even */
            if (r == r) {
                if (r > 127.0f) r = 127.0f;     /* only reachable through inf/inf style inputs */
                if (r < -127.0f) r = -127.0f;
                c = (int8_t)(int)r;
            }
        }
        q[qbase + k * qstride] = c;
    }
}

/* x [M,K] row-major, leading dimension ldx (elements) -> q int8 [M,K] (leading dimension ldq),
 * scales fp32 [ceil(K/B), M] ("block-major, row-minor", triton_functions.py:214-216, :227). */
int bi8o_quantize_rowwise(const void *x, int x_dtype, int8_t *q, float *scales,
                          int64_t M, int64_t K, int64_t ldx, int64_t ldq, int block) {
    if (bad_dtype(x_dtype) || block <= 0 || M < 0 || K < 0) return 1;
    int64_t nblk = (K + block - 1) / block;
#pragma omp parallel for schedule(static)
    for (int64_t m = 0; m < M; ++m) {
        for (int64_t j = 0; j < nblk; ++j) {
            int64_t k0 = j * block;
            int64_t n = (K - k0 < block) ? (K - k0) : block;
            quantize_block(x, x_dtype, m * ldx + k0, 1, n, q, m * ldq + k0, 1, &scales[j * M + m]);
        }
    }
    return 0;
}

/* Same result as quantizing x.t().contiguous() (block_linear.py:93-94, :100-103):
 * x [R,C] row-major -> qT int8 [C,R], scalesT fp32 [ceil(R/B), C]; blocks run down the columns of x. */
int bi8o_quantize_transposed(const void *x, int x_dtype, int8_t *qT, float *scalesT,
                             int64_t R, int64_t C, int64_t ldx, int64_t ldq, int block) {
    if (bad_dtype(x_dtype) || block <= 0 || R < 0 || C < 0) return 1;
    int64_t nblk = (R + block - 1) / block;
#pragma omp parallel for schedule(static)
    for (int64_t c = 0; c < C; ++c) {
        for (int64_t j = 0; j < nblk; ++j) {
            int64_t r0 = j * block;
            int64_t n = (R - r0 < block) ? (R - r0) : block;
            quantize_block(x, x_dtype, r0 * ldx + c, ldx, n, qT, c * ldq + r0, 1, &scalesT[j * C + c]);
        }
    }
    return 0;
}

/* triton_functions.py:487: output = max_val * x * inv_127, left to right, inv_127 = fp32(1./127) (:499),
 * then the store casts to the output dtype. */
int bi8o_dequantize_rowwise(const int8_t *q, const float *scales, void *out, int out_dtype,
                            int64_t M, int64_t K, int64_t ldq, int64_t ldo, int block) {
    if (bad_dtype(out_dtype) || block <= 0 || M < 0 || K < 0) return 1;
    const float inv127 = (float)(1.0 / 127.0);
#pragma omp parallel for schedule(static)
    for (int64_t m = 0; m < M; ++m) {
        for (int64_t k = 0; k < K; ++k) {
            float s = scales[(k / block) * M + m];
            volatile float t = s * (float)q[m * ldq + k];
            float v = t * inv127;
            store_from_f32(out, out_dtype, m * ldo + k, v);
        }
    }
    return 0;
}

/* P[j,m,n] = sum_{k in block j} A[m,k] * W[n,k]  (int32, exact; triton_functions.py:115).
 * A [M,K] (lda), W [N,K] (ldw): both operands K-contiguous, as the reference's b = W_int8.t() view. */
int bi8o_gemm_nt_partials(const int8_t *A, const int8_t *W, int32_t *P,
                          int64_t M, int64_t N, int64_t K, int64_t lda, int64_t ldw, int block) {
    if (block <= 0 || M < 0 || N < 0 || K < 0) return 1;
    int64_t nblk = (K + block - 1) / block;
#pragma omp parallel for schedule(static) collapse(2)
    for (int64_t j = 0; j < nblk; ++j) {
        for (int64_t m = 0; m < M; ++m) {
            int64_t k0 = j * block;
            int64_t k1 = (k0 + block < K) ? (k0 + block) : K;
            for (int64_t n = 0; n < N; ++n) {
                int32_t acc = 0;
                const int8_t *a = A + m * lda;
                const int8_t *w = W + n * ldw;
                for (int64_t k = k0; k < k1; ++k) acc += (int32_t)a[k] * (int32_t)w[k];
                P[(j * M + m) * N + n] = acc;
            }
        }
    }
    return 0;
}

/* triton_functions.py:106-131.
 *   acc  = 0                                                        (:106)
 *   acc += w_factor * (x_factor * (float(P_j) * divfactor))         (:115-120), j ascending
 *   c    = cast(acc)                                                (:127)
 *   c    = c + cast(bias)   evaluated in the output dtype           (:129-131)
 * divfactor = fp32(1. / (127. * 127.))                              (:143)
 * sA [nblk,M], sW [nblk,N] as written by the quantizer.  bias may be NULL. */
int bi8o_gemm_nt_dequant(const int8_t *A, const int8_t *W, const float *sA, const float *sW,
                         const void *bias, int bias_dtype, void *C, int c_dtype,
                         int64_t M, int64_t N, int64_t K, int64_t lda, int64_t ldw, int64_t ldc, int block) {
    if (bad_dtype(c_dtype) || (bias && bad_dtype(bias_dtype)) || block <= 0 || M < 0 || N < 0 || K < 0) return 1;
    int64_t nblk = (K + block - 1) / block;
    const float divfactor = (float)(1.0 / (127.0 * 127.0));
#pragma omp parallel for schedule(static)
    for (int64_t m = 0; m < M; ++m) {
        const int8_t *a = A + m * lda;
        for (int64_t n = 0; n < N; ++n) {
            const int8_t *w = W + n * ldw;
            float acc = 0.0f;
            for (int64_t j = 0; j < nblk; ++j) {
                int64_t k0 = j * block;
                int64_t k1 = (k0 + block < K) ? (k0 + block) : K;
                int32_t p = 0;
                for (int64_t k = k0; k < k1; ++k) p += (int32_t)a[k] * (int32_t)w[k];
                volatile float t0 = (float)p * divfactor;
                volatile float t1 = sA[j * M + m] * t0;
                volatile float t2 = sW[j * N + n] * t1;
                acc = acc + t2;
            }
            float c = round_to_dtype(acc, c_dtype);
            if (bias) {
                float b = round_to_dtype(load_as_f32(bias, bias_dtype, n), c_dtype);
                c = c + b;                      /* rounded to c_dtype by the store below */
            }
            store_from_f32(C, c_dtype, m * ldc + n, c);
        }
    }
    return 0;
}

/* element conversions exported for the tests of this file */
float bi8o_bf16_to_f32(uint16_t h) { return bf16_to_f32(h); }
uint16_t bi8o_f32_to_bf16(float f) { return f32_to_bf16(f); }
float bi8o_f16_to_f32(uint16_t h) { return f16_to_f32(h); }
uint16_t bi8o_f32_to_f16(float f) { return f32_to_f16(f); }
