/*
 * CPU proof-by-exhaustion companion for the quantizer's division: the HIP kernel replaces the
 * per-element IEEE division v / s by  y = fl(1/s)  (one IEEE division per block) followed by a
 * rounded product and FMA corrections.  This program restates that sequence with fmaf() and
 * (one correction for 16-bit inputs, two for binary32) and compares it with the C `/` operator
 *   - for EVERY pair of bf16 values and EVERY pair of f16 values with |v| <= s (all significands
 *     and every exponent difference that can still give a non-zero code), and
 *   - for a large number of random and adversarial binary32 pairs, and
 *   - for DIRECTED hard-to-round binary32 pairs: quotients that lie within 2^-48 (relative) of the midpoint between
 *     two adjacent binary32 values, the closest a quotient of two 24-bit significands can come to one.
 * Prints the number of mismatching quotients; exit status 0 only if there are none.
 *
 * Build: gcc -O2 -ffp-contract=off -fopenmp recip_division_check.c -lm
 */
#include <math.h>
#include <stdint.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>
#ifdef _OPENMP
#include <omp.h>
#endif

static inline float u2f(uint32_t u) { float f; memcpy(&f, &u, 4); return f; }

/* ncorr = 1 is what the kernel uses for 16-bit inputs (proved here by exhaustion),
 * ncorr = 2 for binary32 inputs (Markstein's theorem; sampled here). */
static inline float div_by_recip(float v, float s, float y, int ncorr) {
    float q = v * y;
    for (int i = 0; i < ncorr; ++i) {
        float r = fmaf(-q, s, v);
        q = fmaf(r, y, q);
    }
    return q;
}

static inline int code_of(float q) { return (int)nearbyintf(127.0f * q); }

static long check_pair(float v, float s, int ncorr) {
    volatile float y = 1.0f / s;
    volatile float want = v / s;
    float got = div_by_recip(v, s, y, ncorr);
    if (got != want) return 1;
    if (code_of(got) != code_of(want)) return 1;
    got = div_by_recip(-v, s, y, ncorr);
    return got != -want;
}

static uint64_t rng_state = 0x9E3779B97F4A7C15ull;
static inline uint64_t rng(uint64_t *st) {
    uint64_t z = (*st += 0x9E3779B97F4A7C15ull);
    z = (z ^ (z >> 30)) * 0xBF58476D1CE4E5B9ull;
    z = (z ^ (z >> 27)) * 0x94D049BB133111EBull;
    return z ^ (z >> 31);
}

int main(int argc, char **argv) {
    long n_random = argc > 1 ? atol(argv[1]) : 200000000L;
    long bad = 0, total = 0;

    /* bf16: 7 explicit significand bits; f16: 10.  Scale exponent fixed at a few representative
     * values (the algorithm is invariant under powers of two while everything stays normal); the
     * element exponent runs from equal down to 12 binades below (127 * 2^-12 rounds to 0). */
    const int mant_bits[2] = {7, 10};
    const int s_exps[3] = {127 - 59, 127, 127 + 99};
    for (int t = 0; t < 2; ++t) {
        int mb = mant_bits[t];
        long nm = 1L << mb;
        for (int se = 0; se < 3; ++se) {
#pragma omp parallel for reduction(+ : bad, total) schedule(dynamic, 16)
            for (long ms = 0; ms < nm; ++ms) {
                float s = u2f(((uint32_t)s_exps[se] << 23) | ((uint32_t)ms << (23 - mb)));
                for (int de = 0; de <= 12; ++de) {
                    for (long mv = 0; mv < nm; ++mv) {
                        float v = u2f(((uint32_t)(s_exps[se] - de) << 23) | ((uint32_t)mv << (23 - mb)));
                        if (v > s) continue;
                        bad += check_pair(v, s, 1);
                        total++;
                    }
                }
            }
        }
    }
    printf("exhaustive 16-bit pairs: %ld checked, %ld mismatches\n", total, bad);

    /* binary32: random significands, |v| <= s, scale exponent anywhere in the reciprocal path's range */
    long bad32 = 0;
#pragma omp parallel reduction(+ : bad32)
    {
        uint64_t st = rng_state;
#ifdef _OPENMP
        st += 0x1234567ull * (uint64_t)(omp_get_thread_num() + 1);
#endif
#pragma omp for schedule(static)
        for (long i = 0; i < n_random; ++i) {
            uint64_t a = rng(&st), b = rng(&st);
            uint32_t se = 127 - 60 + (uint32_t)(a % 160);          /* 2^-60 .. 2^99 */
            uint32_t ms = (uint32_t)(a >> 20) & 0x7FFFFF;
            uint32_t mv = (uint32_t)(b >> 20) & 0x7FFFFF;
            uint32_t de = (uint32_t)(b % 10);
            int kind = (int)((a >> 60) & 7);
            if (kind == 0) ms = 0x7FFFFF;                          /* significand all ones */
            if (kind == 1) ms = 0;                                  /* power of two */
            if (kind == 2) mv = 0x7FFFFF;
            if (kind == 3) ms = (uint32_t)(b >> 44) & 0xFF;         /* few significant bits */
            float s = u2f((se << 23) | ms);
            float v = u2f(((se - de) << 23) | mv);
            if (v > s) v = s;
            bad32 += check_pair(v, s, 2);
        }
    }
    /* quotients next to the rounding ties of the code: v close to s * (n + 0.5) / 127 */
    long badt = 0, ntie = 0;
    {
        uint64_t st = 42;
        for (long i = 0; i < 2000000; ++i) {
            uint64_t a = rng(&st);
            uint32_t ms = (uint32_t)(a >> 20) & 0x7FFFFF;
            float s = u2f((127u << 23) | ms);
            int n = (int)(a % 127);
            float v0 = (float)((double)s * ((double)n + 0.5) / 127.0);
            for (int d = -2; d <= 2; ++d) {
                float v = v0;
                for (int k = 0; k < abs(d); ++k) v = nextafterf(v, d < 0 ? 0.0f : 4.0f);
                if (v > s) continue;
                badt += check_pair(v, s, 2);
                ntie++;
            }
        }
    }
    /* Directed hard cases.  For significands S (of s) and V (of v), V / S rounds hardest when V * 2^25 = S * X - r with
     * X odd (X / 2^25 is then the midpoint between two adjacent 24-bit quotients) and |r| as small as it can be: r odd,
     * |r| = 1, 3, 5, 7.  For odd S, X = r * S^-1 mod 2^25 solves that; it is usable when it has 25 bits and V has 24. */
    long badh = 0, nhard = 0;
#pragma omp parallel reduction(+ : badh, nhard)
    {
        uint64_t st = 0xC0FFEEull;
#ifdef _OPENMP
        st += 0x7654321ull * (uint64_t)(omp_get_thread_num() + 1);
#endif
#pragma omp for schedule(static)
        for (long i = 0; i < 6000000; ++i) {
            uint32_t S = (uint32_t)(0x800000u | (rng(&st) & 0x7FFFFFu)) | 1u;      /* odd, 24 bits */
            if (i < 64) S = 0xFFFFFFu - 2u * (uint32_t)i;                          /* significands close to all ones */
            else if (i < 128) S = 0x800001u + 2u * (uint32_t)(i - 64);            /* and just above a power of two */
            uint32_t inv = S;                                                      /* S * inv = 1 mod 2^32 (Newton) */
            for (int k = 0; k < 5; ++k) inv *= 2u - S * inv;
            for (int r = -7; r <= 7; r += 2) {
                uint32_t X = ((uint32_t)r * inv) & 0x1FFFFFFu;
                if (X < 0x1000000u) continue;                                      /* needs 25 bits: quotient in [1/2, 1) */
                int64_t T = (int64_t)S * (int64_t)X - r;                           /* = V * 2^25 */
                if (T & 0x1FFFFFF) { badh++; continue; }                           /* cannot happen */
                int64_t V = T >> 25;
                if (V < 0x800000 || V > 0xFFFFFF) continue;
                for (int de = 0; de <= 8; de += 4) {                               /* the same significands, smaller quotients */
                    float s = ldexpf((float)S, -23 + (int)(i % 50) - 20);
                    float v = ldexpf((float)V, -24 + (int)(i % 50) - 20 - de);
                    if (v > s) continue;
                    badh += check_pair(v, s, 2);
                    nhard++;
                }
            }
        }
    }
    printf("random binary32 pairs: %ld checked, %ld mismatches\n", n_random, bad32);
    printf("directed hard-to-round binary32 pairs: %ld checked, %ld mismatches\n", nhard, badh);
    printf("near-tie binary32 pairs: %ld checked, %ld mismatches\n", ntie, badt);
    return (bad || bad32 || badt || badh || nhard < 1000000) ? 1 : 0;
}
