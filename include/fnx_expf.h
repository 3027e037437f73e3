/* exp for floats, fixed operation by operation, so that the device library and a CPU restatement of it get the same bits:
 * the SwiGLU and the shared expert's gate (kernels.cu:67-68: sigm, silu_) and the routing weights (moe.cuh:382-411:
 * exp(l_k - l_0)) feed roundings to int8 and comparisons, where a last-bit difference between two exp routines shows as a
 * different q8_1 code. The reference uses CUDA's __expf / expf there, whose bits are the toolkit's; these are this
 * library's. Every step is a single IEEE operation (fmaf, multiply by a power of two, round to nearest): compile with
 * -ffp-contract=off. Relative error below 1e-7 (about one unit in the last place); exp(x) = 0 below -87.3 (no denormal
 * results), +inf above 88.72, NaN for NaN. */
#ifndef FNX_EXPF_H
#define FNX_EXPF_H

#include <math.h>
#include <stdint.h>
#include <string.h>

#if defined(__HIPCC__)
#define FNX_EXPF_FN __host__ __device__ static inline
#else
#define FNX_EXPF_FN static inline
#endif

FNX_EXPF_FN float fnx_expf(float x) {
    if (x != x) return x;
    if (x > 88.72f) return INFINITY;
    if (x < -87.3f) return 0.0f;
    /* x = n ln 2 + r with |r| <= ln 2 / 2: n = round(x / ln 2), r = x - n ln2_hi - n ln2_lo (ln2_hi has 9 zero bits at its
     * end, so n ln2_hi is exact for |n| < 512) */
    const float n = rintf(x * 1.44269504088896341f);
    float r = fmaf(n, -0.693145751953125f, x);
    r = fmaf(n, -1.42860682030941723e-6f, r);
    /* exp(r) = 1 + r + r^2 (1/2 + r (1/6 + r (1/24 + r (1/120 + r (1/720 + r / 5040))))) */
    float p = 1.9841270113829523e-4f;
    p = fmaf(p, r, 1.3888889225199819e-3f);
    p = fmaf(p, r, 8.3333333954215050e-3f);
    p = fmaf(p, r, 4.1666667908430099e-2f);
    p = fmaf(p, r, 1.6666667163372040e-1f);
    p = fmaf(p, r, 0.5f);
    p = fmaf(p * r, r, r);
    p = p + 1.0f;
    /* times 2^n, n in -126 .. 128, as two exact multiplications by powers of two (2^128 is not a float) */
    const int ni = (int) n, n1 = ni / 2, n2 = ni - n1;
    uint32_t b1 = (uint32_t) (n1 + 127) << 23, b2 = (uint32_t) (n2 + 127) << 23;
    float s1, s2;
    memcpy(&s1, &b1, 4);
    memcpy(&s2, &b2, 4);
    return p * s1 * s2;
}

#endif
