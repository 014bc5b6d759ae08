/*
 * Natural logarithm and exponential built only from IEEE-754 basic operations (no fused multiply-add when compiled
 * with -ffp-contract=off, no library call), so that every compiler and both host and device evaluate bit-identical
 * results.  Plain C99 / C++ / HIP.  They follow the classic table-free argument reductions:
 *   log: x = 2^k (1 + f), s = f / (2 + f), log(1 + f) = f - hfsq + s (hfsq + R(s^2));
 *   exp: x = k ln2 + r, |r| <= ln2 / 2, exp(r) = 1 + r + r c / (2 - c) with c = r - r^2 P(r^2).
 * The double precision logarithm stays below 1 ulp.
 */
#ifndef MCTSNC_DET_MATH_H
#define MCTSNC_DET_MATH_H
#include <stdint.h>

#if defined(__HIPCC__)
#define DETM_FN __host__ __device__ inline
#else
#define DETM_FN static inline
#endif

/* Valid for positive normal x. */
DETM_FN double detm_log(double x) {
    const double ln2_hi = 6.93147180369123816490e-01, ln2_lo = 1.90821492927058770002e-10;
    const double Lg1 = 6.666666666666735130e-01, Lg2 = 3.999999999940941908e-01, Lg3 = 2.857142874366239149e-01,
                 Lg4 = 2.222219843214978396e-01, Lg5 = 1.818357216161805012e-01, Lg6 = 1.531383769920937332e-01,
                 Lg7 = 1.479819860511658591e-01;
    union { double d; uint64_t u; } v;
    v.d = x;
    int32_t hx = (int32_t)(v.u >> 32);
    const uint32_t lx = (uint32_t)v.u;
    int32_t k = (hx >> 20) - 1023;
    hx &= 0x000fffff;
    int32_t i = (hx + 0x95f64) & 0x100000;
    v.u = ((uint64_t)(uint32_t)(hx | (i ^ 0x3ff00000)) << 32) | lx; /* normalise x or x/2 */
    k += (i >> 20);
    const double f = v.d - 1.0;
    const double dk = (double)k;
    if ((0x000fffff & (2 + hx)) < 3) { /* |f| < 2^-20 */
        if (f == 0.0) {
            if (k == 0) return 0.0;
            return dk * ln2_hi + dk * ln2_lo;
        }
        const double R = f * f * (0.5 - 0.33333333333333333 * f);
        if (k == 0) return f - R;
        return dk * ln2_hi - ((R - dk * ln2_lo) - f);
    }
    const double s = f / (2.0 + f);
    const double z = s * s;
    i = hx - 0x6147a;
    const double w = z * z;
    const int32_t j = 0x6b851 - hx;
    const double t1 = w * (Lg2 + w * (Lg4 + w * Lg6));
    const double t2 = z * (Lg1 + w * (Lg3 + w * (Lg5 + w * Lg7)));
    i |= j;
    const double R = t2 + t1;
    if (i > 0) {
        const double hfsq = 0.5 * f * f;
        if (k == 0) return f - (hfsq - s * (hfsq + R));
        return dk * ln2_hi - ((hfsq - (s * (hfsq + R) + dk * ln2_lo)) - f);
    }
    if (k == 0) return f - s * (f - R);
    return dk * ln2_hi - ((s * (f - R) - dk * ln2_lo) - f);
}

/* Single precision, branch-free: natural logarithm of a positive normal x and exponential of x <= 0 (0 below -86,
 * where the result would near the end of the normal range).  Same reductions as above with shorter polynomials; errors stay
 * below 2 ulp.  Every lane of a wavefront runs the same instructions whatever its argument. */
DETM_FN float detm_logf(float x) {
    const float ln2_hi = 6.9313812256e-01f, ln2_lo = 9.0580006145e-06f;
    const float Lg1 = 0.66666662693f, Lg2 = 0.40000972152f, Lg3 = 0.28498786688f, Lg4 = 0.24279078841f;
    union { float f; uint32_t u; } v;
    v.f = x;
    uint32_t ix = v.u + (0x3f800000u - 0x3f3504f3u);
    const int32_t k = (int32_t)(ix >> 23) - 0x7f;
    v.u = (ix & 0x007fffffu) + 0x3f3504f3u; /* x / 2^k in [sqrt(1/2), sqrt(2)) */
    const float f = v.f - 1.0f;
    const float s = f / (2.0f + f);
    const float z = s * s;
    const float w = z * z;
    const float t1 = w * (Lg2 + w * Lg4);
    const float t2 = z * (Lg1 + w * Lg3);
    const float R = t2 + t1;
    const float hfsq = 0.5f * f * f;
    const float dk = (float)k;
    return s * (hfsq + R) + dk * ln2_lo - hfsq + f + dk * ln2_hi;
}

DETM_FN float detm_expf(float x) {
    const float ln2_hi = 6.9314575195e-01f, ln2_lo = 1.4286067653e-06f, inv_ln2 = 1.4426950216e+00f;
    const float P1 = 1.6666625440e-1f, P2 = -2.7667332906e-3f;
    const float xc = x < -86.0f ? -86.0f : x;
    const int32_t k = (int32_t)(inv_ln2 * xc - 0.5f);
    const float t = (float)k;
    const float hi = xc - t * ln2_hi;
    const float lo = t * ln2_lo;
    const float r = hi - lo;
    const float rr = r * r;
    const float c = r - rr * (P1 + rr * P2);
    const float y = 1.0f + (r * c / (2.0f - c) - lo + hi);
    union { float f; uint32_t u; } v;
    v.f = y;
    v.u += (uint32_t)k << 23; /* k in [-125, 0]: the result stays normal */
    return x < -86.0f ? 0.0f : v.f;
}

#endif
