/*
 * Natural logarithm and exponential built only from IEEE-754 double basic operations (no fused multiply-add when
 * compiled with -ffp-contract=off, no library call), so that every compiler and both host and device evaluate
 * bit-identical results.  Plain C99 / C++ / HIP.  Both follow the classic table-free argument reductions:
 *   log: x = 2^k (1 + f), s = f / (2 + f), log(1 + f) = f - hfsq + s (hfsq + R(s^2));
 *   exp: x = k ln2 + r, |r| <= ln2 / 2, exp(r) = 1 + r + r c / (2 - c) with c = r - r^2 P(r^2).
 * Errors stay below 1 ulp.
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

/* Any finite x; overflows to +inf above 709.78, returns 0 below -745.13 (no subnormal results are needed by the
 * callers, which only use arguments <= 0 and a few small positive ones). */
DETM_FN double detm_exp(double x) {
    const double ln2_hi = 6.93147180369123816490e-01, ln2_lo = 1.90821492927058770002e-10,
                 inv_ln2 = 1.44269504088896338700e+00;
    const double P1 = 1.66666666666666019037e-01, P2 = -2.77777777770155933842e-03, P3 = 6.61375632143793436117e-05,
                 P4 = -1.65339022054652515390e-06, P5 = 4.13813679705723846039e-08;
    if (x != x) return x;
    if (x > 7.09782712893383973096e+02) {
        union { uint64_t u; double d; } inf;
        inf.u = 0x7ff0000000000000ull;
        return inf.d;
    }
    if (x < -7.45133219101941108420e+02) return 0.0;
    const double ax = x < 0.0 ? -x : x;
    double hi = x, lo = 0.0;
    int32_t k = 0;
    if (ax > 0.34657359027997264) { /* |x| > ln2 / 2 */
        if (ax < 1.0397207708399179) {
            k = x < 0.0 ? -1 : 1;
        } else {
            k = (int32_t)(inv_ln2 * x + (x < 0.0 ? -0.5 : 0.5));
        }
        const double t = (double)k;
        hi = x - t * ln2_hi;
        lo = t * ln2_lo;
        x = hi - lo;
    } else if (ax < 3.725290298461914e-09) { /* 2^-28 */
        return 1.0 + x;
    }
    const double t = x * x;
    const double c = x - t * (P1 + t * (P2 + t * (P3 + t * (P4 + t * P5))));
    if (k == 0) return 1.0 - ((x * c) / (c - 2.0) - x);
    double y = 1.0 - ((lo - (x * c) / (2.0 - c)) - hi);
    union { double d; uint64_t u; } v;
    v.d = y;
    if (k >= -1021) {
        v.u += (uint64_t)(int64_t)k << 52;
        return v.d;
    }
    v.u += (uint64_t)(int64_t)(k + 1000) << 52;
    return v.d * 9.33263618503218878990e-302; /* 2^-1000 */
}

#endif
