/*
 * tanh in fp64 for the fused epilogues (y = tanh(x W + b)): about forty
 * full-rate instructions instead of the 150 of the device library's routine,
 * which matters because the epilogue of a memory-bound reconstruction has no
 * VALU time to spare (a 4096 x 4096 layer: 148 -> 90 us).
 *
 *   tanh(x) = sign(x) * em / (em + 2),   em = expm1(2|x|)
 *   2|x| = k ln2 + r, |r| <= ln2 / 2;    expm1(r) = r + r^2 S(r), S the Taylor
 *   series of (e^r - 1 - r) / r^2 to r^12 (truncation below 1e-19);
 *   em = (2^k r + (2^k - 1)) + 2^k r^2 S(r), the scalings exact for k <= 53.
 *
 * For k = 0 the value is expm1(r) itself, so small arguments keep full
 * relative accuracy; measured against a correctly rounded tanh the error stays
 * below 2 ulp over the whole range. |x| below 2^-28 returns x, above 19.1
 * returns +-1 (tanh rounds to 1 from 19.07 on), NaN returns NaN.
 */
#ifndef ESHKOL_HIP_TANH_F64_H
#define ESHKOL_HIP_TANH_F64_H

#include <hip/hip_runtime.h>

__device__ __forceinline__ double eshkol_tanh_f64(double x) {
    const double ax = fabs(x);
    const double y = ax + ax;
    const double k = rint(y * 1.44269504088896338700e+00);
    /* ln2 in two parts, the first with 33 bits: r_hi is exact, r_lo carries the rest */
    const double r_hi = fma(-k, 6.93147180369123816490e-01, y);
    const double r_lo = -k * 1.90821492927058770002e-10;
    const double r = r_hi + r_lo;
    double s = 1.14707455977297247139e-11;            /* 1/14! ... 1/2! */
    s = fma(s, r, 1.60590438368216145994e-10);
    s = fma(s, r, 2.08767569878680989792e-09);
    s = fma(s, r, 2.50521083854417187751e-08);
    s = fma(s, r, 2.75573192239858906526e-07);
    s = fma(s, r, 2.75573192239858906526e-06);
    s = fma(s, r, 2.48015873015873015873e-05);
    s = fma(s, r, 1.98412698412698412698e-04);
    s = fma(s, r, 1.38888888888888888889e-03);
    s = fma(s, r, 8.33333333333333333333e-03);
    s = fma(s, r, 4.16666666666666666667e-02);
    s = fma(s, r, 1.66666666666666666667e-01);
    s = fma(s, r, 5.00000000000000000000e-01);
    /* expm1(2|x|) = 2^k (r + r^2 S) + (2^k - 1): the large terms first, in one
     * rounding, then the small one, so that a negative r does not cost bits */
    const int ki = (int)k;
    const double two_k = ldexp(1.0, ki);
    const double lead = fma(two_k, r_hi, two_k - 1.0);
    const double em = fma(two_k, fma(r * r, s, r_lo), lead);
    /* em / (em + 2) with the rounding error of the sum taken back out (it is worth
     * an ulp of the result when the result sits at the top of its binade) */
    const double den = em + 2.0;
    const double bb = den - em;
    const double den_err = (em - (den - bb)) + (2.0 - bb);
    const double q = em / den;
    double t = fma(-q, den_err * __builtin_amdgcn_rcp(den), q);
    if (ax < 3.725290298461914e-09) t = ax;           /* 2^-28 */
    if (ax > 19.1) t = 1.0;
    return copysign(t, x);
}

#endif
