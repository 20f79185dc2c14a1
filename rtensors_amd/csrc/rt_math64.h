// f64 natural logarithm written out by hand.  The library routine keeps ln / ln1p / log_b / asinh / acosh / atanh over f64 ALU-bound
// (0.36 .. 0.56 of the memory rate of a 1 GiB pass); this one is the classical table-free scheme at about 40 operations:
//   x = 2^k * m, sqrt(2)/2 <= m < sqrt(2);  f = m - 1;  s = f / (2 + f);
//   ln(m) = f - f^2/2 + s * (f^2/2 + R(s^2)),  R = Lg1 s^2 + Lg2 s^4 + ... + Lg7 s^14  (a minimax fit of 2 atanh(s) / s - 2, the
//   series ln((1 + s) / (1 - s)) = 2 s + 2 s^3 / 3 + ..., published with Sun's fdlibm `e_log.c` and used unchanged by musl's log.c)
//   ln(x) = k * ln2_hi + (ln(m) + k * ln2_lo), ln2 split so that k * ln2_hi is exact.
// The published error bound of the scheme is below 1 ulp; with the polynomial evaluated in fused multiply-adds and the quotient s
// formed from a refined reciprocal the result stays within 1 ulp of the exact logarithm (asserted on the host against 80-bit arithmetic by tests/test_math64_host.py, and on the device
// by the parity tests).  Specials as IEEE / Rust's f64::ln: ln(+-0) = -inf, ln(x < 0) = NaN, ln(+inf) = +inf, NaN -> NaN; denormals
// are scaled by 2^54 first.
//
// The file compiles for the device (hipcc) and for the host (g++), like rt_div128.h.
#pragma once

#include <stdint.h>
#include <string.h>

#if defined(__HIPCC__)
#define RT_M64 __host__ __device__ __forceinline__
#else
#define RT_M64 static inline
#endif

// 1 / d for a finite d of ordinary magnitude (no overflow, no denormals on the way): the hardware estimate refined by two Newton steps,
// relative error below 2^-52.  On the host the estimate is the quotient cut to 20 bits, cruder than the hardware's.
RT_M64 double rt_rcp_f64(double d) {
#if defined(__HIP_DEVICE_COMPILE__)
    double r = __builtin_amdgcn_rcp(d);
#else
    double r = 1.0 / d;
    uint64_t rb;
    memcpy(&rb, &r, 8);
    rb &= ~((1ull << 32) - 1);                                  // keep 20 bits of the fraction
    memcpy(&r, &rb, 8);
#endif
    r = __builtin_fma(__builtin_fma(-d, r, 1.0), r, r);
    r = __builtin_fma(__builtin_fma(-d, r, 1.0), r, r);
    return r;
}

RT_M64 double rt_log_f64(double x0) {
    const double ln2_hi = 6.93147180369123816490e-01, ln2_lo = 1.90821492927058770002e-10;
    const double Lg1 = 6.666666666666735130e-01, Lg2 = 3.999999999940941908e-01, Lg3 = 2.857142874366239149e-01, Lg4 = 2.222219843214978396e-01,
                 Lg5 = 1.818357216161805012e-01, Lg6 = 1.531383769920937332e-01, Lg7 = 1.479819860511658591e-01;
    // Straight-line code: the rare inputs (zero, negative, infinite, NaN) are patched by selects at the end, so that a wave never
    // splits over them.  Mantissa in [0.5, 1) and exponent come from the hardware's frexp pair, which takes denormals as they are.
#if defined(__HIP_DEVICE_COMPILE__)
    double x = __builtin_amdgcn_frexp_mant(x0);
    int k = __builtin_amdgcn_frexp_exp(x0);
#else
    int k;
    double x = __builtin_frexp(x0, &k);
#endif
    // to [sqrt(2) / 2, sqrt(2))
    const bool low = x < 0.70710678118654752440;
    x = low ? x + x : x;
    k = low ? k - 1 : k;
    const double f = x - 1.0;
    const double hfsq = 0.5 * f * f;
    // s = f / (2 + f): the divisor lies in [1.7, 2.5], so reciprocal, product and one correction of the product replace the
    // general division sequence (s within an ulp instead of correctly rounded, at less than half the operations)
    const double d = 2.0 + f;
    const double r = rt_rcp_f64(d);
    double s = f * r;
    s = __builtin_fma(__builtin_fma(-d, s, f), r, s);
    const double z = s * s;
    const double w = z * z;
    const double t1 = w * __builtin_fma(w, __builtin_fma(w, Lg6, Lg4), Lg2);
    const double t2 = z * __builtin_fma(w, __builtin_fma(w, __builtin_fma(w, Lg7, Lg5), Lg3), Lg1);
    const double R = t2 + t1;
    const double dk = (double)k;
    double res = s * (hfsq + R) + dk * ln2_lo - hfsq + f + dk * ln2_hi;
    res = x0 == __builtin_inf() ? x0 : res;
    res = !(x0 >= 0.0) ? __builtin_nan("") : res;               // negative, NaN
    res = x0 == 0.0 ? -__builtin_inf() : res;                   // +-0
    return res;
}

// ln(1 + x) from the logarithm (Kahan): with u = fl(1 + x), ln(u) * x / (u - 1) cancels the rounding of u.
RT_M64 double rt_log1p_f64(double x) {
    const double u = 1.0 + x;
    // x / (u - 1) lies within a factor of two of 1.  From 2^60 on, u - 1 equals x exactly; below that the divisor is between 2^-53 and
    // 2^60 in magnitude, where the refined reciprocal and one correction step give the quotient within an ulp at half the operations of
    // the general division sequence.
    const double d = u - 1.0;
    const double r = rt_rcp_f64(d);
    double q = x * r;
    q = __builtin_fma(__builtin_fma(-d, q, x), r, q);
    q = __builtin_fabs(x) >= 0x1p60 ? 1.0 : q;
    double res = rt_log_f64(u) * q;                             // u == 1 gives 0 * NaN: patched below
    res = u == 1.0 ? x : res;                                   // |x| below half an ulp of 1 (keeps -0.0)
    res = u == __builtin_inf() ? u : res;
    return res;
}
