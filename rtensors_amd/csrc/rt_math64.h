// f64 natural logarithm written out by hand.  The library routine keeps ln / ln1p / log_b / asinh / acosh / atanh over f64 ALU-bound
// (0.36 .. 0.56 of the memory rate of a 1 GiB pass); this one is the classical table-free scheme at about 50 operations:
//   x = 2^k * m, sqrt(2)/2 <= m < sqrt(2);  f = m - 1;  s = f / (2 + f);
//   ln(m) = f - f^2/2 + s * (f^2/2 + R(s^2)),  R = Lg1 s^2 + Lg2 s^4 + ... + Lg7 s^14  (a minimax fit of 2 atanh(s) / s - 2, the
//   series ln((1 + s) / (1 - s)) = 2 s + 2 s^3 / 3 + ..., published with Sun's fdlibm `e_log.c` and used unchanged by musl's log.c)
//   ln(x) = k * ln2_hi + (ln(m) + k * ln2_lo), ln2 split so that k * ln2_hi is exact.
// The published error bound of the scheme is below 1 ulp; with the polynomial evaluated in fused multiply-adds and the quotient s
// formed from a refined reciprocal the result stays within 1 ulp of the exact logarithm (asserted on the host against 80-bit arithmetic
// by tests/test_math64_host.py, and on the device by the parity tests).  Specials as IEEE / Rust's f64::ln: ln(+-0) = -inf,
// ln(x < 0) = NaN, ln(+inf) = +inf, NaN -> NaN; the hardware's mantissa / exponent pair takes denormals as they are.
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

// The hardware's reciprocal estimate (good to about 2^-23).  On the host the estimate is the quotient cut to 20 bits, cruder than the
// hardware's, so that the error measured on the host bounds the device's.
RT_M64 double rt_rcp_seed_f64(double d) {
#if defined(__HIP_DEVICE_COMPILE__)
    return __builtin_amdgcn_rcp(d);
#else
    double r = 1.0 / d;
    uint64_t rb;
    memcpy(&rb, &r, 8);
    rb &= ~((1ull << 32) - 1);                                  // keep 20 bits of the fraction
    memcpy(&r, &rb, 8);
    return r;
#endif
}

// 1 / d for a finite d of ordinary magnitude (no overflow, no denormals on the way): the estimate refined by two Newton steps, relative
// error below 2^-52.
RT_M64 double rt_rcp_f64(double d) {
    double r = rt_rcp_seed_f64(d);
    r = __builtin_fma(__builtin_fma(-d, r, 1.0), r, r);
    r = __builtin_fma(__builtin_fma(-d, r, 1.0), r, r);
    return r;
}

// a / d within an ulp, for a and d of ordinary magnitude and finite: one Newton step on the estimate (2^-40 at worst), the product, and
// one correction of the product by its own residual, which squares what is left of the reciprocal's error.  Six operations against the
// general division sequence's twenty.
RT_M64 double rt_quot_f64(double a, double d) {
    double r = rt_rcp_seed_f64(d);
    r = __builtin_fma(__builtin_fma(-d, r, 1.0), r, r);
    const double q = a * r;
    return __builtin_fma(__builtin_fma(-d, q, a), r, q);
}

// The same with the reciprocal of d given (refined, as rt_rcp_f64 returns it): three operations per quotient for a divisor that many
// elements share.
RT_M64 double rt_quot_by_rcp_f64(double a, double d, double r) {
    const double q = a * r;
    return __builtin_fma(__builtin_fma(-d, q, a), r, q);
}

// ln of the arguments the straight-line code below does not cover -- zero, negative, +inf, NaN -- is what the hardware's f32 logarithm
// returns for them: -inf, NaN, +inf, NaN.  rt_log_is_special says whether x is one of them; rt_log_special takes the mantissa of x as
// rt_log_split returns it (+-0, negative, +inf and NaN keep their kind there, and unlike x itself it cannot underflow when narrowed).
RT_M64 bool rt_log_is_special(double x) {
#if defined(__HIP_DEVICE_COMPILE__)
    return __builtin_amdgcn_class(x, 0x27F);                    // everything but positive normal and positive denormal numbers
#else
    return !(x > 0.0) || x == __builtin_inf();
#endif
}
RT_M64 double rt_log_special(double mant) {
#if defined(__HIP_DEVICE_COMPILE__)
    return (double)__builtin_amdgcn_logf((float)mant);
#else
    return (double)__builtin_logf((float)mant);
#endif
}

// Mantissa in [sqrt(2) / 2, sqrt(2)) and its exponent; denormals are taken as they are.
RT_M64 double rt_log_split(double x0, int* k_out) {
#if defined(__HIP_DEVICE_COMPILE__)
    double m = __builtin_amdgcn_frexp_mant(x0);
    int k = __builtin_amdgcn_frexp_exp(x0);
#else
    int k;
    double m = __builtin_frexp(x0, &k);
#endif
    // from [0.5, 1) to [sqrt(2) / 2, sqrt(2))
    const int low = m < 0.70710678118654752440 ? 1 : 0;
    *k_out = k - low;
    return __builtin_ldexp(m, low);
}

// ln(1 + f) + lo + hi for f in [sqrt(2) / 2 - 1, sqrt(2) - 1): the caller passes k * ln2_lo (plus any small correction) as `lo` and
// k * ln2_hi as `hi`.
RT_M64 double rt_log_core(double f, double lo, double hi) {
    const double Lg1 = 6.666666666666735130e-01, Lg2 = 3.999999999940941908e-01, Lg3 = 2.857142874366239149e-01, Lg4 = 2.222219843214978396e-01,
                 Lg5 = 1.818357216161805012e-01, Lg6 = 1.531383769920937332e-01, Lg7 = 1.479819860511658591e-01;
    const double hfsq = 0.5 * f * f;
    // s = f / (2 + f): the divisor lies in [1.7, 2.5]
    const double s = rt_quot_f64(f, 2.0 + f);
    const double z = s * s;
    const double w = z * z;
    const double t1 = w * __builtin_fma(w, __builtin_fma(w, Lg6, Lg4), Lg2);
    const double t2 = z * __builtin_fma(w, __builtin_fma(w, __builtin_fma(w, Lg7, Lg5), Lg3), Lg1);
    const double R = t2 + t1;
    return s * (hfsq + R) + lo - hfsq + f + hi;
}

#define RT_LN2_HI 6.93147180369123816490e-01
#define RT_LN2_LO 1.90821492927058770002e-10

RT_M64 double rt_log_f64(double x0) {
    // Straight-line code: the rare inputs (zero, negative, infinite, NaN) are patched by one select at the end, so that a wave never
    // splits over them.
    int k;
    const double m = rt_log_split(x0, &k);
    const double dk = (double)k;
    const double res = rt_log_core(m - 1.0, dk * RT_LN2_LO, dk * RT_LN2_HI);
    return rt_log_is_special(x0) ? rt_log_special(m) : res;
}

// ln(1 + x).  u = fl(1 + x) and the rounding error e of that sum (exactly, by the two-sum) stand for 1 + x.  When u lies in
// [sqrt(2) / 2, sqrt(2)) the argument of the core is x itself, which is exact; elsewhere it is the mantissa of u, and e / u -- at most
// 2^-53 against a result of at least 0.29, so the raw reciprocal estimate is enough -- is added to the small term.  The result has the
// sign of x for every x > -1, which also gives ln1p(-0.0) = -0.0.
RT_M64 double rt_log1p_f64(double x) {
    const double u = 1.0 + x;
    const double bb = u - 1.0;
    const double e = (1.0 - (u - bb)) + (x - bb);
    int k;
    const double m = rt_log_split(u, &k);
    const bool near = k == 0;
    const double f = near ? x : m - 1.0;
    const double c = near ? 0.0 : e * rt_rcp_seed_f64(u);
    const double dk = (double)k;
    const double res = __builtin_copysign(rt_log_core(f, dk * RT_LN2_LO + c, dk * RT_LN2_HI), x);
    return rt_log_is_special(u) ? rt_log_special(m) : res;
}
