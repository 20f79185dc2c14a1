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

// ---- f64 arcsine and arccosine -------------------------------------------------------------------------------------------------------
// The classical scheme (Sun's fdlibm e_asin.c / e_acos.c, used unchanged by musl): with R(t) = t P(t) / Q(t), a rational fit of
// (asin(sqrt(t)) - sqrt(t)) / sqrt(t) on [0, 0.25],
//   |x| <  0.5:  asin(x) = x + x R(x^2);                  acos(x) = pi/2 - (x - (pio2_lo - x R(x^2)))
//   |x| >= 0.5:  t = (1 - |x|) / 2, s = sqrt(t), v = s + s R(t):
//                asin(x) = sign(x) (pi/2 - 2 v);           acos(x) = 2 v  (x > 0),  pi - 2 v  (x < 0)
// written as straight-line code: both ranges share one evaluation of R (its argument is selected), the square root is formed from the
// hardware's reciprocal-square-root estimate, and the quotient P / Q (Q lies in [0.5, 1]) from the reciprocal estimate.  The library
// routines take about 100 instructions per element and leave a 1 GiB pass ALU-bound at 0.6 of the memory rate; these take about half.
// Without the library's extra-precision tail for 0.5 <= |x| < 0.975 the results stay within 2 ulp (tests/test_math64_host.py measures
// the error against 80-bit arithmetic).  |x| > 1 and NaN give NaN, asin(+-1) = +-pi/2, acos(1) = 0, acos(-1) = pi, asin(-0.0) = -0.0.

// sqrt(a) for a in [2^-60, 4] (or a = 0, NaN, negative: 0, NaN, NaN): the reciprocal-square-root estimate, one coupled refinement of
// root and half-reciprocal, one correction of the root by its residual.  *tail receives what the rounded root still lacks (the
// residual a - g^2, which a fused multiply-add forms exactly, times 1 / (2 g)): root + tail is good to about 2^-100.
RT_M64 double rt_sqrt_unit_f64(double a, double* tail) {
#if defined(__HIP_DEVICE_COMPILE__)
    const double y = __builtin_amdgcn_rsq(a);
#else
    double y = 1.0 / __builtin_sqrt(a);
    uint64_t yb;
    memcpy(&yb, &y, 8);
    yb &= ~((1ull << 32) - 1);                                  // keep 20 bits of the fraction: cruder than the hardware's estimate
    memcpy(&y, &yb, 8);
#endif
    double g = a * y, h = 0.5 * y;
    const double r = __builtin_fma(-h, g, 0.5);
    g = __builtin_fma(g, r, g);
    h = __builtin_fma(h, r, h);
    g = __builtin_fma(__builtin_fma(-g, g, a), h, g);
    const bool zero = a == 0.0;                                 // the estimate of 0 is inf
    *tail = zero ? 0.0 : __builtin_fma(-g, g, a) * h;
    return zero ? 0.0 : g;
}

// sqrt(a) for a >= 1 (+inf and NaN stay what they are): the same refinement without the zero case.
RT_M64 double rt_sqrt_ge1_f64(double a) {
#if defined(__HIP_DEVICE_COMPILE__)
    const double y = __builtin_amdgcn_rsq(a);
#else
    double y = 1.0 / __builtin_sqrt(a);
    uint64_t yb;
    memcpy(&yb, &y, 8);
    yb &= ~((1ull << 32) - 1);
    memcpy(&y, &yb, 8);
#endif
    double g = a * y, h = 0.5 * y;
    const double r = __builtin_fma(-h, g, 0.5);
    g = __builtin_fma(g, r, g);
    h = __builtin_fma(h, r, h);
    g = __builtin_fma(__builtin_fma(-g, g, a), h, g);
    return a == __builtin_inf() ? a : g;                        // the estimate of inf is 0
}

RT_M64 double rt_asin_R(double t) {
    const double pS0 = 1.66666666666666657415e-01, pS1 = -3.25565818622400915405e-01, pS2 = 2.01212532134862925881e-01,
                 pS3 = -4.00555345006794114027e-02, pS4 = 7.91534994289814532176e-04, pS5 = 3.47933107596021167570e-05,
                 qS1 = -2.40339491173441421878e+00, qS2 = 2.02094576023350569471e+00, qS3 = -6.88283971605453293030e-01,
                 qS4 = 7.70381505559019352791e-02;
    const double p = t * __builtin_fma(t, __builtin_fma(t, __builtin_fma(t, __builtin_fma(t, __builtin_fma(t, pS5, pS4), pS3), pS2), pS1), pS0);
    const double q = __builtin_fma(t, __builtin_fma(t, __builtin_fma(t, __builtin_fma(t, qS4, qS3), qS2), qS1), 1.0);
    return rt_quot_f64(p, q);
}

#define RT_PIO2_HI 1.57079632679489655800e+00
#define RT_PIO2_LO 6.12323399573676603587e-17

RT_M64 double rt_asin_f64(double x) {
    const double ax = __builtin_fabs(x);
    const bool big = ax >= 0.5;                                 // false for NaN: x * x below carries it through
    const double t = big ? (1.0 - ax) * 0.5 : x * x;
    const double R = rt_asin_R(t);
    double c;
    const double s = rt_sqrt_unit_f64(t, &c);                   // NaN beyond the domain (t < 0)
    // pi/2 - 2 (s + c) (1 + R): the large part pi/2 - 2 s first, then everything small
    const double hi = (RT_PIO2_HI - 2.0 * s) - (2.0 * __builtin_fma(s, R, c) - RT_PIO2_LO);
    const double lo = __builtin_fma(x, R, x);
    return big ? __builtin_copysign(hi, x) : lo;
}

RT_M64 double rt_acos_f64(double x) {
    const double ax = __builtin_fabs(x);
    const bool big = ax >= 0.5;
    const double t = big ? (1.0 - ax) * 0.5 : x * x;
    const double R = rt_asin_R(t);
    double c;
    const double s = rt_sqrt_unit_f64(t, &c);
    const double v = s + __builtin_fma(s, R, c);
    const double pos = 2.0 * v;
    const double neg = 3.14159265358979311600e+00 - 2.0 * (v - RT_PIO2_LO);
    const double mid = RT_PIO2_HI - (x - (RT_PIO2_LO - x * R));
    return big ? (x < 0.0 ? neg : pos) : mid;
}

// ---- f64 tangent ---------------------------------------------------------------------------------------------------------------------
// For |x| < 2^30: n = nearest integer to x * 2/pi, r = x - n * pi/2 with pi/2 as the sum of three doubles -- the first product is
// subtracted exactly by the fused multiply-add (every bit of x - n * P1 lies between 2^-52 and 1), the other two bring the remainder
// to full precision even where x is within 2^-60 of a multiple of pi/2 -- then the classical kernels on |r| <= pi/4 (Sun's fdlibm
// k_sin.c / k_cos.c: odd and even minimax polynomials of degree 13 and 14), and their quotient, sin / cos in even quadrants and
// -cos / sin in odd ones, from the reciprocal estimate.  Straight-line code at 20 instructions per element fewer than the library's
// tangent, which leaves a 1 GiB pass ALU-bound at 0.62 of the memory rate.  (The library's sine and cosine are as short as these
// kernels and more accurate: they stay.)  The tangent is within 3 ulp, measured against 80-bit arithmetic by
// tests/test_math64_host.py; sine and cosine of the kernels themselves within 1.5.  Larger arguments, infinities and NaN are not for
// this code (rt_trig_in_range says so): the caller sends them to the library routine, whose reduction handles the whole range.
RT_M64 bool rt_trig_in_range(double x) { return __builtin_fabs(x) < 0x1p30; }

RT_M64 double rt_pio2_reduce(double x, int* n) {
    const double fn = __builtin_rint(x * 0x1.45f306dc9c883p-1);                 // 2 / pi
    double r = __builtin_fma(-fn, 0x1.921fb54442d18p+0, x);                     // pi/2 = P1 + P2 + P3 + 5.6e-50
    r = __builtin_fma(-fn, 0x1.1a62633145c07p-54, r);
    r = __builtin_fma(-fn, -0x1.f1976b7ed8fbcp-110, r);
    *n = (int)fn;
    return r;
}

// sin(r) and cos(r) for |r| <= pi/4
RT_M64 void rt_sincos_kernel(double r, double* s_out, double* c_out) {
    const double S1 = -1.66666666666666324348e-01, S2 = 8.33333333332248946124e-03, S3 = -1.98412698298579493134e-04,
                 S4 = 2.75573137070700676789e-06, S5 = -2.50507602534068634195e-08, S6 = 1.58969099521155010221e-10;
    const double C1 = 4.16666666666666019037e-02, C2 = -1.38888888888741095749e-03, C3 = 2.48015872894767294178e-05,
                 C4 = -2.75573143513906633035e-07, C5 = 2.08757232129817482790e-09, C6 = -1.13596475577881948265e-11;
    const double z = r * r;
    const double ps = __builtin_fma(z, __builtin_fma(z, __builtin_fma(z, __builtin_fma(z, __builtin_fma(z, S6, S5), S4), S3), S2), S1);
    *s_out = __builtin_fma(z * r, ps, r);
    const double pc = z * __builtin_fma(z, __builtin_fma(z, __builtin_fma(z, __builtin_fma(z, __builtin_fma(z, C6, C5), C4), C3), C2), C1);
    const double hz = 0.5 * z, w = 1.0 - hz;
    *c_out = w + (((1.0 - w) - hz) + z * pc);
}

RT_M64 double rt_tan_f64(double x) {
    int n;
    const double r = rt_pio2_reduce(x, &n);
    double s, c;
    rt_sincos_kernel(r, &s, &c);
    const bool odd = (n & 1) != 0;
    const double q = rt_quot_f64(odd ? -c : s, odd ? s : c);
    return x == 0.0 ? x : q;
}

// exp(x) for x <= 0 (the terms of a logsumexp, whose arguments are distances below the running maximum): k = nearest integer to
// x / ln 2, r = x - k ln 2 by two fused multiply-adds with ln 2 as the sum of two doubles (|r| <= 0.347), then
// exp(r) = 1 + r + r^2 P(r) with P of degree 9, the Chebyshev interpolant of (exp(r) - 1 - r) / r^2 on |r| <= 0.3466 (the polynomial is
// within 0.15 ulp of exp), scaled by 2^k in one instruction that also forms denormals and the final 0.  No overflow branch, no table:
// 19 operations where the library's full-range routine takes 38; within 1.5 ulp (1.0 measured against 80-bit arithmetic by
// tests/test_math64_host.py).  exp(-inf) = 0.  The lower clamp is a maximum, so a NaN argument gives 0, not NaN: the caller looks
// after NaN itself (the logsumexp state notes NaN elements apart).  Positive arguments are not for this routine.
RT_M64 double rt_exp_nonpos_f64(double x) {
    const double xc = __builtin_fmax(x, -750.0);                                // 2^-1082 is already 0
    const double fn = __builtin_rint(xc * 0x1.71547652b82fep+0);                // 1 / ln 2
    double r = __builtin_fma(-fn, 0x1.62e42fefa39efp-1, xc);                    // ln 2 = hi + lo + 5.7e-34
    r = __builtin_fma(-fn, 0x1.abc9e3b39803fp-56, r);
    double p = 0x1.af38a71a18cb9p-26;
    p = __builtin_fma(p, r, 0x1.2891834686c7ep-22);
    p = __builtin_fma(p, r, 0x1.71de0daf7a6ccp-19);
    p = __builtin_fma(p, r, 0x1.a019b90eefe8ep-16);
    p = __builtin_fma(p, r, 0x1.a01a01a7c3d59p-13);
    p = __builtin_fma(p, r, 0x1.6c16c1788b646p-10);
    p = __builtin_fma(p, r, 0x1.11111111109b4p-7);
    p = __builtin_fma(p, r, 0x1.5555555553d64p-5);
    p = __builtin_fma(p, r, 0x1.5555555555556p-3);
    p = __builtin_fma(p, r, 0x1.0000000000001p-1);
    const double e = 1.0 + __builtin_fma(r * r, p, r);
    return __builtin_ldexp(e, (int)fn);
}
