// f64 natural logarithm written out by hand.  The library routine keeps ln / ln1p / log_b / asinh / acosh / atanh over f64 ALU-bound
// (0.36 .. 0.56 of the memory rate of a 1 GiB pass); this one is the classical table-free scheme at about 40 operations:
//   x = 2^k * m, sqrt(2)/2 <= m < sqrt(2);  f = m - 1;  s = f / (2 + f);
//   ln(m) = f - f^2/2 + s * (f^2/2 + R(s^2)),  R = Lg1 s^2 + Lg2 s^4 + ... + Lg7 s^14  (a minimax fit of 2 atanh(s) / s - 2, the
//   series ln((1 + s) / (1 - s)) = 2 s + 2 s^3 / 3 + ..., published with Sun's fdlibm `e_log.c` and used unchanged by musl's log.c)
//   ln(x) = k * ln2_hi + (ln(m) + k * ln2_lo), ln2 split so that k * ln2_hi is exact.
// The published error bound of the scheme is below 1 ulp; with the polynomial evaluated in fused multiply-adds the result stays
// within 1 ulp of the exact logarithm (asserted on the host against 80-bit arithmetic by tests/test_math64_host.py, and on the device
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

RT_M64 double rt_log_f64(double x) {
    const double ln2_hi = 6.93147180369123816490e-01, ln2_lo = 1.90821492927058770002e-10;
    const double Lg1 = 6.666666666666735130e-01, Lg2 = 3.999999999940941908e-01, Lg3 = 2.857142874366239149e-01, Lg4 = 2.222219843214978396e-01,
                 Lg5 = 1.818357216161805012e-01, Lg6 = 1.531383769920937332e-01, Lg7 = 1.479819860511658591e-01;
    uint64_t bits;
    memcpy(&bits, &x, 8);
    uint32_t hx = (uint32_t)(bits >> 32);
    int k = 0;
    if (hx < 0x00100000u || (hx >> 31)) {                       // below the smallest normal number, zero, or negative
        if ((bits << 1) == 0) return -__builtin_inf();          // +-0
        if (hx >> 31) return __builtin_nan("");                 // negative (including -inf)
        k -= 54;                                                // denormal: scale up
        x *= 18014398509481984.0;                               // 2^54
        memcpy(&bits, &x, 8);
        hx = (uint32_t)(bits >> 32);
    } else if (hx >= 0x7ff00000u) {
        return x;                                               // +inf, NaN
    } else if (hx == 0x3ff00000u && (uint32_t)bits == 0) {
        return 0.0;                                             // ln(1) = +0
    }
    // reduce to [sqrt(2) / 2, sqrt(2))
    hx += 0x3ff00000u - 0x3fe6a09eu;
    k += (int)(hx >> 20) - 0x3ff;
    hx = (hx & 0x000fffffu) + 0x3fe6a09eu;
    bits = ((uint64_t)hx << 32) | (bits & 0xffffffffull);
    memcpy(&x, &bits, 8);
    const double f = x - 1.0;
    const double hfsq = 0.5 * f * f;
    const double s = f / (2.0 + f);
    const double z = s * s;
    const double w = z * z;
    const double t1 = w * __builtin_fma(w, __builtin_fma(w, Lg6, Lg4), Lg2);
    const double t2 = z * __builtin_fma(w, __builtin_fma(w, __builtin_fma(w, Lg7, Lg5), Lg3), Lg1);
    const double R = t2 + t1;
    const double dk = (double)k;
    return s * (hfsq + R) + dk * ln2_lo - hfsq + f + dk * ln2_hi;
}

// ln(1 + x) from the logarithm (Kahan): with u = fl(1 + x), ln(u) * x / (u - 1) cancels the rounding of u.
RT_M64 double rt_log1p_f64(double x) {
    const double u = 1.0 + x;
    if (u == 1.0) return x;                                     // |x| below half an ulp of 1 (keeps -0.0)
    if (u == __builtin_inf()) return u;
    return rt_log_f64(u) * (x / (u - 1.0));
}
