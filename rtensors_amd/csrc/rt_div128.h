// Truncating division of 128-bit integers, written out by hand: the device has no 128-bit divide routine, and the compiler's own
// expansion is a loop of 128 shift-and-subtract steps.  Here the work is at most four 64-bit divisions:
//   both operands below 2^64                one 64-bit division
//   divisor below 2^64                      high half by one 64-bit division, then 128 / 64 -> 64 on (remainder, low half)
//   divisor of 2^64 and more                the quotient fits 64 bits: 128 / 64 -> 64 on the operands scaled so that the divisor's
//                                           leading 64 bits stand alone, an estimate that is exact or one too large, then one
//                                           multiply-and-compare correction (Hacker's Delight, 2nd ed., 9-5, at twice the width)
// The 128 / 64 -> 64 step is Knuth's algorithm D with 32-bit digits (two quotient digits, each estimated from a 64-bit division
// and corrected at most twice; Hacker's Delight 9-4 `divlu`).
//
// The file compiles for the device (hipcc) and for the host (g++), where a test holds it to the compiler's own `/` on __int128.
#pragma once

#include <stdint.h>

#if defined(__HIPCC__)
#define RT_D128 __host__ __device__ __forceinline__
#else
#define RT_D128 static inline
#endif

typedef unsigned __int128 rt_u128;
typedef __int128 rt_i128;

RT_D128 int rt_clz64(uint64_t x) { return __builtin_clzll(x); }             // x != 0

// (u1 * 2^64 + u0) / v for u1 < v (so that the quotient fits 64 bits); v != 0.
RT_D128 uint64_t rt_div_128_by_64(uint64_t u1, uint64_t u0, uint64_t v) {
    const uint64_t B = 1ull << 32;
    const int s = rt_clz64(v);
    v <<= s;                                                                // normalised: top bit set
    const uint64_t vn1 = v >> 32, vn0 = v & 0xffffffffull;
    const uint64_t un32 = s ? ((u1 << s) | (u0 >> (64 - s))) : u1;
    const uint64_t un10 = u0 << s;
    const uint64_t un1 = un10 >> 32, un0 = un10 & 0xffffffffull;
    uint64_t q1 = un32 / vn1, rhat = un32 - q1 * vn1;
    while (q1 >= B || q1 * vn0 > B * rhat + un1) {
        q1 -= 1;
        rhat += vn1;
        if (rhat >= B) break;
    }
    const uint64_t un21 = un32 * B + un1 - q1 * v;                          // modulo 2^64, as the algorithm wants
    uint64_t q0 = un21 / vn1;
    rhat = un21 - q0 * vn1;
    while (q0 >= B || q0 * vn0 > B * rhat + un0) {
        q0 -= 1;
        rhat += vn1;
        if (rhat >= B) break;
    }
    return q1 * B + q0;
}

// a / b, b != 0
RT_D128 rt_u128 rt_udiv128(rt_u128 a, rt_u128 b) {
    const uint64_t ah = (uint64_t)(a >> 64), al = (uint64_t)a, bh = (uint64_t)(b >> 64), bl = (uint64_t)b;
    if (bh == 0) {
        if (ah == 0) return (rt_u128)(al / bl);
        const uint64_t qh = ah / bl, r = ah - qh * bl;
        const uint64_t ql = rt_div_128_by_64(r, al, bl);
        return ((rt_u128)qh << 64) | ql;
    }
    if (ah < bh) return 0;
    const int s = rt_clz64(bh);
    const uint64_t v1 = (uint64_t)((b << s) >> 64);                        // the divisor's leading 64 bits, top bit set
    const rt_u128 u1 = a >> 1;
    const uint64_t q1 = rt_div_128_by_64((uint64_t)(u1 >> 64), (uint64_t)u1, v1);
    uint64_t q0 = (uint64_t)((((rt_u128)q1) << s) >> 63);
    if (q0 != 0) q0 -= 1;                                                   // now exact or one too small
    if (a - (rt_u128)q0 * b >= b) q0 += 1;
    return (rt_u128)q0;
}

// Truncating a / b for b != 0.  MIN / -1 wraps to MIN (the caller reports it).
RT_D128 rt_i128 rt_idiv128(rt_i128 a, rt_i128 b) {
    const bool na = a < 0, nb = b < 0;
    const rt_u128 ua = na ? (rt_u128)0 - (rt_u128)a : (rt_u128)a;
    const rt_u128 ub = nb ? (rt_u128)0 - (rt_u128)b : (rt_u128)b;
    const rt_u128 q = rt_udiv128(ua, ub);
    return (rt_i128)(na != nb ? (rt_u128)0 - q : q);
}
