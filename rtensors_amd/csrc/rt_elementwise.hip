// In-place elementwise family: fill, the 31 unary ops and the 8 scalar ops over the three layouts of the
// reference's Backend trait (contiguous run, 1-D strided, N-d view).
// Element definitions follow the reference's Cpu backend (backend/cpu.rs:485-724), which is the parity target:
// e.g. relu is `x > 0 ? x : 0` (NaN -> 0, -0.0 -> +0.0) and sign(0) = 0.
//
// Memory behaviour: the contiguous kernel moves one 16-byte vector per lane (global_load/store_dwordx4), a whole
// wavefront touching 1 KiB of consecutive addresses, in many small blocks.  Algorithmic traffic is 2*N*sizeof(T) for
// read-modify-write ops and N*sizeof(T) for fill.
#include "rt_common.h"
#include "rt_div128.h"
#include "rt_math64.h"

#include <type_traits>

namespace {

// ---- element types ---------------------------------------------------------------------------------------------
struct boolean_t { uint8_t v; };      // core/value.rs:650-765: + is OR, - is XOR, * is AND

template <class T> struct is_flt : std::integral_constant<bool, std::is_same<T, float>::value || std::is_same<T, double>::value> {};
template <class T> struct is_bool : std::is_same<T, boolean_t> {};
typedef unsigned __int128 u128_t;      // core/value.rs: u128 / i128 (division by hand, rt_div128.h)
typedef __int128 i128_t;
template <class T> struct is_sint : std::integral_constant<bool, (std::is_integral<T>::value && std::is_signed<T>::value) || std::is_same<T, i128_t>::value> {};
template <class T> struct is_uint : std::integral_constant<bool, (std::is_integral<T>::value && std::is_unsigned<T>::value) || std::is_same<T, u128_t>::value> {};
template <class T> struct is_int : std::integral_constant<bool, is_sint<T>::value || is_uint<T>::value> {};

template <class T, class E = void> struct carrier { typedef T type; };
template <class T> struct carrier<T, typename std::enable_if<is_int<T>::value && sizeof(T) <= 4>::type> { typedef uint32_t type; };
template <class T> struct carrier<T, typename std::enable_if<is_int<T>::value && sizeof(T) == 8>::type> { typedef uint64_t type; };
template <class T> struct carrier<T, typename std::enable_if<is_int<T>::value && sizeof(T) == 16>::type> { typedef u128_t type; };

// wrapping integer arithmetic (Rust release semantics) through an unsigned carrier; IEEE for floats
template <class T> __device__ __forceinline__ T w_add(T a, T b) {
    if constexpr (is_flt<T>::value) return a + b;
    else if constexpr (is_bool<T>::value) return boolean_t{(uint8_t)(a.v | b.v)};
    else { typedef typename carrier<T>::type W; return (T)(W)((W)a + (W)b); }
}
template <class T> __device__ __forceinline__ T w_sub(T a, T b) {
    if constexpr (is_flt<T>::value) return a - b;
    else if constexpr (is_bool<T>::value) return boolean_t{(uint8_t)(a.v ^ b.v)};
    else { typedef typename carrier<T>::type W; return (T)(W)((W)a - (W)b); }
}
template <class T> __device__ __forceinline__ T w_mul(T a, T b) {
    if constexpr (is_flt<T>::value) return a * b;
    else if constexpr (is_bool<T>::value) return boolean_t{(uint8_t)(a.v & b.v)};
    else { typedef typename carrier<T>::type W; return (T)(W)((W)a * (W)b); }
}
// Integer division truncates toward zero.  A zero divisor (and MIN / -1) panics in the reference; the host refuses
// a zero scalar up front, and the device result for the remaining undefined cases is 0 / MIN respectively.
template <class T> __device__ __forceinline__ T w_div(T a, T b) {
    if constexpr (is_flt<T>::value) return a / b;
    else if constexpr (is_bool<T>::value) return boolean_t{0};
    else if constexpr (sizeof(T) == 16) {
        if (b == 0) return 0;
        if constexpr (is_sint<T>::value) return rt_idiv128(a, b);         // MIN / -1 wraps to MIN
        else return rt_udiv128(a, b);
    } else if constexpr (is_sint<T>::value) {
        if (b == 0) return 0;
        if (b == (T)-1) return w_sub<T>((T)0, a);
        if constexpr (sizeof(T) <= 2) return rt_div_narrow<T>(a, b);
        else if constexpr (sizeof(T) == 8) return rt_div64<T>(a, b);
        else return (T)(a / b);
    } else {
        if (b == 0) return 0;
        if constexpr (sizeof(T) <= 2) return rt_div_narrow<T>(a, b);
        else if constexpr (sizeof(T) == 8) return rt_div64<T>(a, b);
        else return (T)(a / b);
    }
}
template <class T> __device__ __forceinline__ bool gt0(T x) {
    if constexpr (is_bool<T>::value) return x.v != 0;
    else return x > (T)0;
}
template <class T> __device__ __forceinline__ T zero_of() {
    if constexpr (is_bool<T>::value) return boolean_t{0};
    else return (T)0;
}
template <class T> __device__ __forceinline__ T min_of() {                // signed integers
    typedef typename carrier<T>::type W;
    return (T)((W)1 << (sizeof(T) * 8 - 1));
}
template <class T> __device__ __forceinline__ T one_of() {
    if constexpr (is_bool<T>::value) return boolean_t{1};
    else return (T)1;
}

// libm spellings per precision
__device__ __forceinline__ float m_exp(float x) { return expf(x); }
__device__ __forceinline__ double m_exp(double x) { return exp(x); }
__device__ __forceinline__ float m_expm1(float x) { return expm1f(x); }
__device__ __forceinline__ double m_expm1(double x) { return expm1(x); }
__device__ __forceinline__ float m_log(float x) { return logf(x); }
__device__ __forceinline__ double m_log(double x) { return rt_log_f64(x); }      // by hand: the library routine is ALU-bound (rt_math64.h)
// ln(1 + x) in f32 from the plain logarithm (Kahan): with u = fl(1 + x), ln(u) * x / (u - 1) cancels the rounding of u, a few ulp over
// the whole range and about twice as fast as the library routine, which left the 1 GiB pass ALU-bound at 0.47 of the memory rate.
__device__ __forceinline__ float m_log1p(float x) {
    const float u = 1.0f + x;
    if (u == 1.0f) return x;                                   // |x| below half an ulp of 1 (keeps -0.0)
    if (u == __builtin_inff()) return u;
    return logf(u) * (x / (u - 1.0f));
}
__device__ __forceinline__ double m_log1p(double x) { return rt_log1p_f64(x); }
__device__ __forceinline__ float m_sqrt(float x) { return sqrtf(x); }
__device__ __forceinline__ double m_sqrt(double x) { return sqrt(x); }
__device__ __forceinline__ float m_sin(float x) { return sinf(x); }
__device__ __forceinline__ double m_sin(double x) { return sin(x); }
__device__ __forceinline__ float m_cos(float x) { return cosf(x); }
__device__ __forceinline__ double m_cos(double x) { return cos(x); }
__device__ __forceinline__ float m_tan(float x) { return tanf(x); }
// f64 tangent: by hand below 2^30 (rt_math64.h), the library routine with its full-range reduction beyond, for infinities and NaN
__device__ __forceinline__ double m_tan(double x) { return rt_trig_in_range(x) ? rt_tan_f64(x) : tan(x); }
__device__ __forceinline__ float m_asin(float x) { return asinf(x); }
__device__ __forceinline__ double m_asin(double x) { return rt_asin_f64(x); }      // by hand, as the logarithm (rt_math64.h)
__device__ __forceinline__ float m_acos(float x) { return acosf(x); }
__device__ __forceinline__ double m_acos(double x) { return rt_acos_f64(x); }
__device__ __forceinline__ float m_atan(float x) { return atanf(x); }
__device__ __forceinline__ double m_atan(double x) { return atan(x); }
__device__ __forceinline__ float m_floor(float x) { return floorf(x); }
__device__ __forceinline__ double m_floor(double x) { return floor(x); }
__device__ __forceinline__ float m_ceil(float x) { return ceilf(x); }
__device__ __forceinline__ double m_ceil(double x) { return ceil(x); }
__device__ __forceinline__ float m_round(float x) { return roundf(x); }     // half away from zero, like Rust's round()
__device__ __forceinline__ double m_round(double x) { return round(x); }
__device__ __forceinline__ float m_trunc(float x) { return truncf(x); }
__device__ __forceinline__ double m_trunc(double x) { return trunc(x); }
__device__ __forceinline__ float m_abs(float x) { return fabsf(x); }
__device__ __forceinline__ double m_abs(double x) { return fabs(x); }

// a / ln(base).  ln(base) is one value for the whole launch.  f32: the plain division.  f64: the host computes ln(base) and its
// reciprocal once (LogBase64) and every element takes three operations (the correctly rounded quotient in all but rare cases, within one
// ulp always) instead of the general division sequence's twenty and a logarithm of the base per lane; a base whose logarithm is zero,
// infinite, NaN or beyond 2^+-500 keeps the general division, which alone gets those right.
__device__ __forceinline__ float over_log_base(float a, float base) { return a / m_log(base); }
struct LogBase64 {
    double d = 0.0, r = 0.0;                                    // ln(base); its reciprocal, or 0 for "divide"
    static LogBase64 of(double base) {
        LogBase64 b;
        b.d = rt_log_f64(base);
        const double ad = __builtin_fabs(b.d);
        b.r = (ad > 0x1p-500 && ad < 0x1p500) ? rt_rcp_f64(b.d) : 0.0;
        return b;
    }
};
__device__ __forceinline__ double over_log_base(double a, const LogBase64& b) {
    if (b.r == 0.0) return a / b.d;                             // wave-uniform
    // a = +-inf: the product is the answer, and its residual inf - inf is NaN; the minimum of a NaN and a number is the number, the
    // correction term stays finite and leaves the infinite product as it is
    const double q = a * b.r;
    const double e = __builtin_fmin(__builtin_fma(-b.d, q, a), 0x1p1023);
    return __builtin_fma(e, b.r, q);
}

// (1 + x) / (1 - x) of atanh.  f64: inside the domain, |x| < 1, the divisor lies in [2^-53, 2] and the dividend in [2^-53, 2], where the
// reciprocal-based quotient (within an ulp) takes a third of the general division sequence.  Everywhere else the logarithm only needs
// the kind of the quotient -- inf at x = 1, 0 at x = -1, negative beyond the domain, NaN for NaN and for +-inf -- which the dividend
// times the raw reciprocal estimate has.  Straight-line code: no lane leaves the wave's path.
__device__ __forceinline__ float atanh_ratio(float x) { return (1.0f + x) / (1.0f - x); }
__device__ __forceinline__ double atanh_ratio(double x) {
    const double a = 1.0 + x, d = 1.0 - x;
    const double q = rt_quot_f64(a, d);
    return __builtin_fabs(x) < 1.0 ? q : a * rt_rcp_seed_f64(d);
}

// 1 / (1 + e) of sigmoid and silu, e = exp(-x) >= 0, and (a - b) / (a + b) of tanh, a = exp(x), b = exp(-x).  f64: the divisor is at
// least 1, so the refined reciprocal (within an ulp) replaces the general division sequence, which is a third of these kernels'
// arithmetic.  The ends of the range are patched by selects, with what the reference's formulas give there: 1 / (1 + inf) = 0;
// (a - b) / (a + b) = +-1 exactly from |x| = 690 on (the smaller exponential is lost in the sum) and inf / inf = NaN once exp overflows.
__device__ __forceinline__ float recip_1p(float e) { return 1.0f / (1.0f + e); }
__device__ __forceinline__ double recip_1p(double e) {
    const double d = 1.0 + e;
    const double r = rt_rcp_f64(d);                              // NaN for d = inf (and for NaN)
    return d == __builtin_inf() ? 0.0 : r;
}
__device__ __forceinline__ float tanh_ratio(float x, float a, float b) { return (a - b) / (a + b); }
__device__ __forceinline__ double tanh_ratio(double x, double a, double b) {
    const double t = a + b;
    const double q = rt_quot_f64(a - b, t);
    const double far = __builtin_copysign(1.0, x) + (t - t);     // t - t: 0 for a finite sum, NaN for inf and NaN
    return __builtin_fabs(x) < 690.0 ? q : far;
}
// exp(-x) next to a = exp(x), for tanh, sinh and cosh.  f64: 1 / a from the refined reciprocal (within an ulp, as the library's
// exponential is) at a quarter of a second exponential's instructions.  Where the refinement has no answer -- a = 0 and a = inf, the
// exponential under- or overflowed -- the raw estimate has the right one (inf, 0).
__device__ __forceinline__ float exp_neg(float x, float a) { return m_exp(-x); }
__device__ __forceinline__ double exp_neg(double x, double a) {
    const double seed = rt_rcp_seed_f64(a);
    double r = __builtin_fma(__builtin_fma(-a, seed, 1.0), seed, seed);
    r = __builtin_fma(__builtin_fma(-a, r, 1.0), r, r);
    return r != r ? seed : r;
}
// sqrt(x^2 + 1) of asinh: the argument is at least 1, so the scaling and the zero / denormal handling of the general square root fall
// away (within an ulp).
__device__ __forceinline__ float sqrt_ge1(float a) { return sqrtf(a); }
__device__ __forceinline__ double sqrt_ge1(double a) { return rt_sqrt_ge1_f64(a); }

// ---- functors ---------------------------------------------------------------------------------------------------
// A functor over 1-byte elements may offer `packed`: the same op on four elements in one 32-bit word (rt_common.h).
// kVectors: 16-byte vectors a lane of the contiguous kernels handles.  One for the ops that are a few instructions per element: the
// wave is gone as soon as its load has come back and been stored.  Four for the ops whose arithmetic takes as long as the memory
// round trip itself (f64 transcendental functions, division-heavy maps): a wave that computes for a microsecond holds its slot
// without having anything in flight, and with one vector per lane the chip runs out of slots before it runs out of bandwidth (f64 ln
// stayed at 0.70 of peak although its ~60 instructions per element are well inside the ALU budget); with all four loads issued first,
// the arithmetic of one vector runs under the latency of the next ones (f64 ln 0.70 -> 0.75, atan 0.70 -> 0.77, sinh 0.70 -> 0.78).
template <int OP, class T> constexpr int unary_vectors() {
    if (std::is_same<T, double>::value) {
        switch (OP) {
            case RT_U_SIGMOID: case RT_U_SILU: case RT_U_EXPM1: return 2;      // measured: 0.82 - 0.83 of peak with two, 0.78 - 0.80 with one or four
            case RT_U_TANH: case RT_U_LN: case RT_U_LN1P: case RT_U_SIN: case RT_U_COS: case RT_U_TAN:
            case RT_U_ASIN: case RT_U_ACOS: case RT_U_ATAN: case RT_U_SINH: case RT_U_COSH: case RT_U_ASINH: case RT_U_ACOSH: case RT_U_ATANH: return 4;
            default: return 1;                      // measured: exp, rsqrt and every f32 op lose 3 .. 8 % with four, the cheap ops 5 % with two
        }
    }
    return 1;
}
// kHeavy: the op's arithmetic is a sizeable part of its time; its contiguous kernels take the block-wise form of the traversal's index
// arithmetic (rt_tile_index_block), which the cheap ops lose 2 % with.
template <int OP, class T> constexpr bool unary_heavy() {
    if (!(std::is_same<T, double>::value || std::is_same<T, float>::value)) return false;
    switch (OP) {
        case RT_U_SIGMOID: case RT_U_SILU: case RT_U_TANH: case RT_U_LN: case RT_U_EXPM1: case RT_U_LN1P: case RT_U_SIN: case RT_U_COS: case RT_U_TAN:
        case RT_U_ASIN: case RT_U_ACOS: case RT_U_ATAN: case RT_U_SINH: case RT_U_COSH: case RT_U_ASINH: case RT_U_ACOSH: case RT_U_ATANH:
            return true;                            // exp alone measured 1 .. 2 % better with the lane form
        default: return false;
    }
}
template <int OP, class T> constexpr bool scalar_heavy() {
    if (std::is_same<T, double>::value || std::is_same<T, float>::value) return OP == RT_S_LOG || OP == RT_S_LOG1P || OP == RT_S_ELU;
    return OP == RT_S_DIV && !is_bool<T>::value;
}
template <int OP, class T> constexpr int scalar_vectors() {
    if (std::is_same<T, double>::value && (OP == RT_S_LOG || OP == RT_S_LOG1P)) return 4;
    if (std::is_same<T, float>::value && OP == RT_S_LOG1P) return 4;
    return 1;                                       // integer division by a scalar measured 3 .. 10 % slower with four
}

template <int OP, class T> struct UnaryF {
    static constexpr bool kReads = true;
    static constexpr int kVectors = unary_vectors<OP, T>();
    static constexpr bool kHeavy = unary_heavy<OP, T>();
    static constexpr bool kPacked = sizeof(T) == 1 && (OP == RT_U_RELU || OP == RT_U_NEG || OP == RT_U_ABS);
    __device__ __forceinline__ uint32_t packed(uint32_t w) const {
        if constexpr (!is_sint<T>::value) {
            // unsigned and bool: relu and abs are the identity; bool negation is 0 ^ x
            if constexpr (OP == RT_U_NEG && is_uint<T>::value) return rt_sub_4x8(0u, w);
            else return w;
        } else {
            if constexpr (OP == RT_U_RELU) return w & ~rt_negmask_4x8(w);
            else if constexpr (OP == RT_U_NEG) return rt_sub_4x8(0u, w);
            else { const uint32_t m = rt_negmask_4x8(w); return rt_sub_4x8(w ^ m, m); }   // two's complement of the negative bytes
        }
    }
    __device__ __forceinline__ T operator()(T x) const {
        if constexpr (OP == RT_U_RELU) {                                  // cpu.rs:650-657
            return gt0(x) ? x : zero_of<T>();
        } else if constexpr (OP == RT_U_ABS) {                            // core/value.rs:515-557
            if constexpr (is_flt<T>::value) return m_abs(x);
            else if constexpr (is_sint<T>::value) return x < 0 ? w_sub<T>((T)0, x) : x;
            else return x;
        } else if constexpr (OP == RT_U_STEP) {                           // ops/unary/mod.rs:234-252
            if constexpr (is_bool<T>::value) return x;
            else return gt0(x) ? (T)1 : (T)0;
        } else if constexpr (OP == RT_U_ABS_GRAD) {                       // ops/unary/mod.rs:213-232
            return gt0(x) ? (T)1 : (T)-1;
        } else if constexpr (OP == RT_U_NEG) {                            // cpu.rs:644-647
            if constexpr (is_flt<T>::value) return -x;
            else return w_sub<T>(zero_of<T>(), x);
        } else {
            const T one = (T)1;
            if constexpr (OP == RT_U_SIGMOID) return recip_1p(m_exp(-x));                         // cpu.rs:661-667
            else if constexpr (OP == RT_U_SILU) return x * recip_1p(m_exp(-x));                   // cpu.rs:669-675
            else if constexpr (OP == RT_U_TANH) { T a = m_exp(x), b = exp_neg(x, a); return tanh_ratio(x, a, b); }   // cpu.rs:624-629
            else if constexpr (OP == RT_U_SQRT) return m_sqrt(x);
            else if constexpr (OP == RT_U_LN) return m_log(x);
            else if constexpr (OP == RT_U_EXPM1) return m_expm1(x);
            else if constexpr (OP == RT_U_LN1P) return m_log1p(x);
            else if constexpr (OP == RT_U_FLOOR) return m_floor(x);
            else if constexpr (OP == RT_U_CEIL) return m_ceil(x);
            else if constexpr (OP == RT_U_ROUND) return m_round(x);
            else if constexpr (OP == RT_U_TRUNC) return m_trunc(x);
            else if constexpr (OP == RT_U_SIN) return m_sin(x);
            else if constexpr (OP == RT_U_COS) return m_cos(x);
            else if constexpr (OP == RT_U_TAN) return m_tan(x);
            else if constexpr (OP == RT_U_ASIN) return m_asin(x);
            else if constexpr (OP == RT_U_ACOS) return m_acos(x);
            else if constexpr (OP == RT_U_ATAN) return m_atan(x);
            else if constexpr (OP == RT_U_SINH) { T a = m_exp(x), b = exp_neg(x, a); return (a - b) / (one + one); }   // cpu.rs:485-490
            else if constexpr (OP == RT_U_COSH) { T a = m_exp(x), b = exp_neg(x, a); return (a + b) / (one + one); }   // cpu.rs:492-497
            else if constexpr (OP == RT_U_ASINH) { T sq = x * x; return m_log(x + sqrt_ge1(sq + one)); }            // cpu.rs:499-505
            else if constexpr (OP == RT_U_ACOSH) { T sq = x * x; return m_log(x + m_sqrt(sq - one)); }              // cpu.rs:507-513
            else if constexpr (OP == RT_U_ATANH) { T two = one + one; return m_log(atanh_ratio(x)) / two; }  // cpu.rs:515-521
            else if constexpr (OP == RT_U_RSQRT) return one / m_sqrt(x);                          // cpu.rs:523-526
            else if constexpr (OP == RT_U_RECIPROCAL) return one / x;                             // cpu.rs:528-531
            else if constexpr (OP == RT_U_SQUARE) return x * x;                                   // cpu.rs:533-536
            else if constexpr (OP == RT_U_CUBE) return x * x * x;                                 // cpu.rs:538-541
            else if constexpr (OP == RT_U_EXP) return m_exp(x);
            else if constexpr (OP == RT_U_SIGN) return x < (T)0 ? -one : (x > (T)0 ? one : (T)0);  // cpu.rs:548-557
            else return x;
        }
    }
};

template <int OP, class T> struct ScalarF {
    static constexpr bool kReads = true;
    static constexpr int kVectors = scalar_vectors<OP, T>();
    static constexpr bool kHeavy = scalar_heavy<OP, T>();
    static constexpr bool kPacked = sizeof(T) == 1 && (OP == RT_S_ADD || OP == RT_S_SUB || (OP == RT_S_MUL && is_bool<T>::value));
    T v;
    int32_t* fault;                     // division of a signed integer by -1 only: set to 1 when an element is MIN (the reference panics)
    int32_t magic = 0;                  // division of 1-byte integers: sign(v) * (65536 / |v| + 1), see div8_magic
    LogBase64 base = {};                // f64 log / log1p: ln(v) and its reciprocal, from the host
    __device__ __forceinline__ uint32_t packed(uint32_t w) const {
        uint8_t b;
        __builtin_memcpy(&b, &v, 1);
        const uint32_t v4 = (uint32_t)b * 0x01010101u;
        if constexpr (is_bool<T>::value) return OP == RT_S_ADD ? (w | v4) : (OP == RT_S_SUB ? (w ^ v4) : (w & v4));
        else return OP == RT_S_ADD ? rt_add_4x8(w, v4) : rt_sub_4x8(w, v4);
    }
    __device__ __forceinline__ T operator()(T x) const {
        if constexpr (OP == RT_S_ADD) return w_add<T>(x, v);                                      // cpu.rs:678-696
        else if constexpr (OP == RT_S_SUB) return w_sub<T>(x, v);
        else if constexpr (OP == RT_S_MUL) return w_mul<T>(x, v);
        else if constexpr (OP == RT_S_DIV) {
            if constexpr (is_sint<T>::value) {
                if (fault && x == min_of<T>()) *fault = 1;                                         // MIN / -1 overflows
            }
            if constexpr (sizeof(T) == 1 && is_sint<T>::value) {
                // x / v for one divisor: the multiplier comes from the host, no reciprocal per element
                const int32_t p = (int32_t)x * magic;
                return (T)((p >> 16) + (int32_t)((uint32_t)p >> 31));
            } else if constexpr (sizeof(T) == 1 && is_uint<T>::value) {
                return (T)(((uint32_t)x * (uint32_t)magic) >> 16);
            } else {
                return w_div<T>(x, v);
            }
        }
        else if constexpr (OP == RT_S_LEAKY_RELU) return gt0(x) ? x : w_mul<T>(x, v);             // cpu.rs:708-715
        else if constexpr (OP == RT_S_LOG) {                                                      // f32::log(base) = ln(x) / ln(base)
            if constexpr (std::is_same<T, double>::value) return over_log_base(m_log(x), base);
            else return over_log_base(m_log(x), v);
        } else if constexpr (OP == RT_S_LOG1P) {                                                  // core/value.rs vlog1p
            if constexpr (std::is_same<T, double>::value) return over_log_base(m_log1p(x), base);
            else return over_log_base(m_log1p(x), v);
        }
        else if constexpr (OP == RT_S_ELU) return x >= (T)0 ? x : v * m_expm1(x);                 // cpu.rs:717-724
        else if constexpr (OP == RT_S_LEAKY_GRAD) return gt0(x) ? one_of<T>() : v;                // ops/scalar/mod.rs:149-166
        else return x;
    }
};

// Multiplier for the division of a 1-byte integer by v != 0: for |a|, |v| < 256 the truncating quotient a / v is (p >> 16) + (p < 0)
// with p = a * sign(v) * (65536 / |v| + 1) -- the product overshoots |a| / |v| by less than 256 / 65536, below the 1 / |v| to the next
// integer, and is never a whole multiple of 65536 unless it is 0 (all pairs checked against integer arithmetic).
inline int32_t div8_magic(int32_t v) {
    const int32_t mag = v < 0 ? -v : v;
    const int32_t m = mag ? 65536 / mag + 1 : 0;
    return v < 0 ? -m : m;
}

template <class T> struct FillF {
    static constexpr bool kReads = false;
    static constexpr int kVectors = 1;
    static constexpr bool kHeavy = false;
    static constexpr bool kPacked = false;
    T v;
    __device__ __forceinline__ T operator()(T) const { return v; }
};

// ---- kernels ------------------------------------------------------------------------------------------------------
template <class T> struct alignas(16) Vec16 { T e[16 / sizeof(T)]; };

template <class T, class F> __device__ __forceinline__ void apply_vec(Vec16<T>& v, const F& f) {
    if constexpr (F::kPacked) {
        rt_words4 w = __builtin_bit_cast(rt_words4, v);
#pragma unroll
        for (int j = 0; j < 4; ++j) w.w[j] = f.packed(w.w[j]);
        v = __builtin_bit_cast(Vec16<T>, w);
    } else {
#pragma unroll
        for (int j = 0; j < (int)(16 / sizeof(T)); ++j) v.e[j] = f(v.e[j]);
    }
}

constexpr int kBlock = 256;     // element-per-lane kernels
constexpr int kCBlock = 128;    // contiguous kernel: one 16-byte vector per lane, 128 lanes per block
constexpr int kEU = 4;          // element-per-lane kernels: elements in flight per lane

template <class F> __device__ __forceinline__ bool ew_tile_index(const TileMap& m, uint32_t block, uint32_t nthreads, uint32_t tid, size_t nvec, size_t* out) {
    if constexpr (F::kHeavy) return rt_tile_index_block(m, block, nthreads, tid, nvec, out);
    else return rt_tile_index(m, block, nthreads, tid, nvec, out);
}

// Body: `nvec` 16-byte vectors starting at the 16-byte aligned address `p`.  One vector per lane and small blocks:
// on MI355X this shape (with non-temporal accesses for read-modify-write, plain stores for write-only) was the
// fastest of the block-size / unroll / grid-stride variants tried, ~6.7 TB/s in place and ~6.8 TB/s for fill.
template <class T, class F>
__global__ __launch_bounds__(512) void ew_contig_kernel(Vec16<T>* __restrict__ p, size_t nvec, uint32_t head, uint32_t tail, TileMap m, F f) {
    // The `head` elements before and the `tail` elements after the 16-byte aligned body (fewer than a vector each) are taken by
    // lanes of the first and the last block: launches of their own cost a run that starts off a 16-byte boundary 9 % (1 GiB f32
    // `+= 1`: 0.363 ms with three launches against 0.331 ms aligned).
    if (blockIdx.x == 0 && threadIdx.x < head) {
        T* e = reinterpret_cast<T*>(p) - head + threadIdx.x;
        T x = zero_of<T>();
        if constexpr (F::kReads) x = *e;
        *e = f(x);
    }
    if (blockIdx.x == gridDim.x - 1 && threadIdx.x < tail) {
        T* e = reinterpret_cast<T*>(p + nvec) + threadIdx.x;
        T x = zero_of<T>();
        if constexpr (F::kReads) x = *e;
        *e = f(x);
    }
    // a block stands for kVectors consecutive blocks of the one-vector-per-lane traversal; every load is issued before the first use
    constexpr int U = F::kVectors;
    if constexpr (U == 1) {
        size_t i1;
        if (!ew_tile_index<F>(m, blockIdx.x, blockDim.x, threadIdx.x, nvec, &i1)) return;
        Vec16<T> v1;
        if constexpr (F::kReads) v1 = rt_ld16_nt(p + i1);
        apply_vec(v1, f);
        rt_st16_nt(p + i1, v1);
        return;
    }
    size_t i[U];
    bool has[U];
    Vec16<T> v[U];
#pragma unroll
    for (int u = 0; u < U; ++u) {
        has[u] = ew_tile_index<F>(m, blockIdx.x * U + u, blockDim.x, threadIdx.x, nvec, &i[u]);
        if constexpr (F::kReads) { if (has[u]) v[u] = rt_ld16_nt(p + i[u]); }
    }
#pragma unroll
    for (int u = 0; u < U; ++u) {
        if (has[u]) {
            apply_vec(v[u], f);
            rt_st16_nt(p + i[u], v[u]);
        }
    }
}

// Edges of a contiguous run that do not fill a 16-byte vector, and 1-D strided views: one element per lane.
template <class T, class F>
__global__ __launch_bounds__(kBlock) void ew_strided_kernel(T* __restrict__ p, int64_t stride, size_t n, F f) {
    // A block owns kEU * kBlock consecutive elements per trip, lane t the elements t, t + kBlock, ...; all loads are issued
    // before the first store (loads and stores retire in issue order, so a load -> store -> load chain would wait for
    // every store)
    const size_t span = (size_t)kEU * kBlock;
    for (size_t base = (size_t)blockIdx.x * span; base < n; base += (size_t)gridDim.x * span) {
        T x[kEU];
#pragma unroll
        for (int u = 0; u < kEU; ++u) {
            const size_t i = base + (size_t)u * kBlock + threadIdx.x;
            x[u] = zero_of<T>();
            if constexpr (F::kReads) { if (i < n) x[u] = p[(int64_t)i * stride]; }
        }
#pragma unroll
        for (int u = 0; u < kEU; ++u) {
            const size_t i = base + (size_t)u * kBlock + threadIdx.x;
            if (i < n) p[(int64_t)i * stride] = f(x[u]);
        }
    }
}

struct NdArgs {
    int rank;                        // >= 2
    uint32_t shape[RT_MAX_RANK];
    int64_t stride[RT_MAX_RANK];
    FastDiv32 div[RT_MAX_RANK];
};

// N-d view, fewer than 2^31 elements: lane i handles the i-th element in row-major order of the collapsed dims.
template <class T, class F>
__global__ __launch_bounds__(kBlock) void ew_nd_kernel(T* __restrict__ p, NdArgs a, uint32_t n, F f) {
    // a block owns kEU * kBlock consecutive elements per trip (n < 2^31, so base + span does not wrap)
    constexpr uint32_t span = kEU * kBlock;
    for (uint64_t base = (uint64_t)blockIdx.x * span; base < n; base += (uint64_t)gridDim.x * span) {
        const uint32_t i = (uint32_t)base + threadIdx.x;
        constexpr uint32_t step = kBlock;
        int64_t off[kEU];
        T x[kEU];
#pragma unroll
        for (int u = 0; u < kEU; ++u) {
            uint32_t rem = min(i + u * step, n - 1);
            off[u] = 0;
#pragma unroll
            for (int d = RT_MAX_RANK - 1; d >= 0; --d) {
                if (d < a.rank) {
                    uint32_t q = fd_div(rem, a.div[d]);
                    uint32_t c = rem - q * a.shape[d];
                    off[u] += (int64_t)c * a.stride[d];
                    rem = q;
                }
            }
            x[u] = zero_of<T>();
            if constexpr (F::kReads) { if (i + u * step < n) x[u] = p[off[u]]; }
        }
#pragma unroll
        for (int u = 0; u < kEU; ++u)
            if (i + u * step < n) p[off[u]] = f(x[u]);
    }
}

// N-d view whose innermost collapsed dim is unit-stride (row ranges, sub-blocks of a matrix ...).  Same work shape as the
// broadcast row kernel: 128-lane blocks, one 16-byte vector per lane and step, two steps along the innermost outer dim
// per block; (outer index, chunk, column tile) from blockIdx by multiply-high division on the scalar unit.
struct RowsArgs {
    uint32_t L, G, gchunk, nchunks, tiles, tpr;
    FastDiv32 tiles_div, nchunks_div;
    int nouter;
    uint32_t oshape[RT_MAX_RANK];
    FastDiv32 odiv[RT_MAX_RANK];
    int64_t ostride[1][RT_MAX_RANK];
    int64_t gstride;
};

// NT: every row covers whole 128-byte lines, so the view is streamed with non-temporal accesses.  Rows that share cache lines
// with elements outside the view go through the cache normally, so that the partly written lines are merged in L2 instead of
// being written to memory piece by piece ((2^24, 16)[:, :15] f32 relu: 0.92 ms non-temporal, 0.62 ms cached).
template <class T, class F, bool NT>
__global__ __launch_bounds__(kCBlock) void ew_rows_kernel(T* __restrict__ p, RowsArgs a, F f) {
    constexpr int N = 16 / sizeof(T);
    uint32_t b = blockIdx.x;
    uint32_t q = fd_div(b, a.tiles_div);
    const uint32_t tile = b - q * a.tiles;
    b = q;
    q = fd_div(b, a.nchunks_div);
    const uint32_t chunk = b - q * a.nchunks;
    int64_t off1[1];
    rt_outer_offsets<1>(q, a.nouter, a.oshape, a.odiv, a.ostride, off1);
    const int64_t off = off1[0];
    const uint32_t tx = threadIdx.x & (a.tpr - 1), ty = threadIdx.x / a.tpr, gy = kCBlock / a.tpr;
    const uint32_t c = (tile * a.tpr + tx) * N;
    if (c >= a.L) return;
    const uint32_t g_begin = chunk * a.gchunk, g_end = min(a.G, g_begin + a.gchunk);
    if (c + N <= a.L) {
        // two rows per trip, both loads issued before the first store
        for (uint32_t g = g_begin + ty; g < g_end; g += 2 * gy) {
            const bool two = g + gy < g_end;
            // vectors stay four 32-bit words across the conditional loads (arrays of 1-byte elements would be split up and re-packed)
            // rows may start at any element: 16-byte accesses at element alignment
            T* v0 = p + off + (int64_t)g * a.gstride + c;
            T* v1 = p + off + (int64_t)(two ? g + gy : g) * a.gstride + c;
            rt_u32x4 w0 = {}, w1 = {};
            if constexpr (F::kReads) {
                w0 = rt_ld16u<T, NT>(v0);
                if (two) w1 = rt_ld16u<T, NT>(v1);
            }
            Vec16<T> e0 = __builtin_bit_cast(Vec16<T>, w0), e1 = __builtin_bit_cast(Vec16<T>, w1);
            apply_vec(e0, f);
            apply_vec(e1, f);
            w0 = __builtin_bit_cast(rt_u32x4, e0);
            w1 = __builtin_bit_cast(rt_u32x4, e1);
            if constexpr (F::kReads && NT) {
                rt_st16u_nt<T>(v0, w0);
                if (two) rt_st16u_nt<T>(v1, w1);
            } else {
                rt_st16u<T>(v0, w0);
                if (two) rt_st16u<T>(v1, w1);
            }
        }
    } else {
        for (uint32_t g = g_begin + ty; g < g_end; g += gy) {
            T* rowp = p + off + (int64_t)g * a.gstride;
            for (uint32_t k = c; k < a.L; ++k) {
                T x = zero_of<T>();
                if constexpr (F::kReads) x = rowp[k];
                rowp[k] = f(x);
            }
        }
    }
}

// Lean form of the row kernel for rows of at least 128 vectors and at most two outer dims besides the row dim: a 256-lane block owns
// the same 1 KiB piece of four consecutive rows, one wave per row, one vector per lane; the outer dims are grid dims y / z, every
// kernel argument is fetched in one batch and all offsets fit 32 bits (checked on the host).  A wave's whole life is one load,
// the op and one store.  relu in place on the left half of a 16384 x 16384 f32 matrix: 0.79 -> 0.85 of peak.
struct Rows4Args {
    uint32_t L, G, tiles;
    FastDiv32 tiles_div;
    int32_t gs, o0s, o1s;           // strides along the row dim and the two outer dims (inner one first)
};

// A wave's 64 vectors sit on the 128-byte line grid of memory whatever the start of the row: the lane's column is shifted back by the
// row's phase (its distance from the line boundary below it, see rt_row_tiling), lanes wholly before the row do nothing, and the up
// to N - 1 elements before the first whole vector and after the last one are handled one by one.  (Vectors at element alignment
// cost `m[:, 1:]` of a 65536 x 4096 f32 matrix 0.72 of peak with cached and 0.63 with non-temporal accesses; 0.83 so, all accesses
// non-temporal.  A fill of all but three columns of that matrix: 0.51 -> 0.76.  On the 16-byte grid only, a wave of a row that
// starts 16 or 32 bytes into a line shares its first and last line with its neighbours: relu on m[:, 4:C-4] of that matrix 0.70
// against 0.85 on the line grid, on m[:, 1:] of 65536 x 4095, where every row has its own phase, 0.65 against 0.81.)
template <class T, class F>
__global__ __launch_bounds__(256) void ew_rows4_kernel(T* p, Rows4Args a, F f) {
    constexpr int N = 16 / sizeof(T);
    uint32_t L = a.L, G = a.G, tiles = a.tiles, tm = a.tiles_div.mul, ts = a.tiles_div.shift;
    int32_t gs = a.gs, o0 = a.o0s, o1 = a.o1s;
    RT_PIN(L); RT_PIN(G); RT_PIN(tiles); RT_PIN(tm); RT_PIN(ts); RT_PIN(gs); RT_PIN(o0); RT_PIN(o1);
    RT_TOUCH(p);
    const uint32_t chunk = (uint32_t)(((uint64_t)__umulhi(blockIdx.x, tm) + blockIdx.x) >> ts);
    const uint32_t tile = blockIdx.x - chunk * tiles;
    const uint32_t g = chunk * 4 + (uint32_t)__builtin_amdgcn_readfirstlane((int)(threadIdx.x >> 6));
    if (g >= G) return;
    T* rowp = p + ((int32_t)blockIdx.z * o1 + (int32_t)blockIdx.y * o0 + (int32_t)g * gs);
    const uint32_t phase = (uint32_t)((reinterpret_cast<uintptr_t>(rowp) / sizeof(T)) & (uintptr_t)(128 / sizeof(T) - 1));
    const int32_t c = (int32_t)((tile * 64 + (threadIdx.x & 63)) * N) - (int32_t)phase;
    if (c >= (int32_t)L || c + (int32_t)N <= 0) return;
    if (c >= 0 && (uint32_t)c + N <= L) {
        Vec16<T>* vp = reinterpret_cast<Vec16<T>*>(rowp + c);
        Vec16<T> e = {};
        if constexpr (F::kReads) e = rt_ld16_nt(vp);
        apply_vec(e, f);
        rt_st16_nt(vp, e);
    } else {
        // the ragged ends of a row: all loads, then all stores
        const uint32_t k0 = c < 0 ? 0u : (uint32_t)c, k1 = min((uint32_t)(c + N), L);
        T x[N];
#pragma unroll
        for (int j = 0; j < N; ++j) {
            x[j] = zero_of<T>();
            if constexpr (F::kReads) { if (k0 + j < k1) x[j] = rowp[k0 + j]; }
        }
#pragma unroll
        for (int j = 0; j < N; ++j)
            if (k0 + j < k1) rowp[k0 + j] = f(x[j]);
    }
}

// 64-bit fallback for views with 2^31 or more elements that are not a single contiguous run.
template <class T, class F>
__global__ __launch_bounds__(kBlock) void ew_nd64_kernel(T* __restrict__ p, NdDesc d, uint64_t n, F f) {
    uint64_t i = (uint64_t)blockIdx.x * kBlock + threadIdx.x;
    const uint64_t step = (uint64_t)gridDim.x * kBlock;
    for (; i < n; i += step) {
        uint64_t rem = i;
        int64_t off = 0;
        for (int k = d.rank - 1; k >= 0; --k) {
            uint64_t q = rem / (uint64_t)d.shape[k];
            off += (int64_t)(rem - q * (uint64_t)d.shape[k]) * d.stride[0][k];
            rem = q;
        }
        T* q = p + off;
        T x = zero_of<T>();
        if constexpr (F::kReads) x = *q;
        *q = f(x);
    }
}

// Views that keep more than RT_MAX_RANK dims after collapsing (the reference accepts rank <= 128, core/primitives.rs:377-383):
// shape and strides are read from device memory (words[0 .. rank) = shape, words[rank .. 2 rank) = strides).
template <class T, class F>
__global__ __launch_bounds__(kBlock) void ew_big_kernel(T* __restrict__ p, const int64_t* __restrict__ w, int rank, uint64_t n, F f) {
    uint64_t i = (uint64_t)blockIdx.x * kBlock + threadIdx.x;
    const uint64_t step = (uint64_t)gridDim.x * kBlock;
    for (; i < n; i += step) {
        uint64_t rem = i;
        int64_t off = 0;
        for (int k = rank - 1; k >= 0; --k) {
            const uint64_t sh = (uint64_t)w[k];
            const uint64_t q = rem / sh;
            off += (int64_t)(rem - q * sh) * w[rank + k];
            rem = q;
        }
        T* q = p + off;
        T x = zero_of<T>();
        if constexpr (F::kReads) x = *q;
        *q = f(x);
    }
}

// ---- launch logic ---------------------------------------------------------------------------------------------------
constexpr uintptr_t kBodyAlign = 128;        // at most 127 one-byte elements before the body: fewer than the lanes of a block
static inline unsigned capped_grid(size_t blocks, size_t cap) { return (unsigned)(blocks < 1 ? 1 : (blocks > cap ? cap : blocks)); }

template <class T, class F>
int32_t launch_contig(rt_ctx* ctx, T* p, size_t n, F f) {
    if (n == 0) return RT_OK;
    constexpr size_t N = 16 / sizeof(T);
    // The vector body starts on a 128-byte line, not merely on a 16-byte boundary, so that a wave's 1 KiB covers eight whole
    // lines; with the body 16 bytes into a line every wave shares its first and last line with a neighbour and the pass is 9 %
    // slower (1 GiB f32 `+= 1` from element 1: 0.361 ms, aligned 0.331 ms).  The up to 127 bytes before it are edge elements.
    uintptr_t addr = reinterpret_cast<uintptr_t>(p);
    size_t head = ((kBodyAlign - (addr & (kBodyAlign - 1))) & (kBodyAlign - 1)) / sizeof(T);
    if (head > n) head = n;
    size_t nvec = (n - head) / N;
    size_t tail = n - head - nvec * N;
    // read-modify-write: 256 lanes, a block owns a 1 KiB quarter of four neighbouring pages; pure stores: 512 lanes, 1 KiB pieces of
    // pages 64 KiB apart (see TileMap)
    const uint32_t bs = F::kReads ? 256u : 512u;
    const TileMap m = F::kReads ? rt_make_tilemap(p + head, nvec, bs) : rt_make_tilemap(p + head, nvec, bs, 1024, 16, 65536);
    size_t blocks = (rt_tilemap_blocks(m, nvec, bs) + F::kVectors - 1) / F::kVectors;
    if (blocks < 1) blocks = 1;                                           // a run shorter than a vector: edges only
    if (blocks > 0x7fffffffull) return rt_fail(RT_E_INVALID, "contiguous run of %zu elements is too long for one launch", n);
    RT_TRY(rt_check_edges("elementwise", head, nvec, N, tail, n, bs));
    hipLaunchKernelGGL((ew_contig_kernel<T, F>), dim3((unsigned)blocks), dim3(bs), 0, ctx->stream,
                       reinterpret_cast<Vec16<T>*>(p + head), nvec, (uint32_t)head, (uint32_t)tail, m, f);
    RT_HIP(hipGetLastError());
    return RT_OK;
}

// Out of place: dst[i] = f(src[i]) for a contiguous run; what `tensor.op()` needs instead of clone + in-place op, at half the
// traffic (2 * N * sizeof(T) instead of 4 * N * sizeof(T)).
template <class T, class F>
__global__ __launch_bounds__(256) void ew_contig_out_kernel(const T* __restrict__ s, T* __restrict__ d, size_t nvec, uint32_t head, uint32_t tail, TileMap m, F f) {
    constexpr size_t N = 16 / sizeof(T);
    // s and d point at the vector body, which starts on a 128-byte line of d; the `head` elements before it and the `tail`
    // elements after it go to lanes of the first and the last block
    if (blockIdx.x == 0 && threadIdx.x < head) { const int64_t e = (int64_t)threadIdx.x - (int64_t)head; d[e] = f(s[e]); }
    if (blockIdx.x == gridDim.x - 1 && threadIdx.x < tail) { const size_t e = nvec * N + threadIdx.x; d[e] = f(s[e]); }
    constexpr int U = F::kVectors;
    if constexpr (U == 1) {
        size_t i1;
        if (!ew_tile_index<F>(m, blockIdx.x, 256, threadIdx.x, nvec, &i1)) return;
        Vec16<T> v1 = __builtin_bit_cast(Vec16<T>, rt_ld16u<T, true>(s + i1 * N));        // the source may be in any phase
        apply_vec(v1, f);
        rt_st16_nt(reinterpret_cast<Vec16<T>*>(d) + i1, v1);
        return;
    }
    size_t i[U];
    bool has[U];
    rt_u32x4 w[U];
#pragma unroll
    for (int u = 0; u < U; ++u) {
        has[u] = ew_tile_index<F>(m, blockIdx.x * U + u, 256, threadIdx.x, nvec, &i[u]);
        if (has[u]) w[u] = rt_ld16u<T, true>(s + i[u] * N);                              // the source may be in any phase
    }
#pragma unroll
    for (int u = 0; u < U; ++u) {
        if (has[u]) {
            Vec16<T> v = __builtin_bit_cast(Vec16<T>, w[u]);
            apply_vec(v, f);
            rt_st16_nt(reinterpret_cast<Vec16<T>*>(d) + i[u], v);
        }
    }
}

template <class T, class F>
int32_t launch_contig_out(rt_ctx* ctx, const T* s, T* d, size_t n, F f) {
    constexpr size_t N = 16 / sizeof(T);
    if (n == 0) return RT_OK;
    const uintptr_t addr = reinterpret_cast<uintptr_t>(d);
    size_t head = ((kBodyAlign - (addr & (kBodyAlign - 1))) & (kBodyAlign - 1)) / sizeof(T);
    if (head > n) head = n;
    const size_t nvec = (n - head) / N, tail = n - head - nvec * N;
    const TileMap m = rt_make_tilemap(d + head, nvec, 256);
    size_t blocks = (rt_tilemap_blocks(m, nvec, 256) + F::kVectors - 1) / F::kVectors;
    if (blocks < 1) blocks = 1;
    if (blocks > 0x7fffffffull) return rt_fail(RT_E_INVALID, "contiguous run of %zu elements is too long for one launch", n);
    RT_TRY(rt_check_edges("elementwise", head, nvec, N, tail, n, 256));
    hipLaunchKernelGGL((ew_contig_out_kernel<T, F>), dim3((unsigned)blocks), dim3(256), 0, ctx->stream, s + head, d + head, nvec, (uint32_t)head,
                       (uint32_t)tail, m, f);
    RT_HIP(hipGetLastError());
    return RT_OK;
}

// `d` is the collapsed single-operand view (operand 0), any element order allowed.
template <class T, class F>
int32_t launch_view(rt_ctx* ctx, T* base, const NdDesc& d, uint64_t count, F f) {
    if (count == 0) return RT_OK;
    T* p = base + d.offset[0];
    if (d.rank == 0) return launch_contig<T, F>(ctx, p, 1, f);
    if (d.rank == 1) {
        if (d.stride[0][0] == 1) return launch_contig<T, F>(ctx, p, (size_t)d.shape[0], f);
        size_t blocks = ((size_t)d.shape[0] + kEU * kBlock - 1) / (kEU * kBlock);
        hipLaunchKernelGGL((ew_strided_kernel<T, F>), dim3(capped_grid(blocks, 0x7fffffffull)), dim3(kBlock), 0, ctx->stream,
                           p, d.stride[0][0], (size_t)d.shape[0], f);
        RT_HIP(hipGetLastError());
        return RT_OK;
    }
    if (count >= (1ull << 31) && d.rank >= 2)                     // slices along the outermost dim, each through the 32-bit kernels below
        return rt_for_slices_below_2g(d, count, [&](const NdDesc& sub, uint64_t n) { return launch_view<T, F>(ctx, base, sub, n, f); });
    if (count >= (1ull << 31)) {
        size_t blocks = (size_t)((count + kBlock - 1) / kBlock);
        hipLaunchKernelGGL((ew_nd64_kernel<T, F>), dim3(capped_grid(blocks, (size_t)ctx->num_cus * 64)), dim3(kBlock), 0, ctx->stream,
                           p, d, count, f);
        RT_HIP(hipGetLastError());
        return RT_OK;
    }
    NdArgs a;
    a.rank = d.rank;
    for (int i = 0; i < RT_MAX_RANK; ++i) {
        a.shape[i] = i < d.rank ? (uint32_t)d.shape[i] : 1;
        a.stride[i] = i < d.rank ? d.stride[0][i] : 0;
        a.div[i] = make_fastdiv(a.shape[i]);
    }
    constexpr int64_t N = 16 / sizeof(T);
    // rows form: unit-stride inner dim of at least two vectors; the rows may start at any element (`m[:, 1:]` of a 8192 x 32768
    // f32 matrix: relu in place 0.57 ms element by element, 0.36 ms with unaligned vectors)
    // (not when a block would be left with a couple of short rows -- rows of 17 under a loop dim of 3, relu on m[..., :17] of
    // (310689, 3, 3, 18) f32: 0.16 of peak; the element kernel below takes those)
    const bool rows_ok = d.stride[0][d.rank - 1] == 1 && d.shape[d.rank - 1] >= 2 * N &&
                         (uint64_t)d.shape[d.rank - 1] * (uint64_t)d.shape[d.rank - 2] * sizeof(T) >= 2048;
    if (rows_ok) {
        RowsArgs r;
        memset(&r, 0, sizeof(r));
        const int gdim = d.rank - 2;
        r.L = (uint32_t)d.shape[d.rank - 1];
        r.G = (uint32_t)d.shape[gdim];
        r.gstride = d.stride[0][gdim];
        bool whole_lines = ((uint64_t)r.L * sizeof(T)) % 128 == 0 && (reinterpret_cast<uintptr_t>(p) & 127) == 0 && (r.gstride * (int64_t)sizeof(T)) % 128 == 0;
        uint64_t outer = 1;
        for (int k = 0; k < gdim; ++k) {
            r.oshape[r.nouter] = (uint32_t)d.shape[k];
            r.odiv[r.nouter] = make_fastdiv((uint32_t)d.shape[k]);
            r.ostride[0][r.nouter] = d.stride[0][k];
            if ((d.stride[0][k] * (int64_t)sizeof(T)) % 128 != 0) whole_lines = false;
            outer *= (uint64_t)d.shape[k];
            r.nouter++;
        }
        for (int k = r.nouter; k < RT_MAX_RANK; ++k) { r.oshape[k] = 1; r.odiv[k] = make_fastdiv(1); }
        const uint32_t vecs = (uint32_t)((r.L + N - 1) / N);
        // The lean kernel takes rows of 128 vectors and more; shorter ones, down to 32 vectors, when they are whole vectors and fill
        // their tiles to 85 % (rows of one partly filled or ragged tile measured faster on the general kernel below: relu on m[:, 1:]
        // of 2^20 x 256 f32 0.71 against 0.68, on m[:, :128] 0.74 against 0.68; but on m[:, 16:C-16] of 2^19 x 512 0.64 against 0.81)
        const RowTiling rt = rt_row_tiling(reinterpret_cast<uintptr_t>(p) / sizeof(T), d.stride[0], d.rank - 1, r.L, (uint32_t)sizeof(T));
        const bool lean = vecs >= 128 || (vecs >= 32 && !rt.ragged && (uint64_t)vecs * 100 >= (uint64_t)rt.tiles * 64 * 85);
        if (lean && r.G >= 4 && d.rank <= 4) {
            uint64_t reach = 0;
            for (int k = 0; k < d.rank; ++k) reach += (uint64_t)(d.shape[k] - 1) * (uint64_t)(d.stride[0][k] < 0 ? -d.stride[0][k] : d.stride[0][k]);
            const uint64_t n0 = d.rank >= 3 ? (uint64_t)d.shape[d.rank - 3] : 1ull, n1 = d.rank >= 4 ? (uint64_t)d.shape[d.rank - 4] : 1ull;
            Rows4Args q;
            q.L = r.L; q.G = r.G;
            q.tiles = rt.tiles;
            // Rows with ragged ends that are read and written: an odd number of tiles per row.  Blocks go to the eight XCDs in turn, so
            // with an even count the first tile of every row -- whose first lane handles the row's ragged start element by element, the
            // longest-lived wave of the row -- keeps landing on the same few XCDs, and the last tile on others.  One more (empty) tile
            // makes the assignment drift: relu on m[:, 1:] of 65536 x 4096 f32 0.70 -> 0.84 of peak, of 8192 x 32768 0.82 -> 0.85, of
            // 262144 x 1024 0.66 -> 0.76, of 524288 x 512 0.70 -> 0.76.  Rotating the tile index instead was slower for long rows, and fills (no loads, nothing
            // long-lived) lose 10 % either way and keep the exact count.
            const bool ragged = rt.ragged;
            if (F::kReads && ragged && q.tiles % 2 == 0) q.tiles += 1;
            q.tiles_div = make_fastdiv(q.tiles);
            const uint64_t gx = (uint64_t)q.tiles * ((r.G + 3) / 4);
            if (reach < (1ull << 31) && n0 <= 65535 && n1 <= 65535 && gx < (1ull << 31)) {
                q.gs = (int32_t)r.gstride;
                q.o0s = d.rank >= 3 ? (int32_t)d.stride[0][d.rank - 3] : 0;
                q.o1s = d.rank >= 4 ? (int32_t)d.stride[0][d.rank - 4] : 0;
                const dim3 grid((unsigned)gx, (unsigned)n0, (unsigned)n1);
                hipLaunchKernelGGL((ew_rows4_kernel<T, F>), grid, dim3(256), 0, ctx->stream, p, q, f);
                RT_HIP(hipGetLastError());
                return RT_OK;
            }
        }
        uint32_t tpr = 1;
        while (tpr < vecs && tpr < (uint32_t)kCBlock) tpr <<= 1;
        r.tpr = tpr;
        r.tiles = (vecs + tpr - 1) / tpr;
        uint32_t gchunk = (kCBlock / tpr) * 2;
        if (gchunk > r.G) gchunk = r.G;
        r.gchunk = gchunk;
        r.nchunks = (r.G + gchunk - 1) / gchunk;
        r.tiles_div = make_fastdiv(r.tiles);
        r.nchunks_div = make_fastdiv(r.nchunks);
        const uint64_t blocks = outer * r.nchunks * r.tiles;
        if (blocks < (1ull << 31)) {
            if (whole_lines) hipLaunchKernelGGL((ew_rows_kernel<T, F, true>), dim3((unsigned)blocks), dim3(kCBlock), 0, ctx->stream, p, r, f);
            else hipLaunchKernelGGL((ew_rows_kernel<T, F, false>), dim3((unsigned)blocks), dim3(kCBlock), 0, ctx->stream, p, r, f);
            RT_HIP(hipGetLastError());
            return RT_OK;
        }
    }
    size_t blocks = ((size_t)count + kEU * kBlock - 1) / (kEU * kBlock);
    hipLaunchKernelGGL((ew_nd_kernel<T, F>), dim3(capped_grid(blocks, 0x7fffffffull)), dim3(kBlock), 0, ctx->stream,
                       p, a, (uint32_t)count, f);
    RT_HIP(hipGetLastError());
    return RT_OK;
}

// One operand view; `dst` null = in place, else the results go to dst[0 .. count) and the view itself is only read.
struct ViewArg {
    void* buf;
    uint64_t buf_len;
    uint64_t offset;
    int rank;
    const uint64_t* shape;
    const int64_t* strides;
    void* dst;
    uint64_t dst_len;
};

// validate + collapse one view, then run F over it
template <class T, class F>
int32_t run_view(rt_ctx* ctx, const char* what, const ViewArg& va, F f) {
    uint64_t count = 0;
    uint64_t offset = va.offset;
    RT_TRY(rt_check_extent(what, offset, va.rank, va.shape, va.strides, va.buf_len, &count));
    if (va.dst && count > va.dst_len)
        return rt_fail(RT_E_OUT_OF_BOUNDS, "%s: %llu results into a buffer of %llu elements", what, (unsigned long long)count, (unsigned long long)va.dst_len);
    if (count == 0) return RT_OK;
    if (!va.buf) return rt_fail(RT_E_INVALID, "%s: null buffer", what);
    if (!va.dst) {
        for (int i = 0; i < va.rank; ++i)
            if (va.shape[i] > 1 && va.strides[i] == 0)
                return rt_fail(RT_E_INVALID, "%s: an in-place op over a zero-stride dim would write one element %llu times", what,
                               (unsigned long long)va.shape[i]);
    }
    NdDesc d;
    const int64_t* sp[1] = {va.strides};
    // out of place the element order matters (dst is row-major): no reordering of dims
    const int32_t cst = rt_collapse(1, va.rank, va.shape, sp, &offset, /*reorder=*/va.dst == nullptr, 0, &d);
    CtxGuard g(ctx);
    if (cst == RT_E_RANK && !va.dst) {
        // more than RT_MAX_RANK dims remain: descriptor in device memory, rank-generic kernel
        BigDesc b;
        RT_TRY(rt_collapse_big(ctx, 1, va.rank, va.shape, sp, &offset, /*reorder=*/true, 0, &b));
        const size_t blocks = (size_t)((count + kBlock - 1) / kBlock);
        hipLaunchKernelGGL((ew_big_kernel<T, F>), dim3(capped_grid(blocks, (size_t)ctx->num_cus * 64)), dim3(kBlock), 0, ctx->stream,
                           (T*)va.buf + b.offset[0], b.words, b.rank, count, f);
        RT_HIP(hipGetLastError());
        return RT_OK;
    }
    if (cst == RT_E_RANK)
        return rt_fail(RT_E_WRONG_DIMS, "%s: the out-of-place form takes a forward contiguous run (gather other views first)", what);
    RT_TRY(cst);
    if (!va.dst) return launch_view<T, F>(ctx, (T*)va.buf, d, count, f);
    if (va.dst == va.buf) return rt_fail(RT_E_INVALID, "%s: the out-of-place form needs a destination other than the source", what);
    if (!(d.rank == 0 || (d.rank == 1 && d.stride[0][0] == 1)))
        return rt_fail(RT_E_WRONG_DIMS, "%s: the out-of-place form takes a forward contiguous run (gather other views first)", what);
    if (rt_spans_meet(rt_run_span(va.buf, (int)sizeof(T), (uint64_t)d.offset[0], count), rt_run_span(va.dst, (int)sizeof(T), 0, count)))
        return rt_fail(RT_E_INVALID, "%s: the destination overlaps the source run", what);
    return launch_contig_out<T, F>(ctx, (const T*)va.buf + d.offset[0], (T*)va.dst, (size_t)count, f);
}

template <class T> T load_scalar(const void* v) { T x; memcpy(&x, v, sizeof(T)); return x; }

// ---- dtype / op dispatch ----------------------------------------------------------------------------------------------
#define RT_FOR_DTYPE(dtype, BODY)                                           \
    switch (dtype) {                                                        \
        case RT_U8: { typedef uint8_t T; BODY; } break;                     \
        case RT_I8: { typedef int8_t T; BODY; } break;                      \
        case RT_U16: { typedef uint16_t T; BODY; } break;                   \
        case RT_I16: { typedef int16_t T; BODY; } break;                    \
        case RT_U32: { typedef uint32_t T; BODY; } break;                   \
        case RT_I32: { typedef int32_t T; BODY; } break;                    \
        case RT_U64: { typedef uint64_t T; BODY; } break;                   \
        case RT_I64: { typedef int64_t T; BODY; } break;                    \
        case RT_U128: { typedef u128_t T; BODY; } break;                    \
        case RT_I128: { typedef i128_t T; BODY; } break;                    \
        case RT_F32: { typedef float T; BODY; } break;                      \
        case RT_F64: { typedef double T; BODY; } break;                     \
        case RT_BOOL: { typedef boolean_t T; BODY; } break;                 \
        default: break;                                                     \
    }

int32_t no_dtype(const char* what, int dtype) {
    return rt_fail(RT_E_DTYPE, "%s: unknown dtype code %d", what, dtype);
}

int32_t fill_any(rt_ctx* ctx, int32_t dtype, void* buf, uint64_t buf_len, const void* value, uint64_t offset, int rank,
                 const uint64_t* shape, const int64_t* strides) {
    RT_TRY(rt_ctx_enter(ctx));
    if (!value) return rt_fail(RT_E_INVALID, "fill: null value");
    const ViewArg va{buf, buf_len, offset, rank, shape, strides, nullptr, 0};
    // a fill moves bits: one instantiation per element width serves every dtype of that width
    switch (rt_elem_size(dtype)) {
        case 1: return run_view<uint8_t, FillF<uint8_t>>(ctx, "fill", va, FillF<uint8_t>{load_scalar<uint8_t>(value)});
        case 2: return run_view<uint16_t, FillF<uint16_t>>(ctx, "fill", va, FillF<uint16_t>{load_scalar<uint16_t>(value)});
        case 4: return run_view<uint32_t, FillF<uint32_t>>(ctx, "fill", va, FillF<uint32_t>{load_scalar<uint32_t>(value)});
        case 8: return run_view<uint64_t, FillF<uint64_t>>(ctx, "fill", va, FillF<uint64_t>{load_scalar<uint64_t>(value)});
        case 16: return run_view<u128_t, FillF<u128_t>>(ctx, "fill", va, FillF<u128_t>{load_scalar<u128_t>(value)});
    }
    return no_dtype("fill", dtype);
}

// Wrapping add / subtract / multiply give the same bits for a signed integer and the unsigned one of its width.
template <class T> struct unsigned_twin { typedef T type; };
template <> struct unsigned_twin<int8_t> { typedef uint8_t type; };
template <> struct unsigned_twin<int16_t> { typedef uint16_t type; };
template <> struct unsigned_twin<int32_t> { typedef uint32_t type; };
template <> struct unsigned_twin<int64_t> { typedef uint64_t type; };
template <> struct unsigned_twin<i128_t> { typedef u128_t type; };

template <class T, int OP>
int32_t unary_go(rt_ctx* ctx, const ViewArg& va) {
    return run_view<T, UnaryF<OP, T>>(ctx, "unary", va, UnaryF<OP, T>{});
}

template <class T>
int32_t unary_float(rt_ctx* ctx, int op, const ViewArg& va) {
#define RT_UCASE(OP) case OP: return unary_go<T, OP>(ctx, va)
    switch (op) {
        RT_UCASE(RT_U_NEG); RT_UCASE(RT_U_RELU); RT_UCASE(RT_U_SIGMOID); RT_UCASE(RT_U_SILU); RT_UCASE(RT_U_TANH); RT_UCASE(RT_U_ABS);
        RT_UCASE(RT_U_SQRT); RT_UCASE(RT_U_LN); RT_UCASE(RT_U_EXPM1); RT_UCASE(RT_U_LN1P); RT_UCASE(RT_U_FLOOR); RT_UCASE(RT_U_CEIL);
        RT_UCASE(RT_U_ROUND); RT_UCASE(RT_U_TRUNC); RT_UCASE(RT_U_SIN); RT_UCASE(RT_U_COS); RT_UCASE(RT_U_TAN); RT_UCASE(RT_U_ASIN);
        RT_UCASE(RT_U_ACOS); RT_UCASE(RT_U_ATAN); RT_UCASE(RT_U_SINH); RT_UCASE(RT_U_COSH); RT_UCASE(RT_U_ASINH); RT_UCASE(RT_U_ACOSH);
        RT_UCASE(RT_U_ATANH); RT_UCASE(RT_U_RSQRT); RT_UCASE(RT_U_RECIPROCAL); RT_UCASE(RT_U_SQUARE); RT_UCASE(RT_U_CUBE);
        RT_UCASE(RT_U_EXP); RT_UCASE(RT_U_SIGN); RT_UCASE(RT_U_STEP); RT_UCASE(RT_U_ABS_GRAD);
    }
#undef RT_UCASE
    return rt_fail(RT_E_INVALID, "unary: unknown op code %d", op);
}

// Non-float dtypes: relu and abs for every dtype, neg for the signed ones (trait bounds, backend/mod.rs:311-355).
template <class T>
int32_t unary_other(rt_ctx* ctx, int op, const ViewArg& va) {
    if (op < 0 || op >= RT_U_EXT_COUNT) return rt_fail(RT_E_INVALID, "unary: unknown op code %d", op);
    if (op == RT_U_RELU) return unary_go<T, RT_U_RELU>(ctx, va);
    if (op == RT_U_STEP) return unary_go<T, RT_U_STEP>(ctx, va);
    if (op == RT_U_ABS) return unary_go<T, RT_U_ABS>(ctx, va);
    if constexpr (is_sint<T>::value) {
        if (op == RT_U_NEG) return unary_go<T, RT_U_NEG>(ctx, va);
        if (op == RT_U_ABS_GRAD) return unary_go<T, RT_U_ABS_GRAD>(ctx, va);
    }
    return rt_fail(RT_E_DTYPE, "unary op %d is not defined for this dtype (the reference bounds it on f32/f64)", op);
}

int32_t unary_any(rt_ctx* ctx, int32_t dtype, int32_t op, const ViewArg& va) {
    RT_TRY(rt_ctx_enter(ctx));
    if (dtype == RT_F32) return unary_float<float>(ctx, op, va);
    if (dtype == RT_F64) return unary_float<double>(ctx, op, va);
    RT_FOR_DTYPE(dtype, return unary_other<T>(ctx, op, va));
    return no_dtype("unary", dtype);
}

template <class T, int OP>
int32_t scalar_go(rt_ctx* ctx, const ViewArg& va, const void* value) {
    int32_t* fault = nullptr;
    if constexpr (OP == RT_S_DIV && is_sint<T>::value) {
        if (load_scalar<T>(value) == (T)-1) {                 // x / -1 overflows for x == MIN: the kernel reports it
            fault = ctx->fault_dev;
            CtxGuard g(ctx);
            ctx->fault_pending = true;
        }
    }
    ScalarF<OP, T> f{load_scalar<T>(value), fault};
    if constexpr (OP == RT_S_DIV && sizeof(T) == 1 && is_int<T>::value) f.magic = div8_magic((int32_t)load_scalar<T>(value));
    if constexpr ((OP == RT_S_LOG || OP == RT_S_LOG1P) && std::is_same<T, double>::value) f.base = LogBase64::of(load_scalar<T>(value));
    return run_view<T, ScalarF<OP, T>>(ctx, "scalar", va, f);
}

template <class T>
int32_t scalar_typed(rt_ctx* ctx, int op, const ViewArg& va, const void* value) {
    switch (op) {
        case RT_S_ADD: return scalar_go<typename unsigned_twin<T>::type, RT_S_ADD>(ctx, va, value);
        case RT_S_SUB: return scalar_go<typename unsigned_twin<T>::type, RT_S_SUB>(ctx, va, value);
        case RT_S_MUL: return scalar_go<typename unsigned_twin<T>::type, RT_S_MUL>(ctx, va, value);
        case RT_S_LEAKY_RELU: return scalar_go<T, RT_S_LEAKY_RELU>(ctx, va, value);
        case RT_S_LEAKY_GRAD: return scalar_go<T, RT_S_LEAKY_GRAD>(ctx, va, value);
        case RT_S_DIV:
            if constexpr (is_bool<T>::value) {
                return rt_fail(RT_E_ARITH, "scalar div: division is not implemented for boolean in the reference (todo!())");
            } else {
                if constexpr (!is_flt<T>::value) {
                    if (load_scalar<T>(value) == (T)0) return rt_fail(RT_E_ARITH, "scalar div: integer division by zero (the reference panics)");
                }
                return scalar_go<T, RT_S_DIV>(ctx, va, value);
            }
        case RT_S_LOG: case RT_S_LOG1P: case RT_S_ELU:
            if constexpr (is_flt<T>::value) {
                if (op == RT_S_LOG) return scalar_go<T, RT_S_LOG>(ctx, va, value);
                if (op == RT_S_LOG1P) return scalar_go<T, RT_S_LOG1P>(ctx, va, value);
                return scalar_go<T, RT_S_ELU>(ctx, va, value);
            } else {
                return rt_fail(RT_E_DTYPE, "scalar op %d is only defined for f32/f64", op);
            }
    }
    return rt_fail(RT_E_INVALID, "scalar: unknown op code %d", op);
}

int32_t scalar_any(rt_ctx* ctx, int32_t dtype, int32_t op, const ViewArg& va, const void* value) {
    RT_TRY(rt_ctx_enter(ctx));
    if (!value) return rt_fail(RT_E_INVALID, "scalar: null value");
    RT_FOR_DTYPE(dtype, return scalar_typed<T>(ctx, op, va, value));
    return no_dtype("scalar", dtype);
}


// ---- fused chain -------------------------------------------------------------------------------------------------------------------
// A short program of elementwise steps applied in registers: acc = in[0][i]; acc = step_k(acc) for every step; dst[i] = acc.  Every
// input is read once and the result written once, whatever the number of steps; each step is the same IEEE / wrapping operation as
// the separate kernel (UnaryF / ScalarF / w_add ...), applied in the same order, so the result is bit for bit that of the sequence of
// backend calls.  The op codes are wave-uniform kernel arguments: the step loop is a handful of scalar branches per vector.
constexpr int kChainUnary = 0, kChainScalar = 1, kChainBinary = 2, kChainBinaryRev = 3;

struct ChainProg {
    int32_t nsteps, ninputs;
    int32_t code[RT_CHAIN_MAX_STEPS];            // kind << 8 | op
    int32_t operand[RT_CHAIN_MAX_STEPS];
    uint64_t value[RT_CHAIN_MAX_STEPS];          // scalar steps: the element's bits (T is at most 8 bytes here)
};
template <class T> struct ChainPtrs { const T* p[RT_CHAIN_MAX_INPUTS]; };

template <class T> __device__ __forceinline__ T chain_value(uint64_t bits) {
    T v;
    __builtin_memcpy(&v, &bits, sizeof(T));
    return v;
}

#define RT_CH(K, OP) ((K) << 8 | (OP))
// one step over N elements held in registers; `y` is the other side of a binary step
template <class T, int N>
__device__ __forceinline__ void chain_apply(T (&a)[N], const T (&y)[N], int code, uint64_t bits) {
    const T v = chain_value<T>(bits);
#define RT_CH_U(OP) case RT_CH(kChainUnary, OP): { _Pragma("unroll") for (int j = 0; j < N; ++j) a[j] = UnaryF<OP, T>{}(a[j]); } break
#define RT_CH_S(OP) case RT_CH(kChainScalar, OP): { const ScalarF<OP, T> f{v, nullptr}; _Pragma("unroll") for (int j = 0; j < N; ++j) a[j] = f(a[j]); } break
    switch (code) {
        RT_CH_U(RT_U_RELU); RT_CH_U(RT_U_ABS); RT_CH_U(RT_U_STEP);
        RT_CH_S(RT_S_ADD); RT_CH_S(RT_S_SUB); RT_CH_S(RT_S_MUL); RT_CH_S(RT_S_LEAKY_RELU); RT_CH_S(RT_S_LEAKY_GRAD);
        case RT_CH(kChainBinary, RT_ADD): { _Pragma("unroll") for (int j = 0; j < N; ++j) a[j] = w_add<T>(a[j], y[j]); } break;
        case RT_CH(kChainBinary, RT_SUB): { _Pragma("unroll") for (int j = 0; j < N; ++j) a[j] = w_sub<T>(a[j], y[j]); } break;
        case RT_CH(kChainBinary, RT_MUL): { _Pragma("unroll") for (int j = 0; j < N; ++j) a[j] = w_mul<T>(a[j], y[j]); } break;
        case RT_CH(kChainBinaryRev, RT_ADD): { _Pragma("unroll") for (int j = 0; j < N; ++j) a[j] = w_add<T>(y[j], a[j]); } break;
        case RT_CH(kChainBinaryRev, RT_SUB): { _Pragma("unroll") for (int j = 0; j < N; ++j) a[j] = w_sub<T>(y[j], a[j]); } break;
        case RT_CH(kChainBinaryRev, RT_MUL): { _Pragma("unroll") for (int j = 0; j < N; ++j) a[j] = w_mul<T>(y[j], a[j]); } break;
        default:
            if constexpr (is_sint<T>::value || is_flt<T>::value) {
                switch (code) {
                    RT_CH_U(RT_U_NEG); RT_CH_U(RT_U_ABS_GRAD);
                    default: break;
                }
            }
            if constexpr (is_flt<T>::value) {
                switch (code) {
                    RT_CH_U(RT_U_SQRT); RT_CH_U(RT_U_FLOOR); RT_CH_U(RT_U_CEIL); RT_CH_U(RT_U_ROUND); RT_CH_U(RT_U_TRUNC); RT_CH_U(RT_U_RSQRT);
                    RT_CH_U(RT_U_RECIPROCAL); RT_CH_U(RT_U_SQUARE); RT_CH_U(RT_U_CUBE); RT_CH_U(RT_U_SIGN);
                    RT_CH_U(RT_U_EXP); RT_CH_U(RT_U_SIGMOID); RT_CH_U(RT_U_SILU); RT_CH_U(RT_U_TANH);
                    RT_CH_S(RT_S_DIV);
                    case RT_CH(kChainBinary, RT_DIV): { _Pragma("unroll") for (int j = 0; j < N; ++j) a[j] = a[j] / y[j]; } break;
                    case RT_CH(kChainBinaryRev, RT_DIV): { _Pragma("unroll") for (int j = 0; j < N; ++j) a[j] = y[j] / a[j]; } break;
                    default: break;
                }
            }
            break;
    }
#undef RT_CH_U
#undef RT_CH_S
}

// the whole program over N elements; fetch(k, y) unpacks the elements of input k
template <class T, int N, class Fetch>
__device__ __forceinline__ void chain_run(T (&acc)[N], const ChainProg& prog, Fetch fetch) {
#pragma unroll 1
    for (int s = 0; s < prog.nsteps; ++s) {
        const int code = prog.code[s];
        T y[N];
        fetch(prog.operand[s], y);
        chain_apply<T, N>(acc, y, code, prog.value[s]);
    }
}

// dst and every input point at the vector body, which starts on a 128-byte line of dst; the inputs may be in any phase.  The `head`
// elements before the body and the `tail` elements after it go to lanes of the first and the last block.
template <class T>
__global__ __launch_bounds__(256) void chain_kernel(ChainPtrs<T> in, T* __restrict__ d, size_t nvec, uint32_t head, uint32_t tail, TileMap m, ChainProg prog) {
    constexpr int N = 16 / sizeof(T);
    const bool at_head = blockIdx.x == 0 && threadIdx.x < head, at_tail = blockIdx.x == gridDim.x - 1 && threadIdx.x < tail;
    if (at_head || at_tail) {
        // one element per lane: before the body (negative index) or after it
        auto one = [&](int64_t e) {
            T x[RT_CHAIN_MAX_INPUTS], acc[1];
#pragma unroll
            for (int k = 0; k < RT_CHAIN_MAX_INPUTS; ++k) x[k] = k < prog.ninputs ? in.p[k][e] : zero_of<T>();
            acc[0] = x[0];
            chain_run<T, 1>(acc, prog, [&](int k, T (&y)[1]) { y[0] = k == 0 ? x[0] : (k == 1 ? x[1] : (k == 2 ? x[2] : x[3])); });
            d[e] = acc[0];
        };
        if (at_head) one((int64_t)threadIdx.x - (int64_t)head);
        if (at_tail) one((int64_t)(nvec * N + threadIdx.x));
    }
    size_t i;
    if (!rt_tile_index(m, blockIdx.x, 256, threadIdx.x, nvec, &i)) return;
    // every input's load is issued before the first use; the vectors stay packed (four 32-bit words) until a step needs their elements
    rt_u32x4 w[RT_CHAIN_MAX_INPUTS];
#pragma unroll
    for (int k = 0; k < RT_CHAIN_MAX_INPUTS; ++k) {
        w[k] = rt_u32x4{0, 0, 0, 0};
        if (k < prog.ninputs) w[k] = rt_ld16u<T, true>(in.p[k] + i * N);
    }
    T acc[N];
    {
        const Vec16<T> v = __builtin_bit_cast(Vec16<T>, w[0]);
#pragma unroll
        for (int j = 0; j < N; ++j) acc[j] = v.e[j];
    }
    chain_run<T, N>(acc, prog, [&](int k, T (&y)[N]) {
        const rt_u32x4 ws = k == 0 ? w[0] : (k == 1 ? w[1] : (k == 2 ? w[2] : w[3]));
        const Vec16<T> v = __builtin_bit_cast(Vec16<T>, ws);
#pragma unroll
        for (int j = 0; j < N; ++j) y[j] = v.e[j];
    });
    Vec16<T> out;
#pragma unroll
    for (int j = 0; j < N; ++j) out.e[j] = acc[j];
    rt_st16_nt(reinterpret_cast<Vec16<T>*>(d) + i, out);
}

// Is (kind, op) a step the chain kernel has for T?  The dtype rules are those of rt_unary_* / rt_scalar_* / rt_broadcast; left out are
// the ops that are ALU-bound on their own (logarithms, trigonometric and hyperbolic inverses ...), integer division (its faults are
// reported per launch) and the 1-byte bool and 16-byte integer types.
template <class T> bool chain_has(int kind, int op) {
    constexpr bool F = is_flt<T>::value, S = is_sint<T>::value;
    if (kind == kChainUnary) {
        switch (op) {
            case RT_U_RELU: case RT_U_ABS: case RT_U_STEP: return true;
            case RT_U_NEG: case RT_U_ABS_GRAD: return F || S;
            case RT_U_SQRT: case RT_U_FLOOR: case RT_U_CEIL: case RT_U_ROUND: case RT_U_TRUNC: case RT_U_RSQRT: case RT_U_RECIPROCAL:
            case RT_U_SQUARE: case RT_U_CUBE: case RT_U_SIGN: case RT_U_EXP: case RT_U_SIGMOID: case RT_U_SILU: case RT_U_TANH: return F;
        }
        return false;
    }
    if (kind == kChainScalar) {
        switch (op) {
            case RT_S_ADD: case RT_S_SUB: case RT_S_MUL: case RT_S_LEAKY_RELU: case RT_S_LEAKY_GRAD: return true;
            case RT_S_DIV: return F;
        }
        return false;
    }
    if (kind == kChainBinary || kind == kChainBinaryRev) return op == RT_ADD || op == RT_SUB || op == RT_MUL || (op == RT_DIV && F);
    return false;
}

template <class T>
int32_t chain_typed(rt_ctx* ctx, int n_inputs, const void* const* inputs, const uint64_t* starts, uint64_t len, int n_steps, const rt_chain_step* steps,
                    void* dst, uint64_t dst_start) {
    constexpr size_t N = 16 / sizeof(T);
    ChainProg prog;
    memset(&prog, 0, sizeof(prog));
    prog.nsteps = n_steps;
    prog.ninputs = n_inputs;
    for (int s = 0; s < n_steps; ++s) {
        const rt_chain_step& st = steps[s];
        if (!chain_has<T>(st.kind, st.op))
            return rt_fail(RT_E_DTYPE, "fused chain: step %d (kind %d, op %d) is not available for this dtype in a chain (issue the separate ops instead)", s, st.kind, st.op);
        const bool bin = st.kind == kChainBinary || st.kind == kChainBinaryRev;
        if (bin && (st.operand < 0 || st.operand >= n_inputs)) return rt_fail(RT_E_INVALID, "fused chain: step %d names input %d of %d", s, st.operand, n_inputs);
        prog.code[s] = RT_CH(st.kind, st.op);
        prog.operand[s] = bin ? st.operand : 0;
        memcpy(&prog.value[s], st.value, sizeof(T));
    }
    T* d = (T*)dst + dst_start;
    ChainPtrs<T> in;
    const uintptr_t addr = reinterpret_cast<uintptr_t>(d);
    size_t head = ((kBodyAlign - (addr & (kBodyAlign - 1))) & (kBodyAlign - 1)) / sizeof(T);
    if (head > len) head = (size_t)len;
    const size_t nvec = ((size_t)len - head) / N, tail = (size_t)len - head - nvec * N;
    for (int k = 0; k < RT_CHAIN_MAX_INPUTS; ++k) in.p[k] = k < n_inputs ? (const T*)inputs[k] + starts[k] + head : nullptr;
    const TileMap m = rt_make_tilemap(d + head, nvec, 256);
    size_t blocks = rt_tilemap_blocks(m, nvec, 256);
    if (blocks < 1) blocks = 1;
    if (blocks > 0x7fffffffull) return rt_fail(RT_E_INVALID, "fused chain: a run of %llu elements is too long for one launch", (unsigned long long)len);
    RT_TRY(rt_check_edges("fused chain", head, nvec, N, tail, (size_t)len, 256));
    CtxGuard g(ctx);
    hipLaunchKernelGGL((chain_kernel<T>), dim3((unsigned)blocks), dim3(256), 0, ctx->stream, in, d + head, nvec, (uint32_t)head, (uint32_t)tail, m, prog);
    RT_HIP(hipGetLastError());
    return RT_OK;
}
#undef RT_CH

}  // namespace

// ---- C ABI ------------------------------------------------------------------------------------------------------------
// The `_contiguous` and `_1d_strided` forms are the N-d form with one dim; all three canonicalise the layout on the
// host (signed strides: a reversed view is walked backwards, it is never mistaken for a forward run).
extern "C" int32_t rt_fill_contiguous(rt_ctx* ctx, int32_t dtype, void* buf, uint64_t buf_len, const void* value, uint64_t start, uint64_t len) {
    const int64_t one = 1;
    return fill_any(ctx, dtype, buf, buf_len, value, start, 1, &len, &one);
}
extern "C" int32_t rt_fill_1d_strided(rt_ctx* ctx, int32_t dtype, void* buf, uint64_t buf_len, const void* value, uint64_t offset,
                                      int64_t stride, uint64_t len) {
    return fill_any(ctx, dtype, buf, buf_len, value, offset, 1, &len, &stride);
}
extern "C" int32_t rt_fill_nd(rt_ctx* ctx, int32_t dtype, void* buf, uint64_t buf_len, const void* value, uint64_t offset, int32_t rank,
                              const uint64_t* shape, const int64_t* strides) {
    return fill_any(ctx, dtype, buf, buf_len, value, offset, rank, shape, strides);
}

extern "C" int32_t rt_unary_contiguous(rt_ctx* ctx, int32_t dtype, int32_t op, void* buf, uint64_t buf_len, uint64_t start, uint64_t len) {
    const int64_t one = 1;
    return unary_any(ctx, dtype, op, ViewArg{buf, buf_len, start, 1, &len, &one, nullptr, 0});
}
extern "C" int32_t rt_unary_1d_strided(rt_ctx* ctx, int32_t dtype, int32_t op, void* buf, uint64_t buf_len, uint64_t offset, int64_t stride,
                                       uint64_t len) {
    return unary_any(ctx, dtype, op, ViewArg{buf, buf_len, offset, 1, &len, &stride, nullptr, 0});
}
extern "C" int32_t rt_unary_nd(rt_ctx* ctx, int32_t dtype, int32_t op, void* buf, uint64_t buf_len, uint64_t offset, int32_t rank,
                               const uint64_t* shape, const int64_t* strides) {
    return unary_any(ctx, dtype, op, ViewArg{buf, buf_len, offset, rank, shape, strides, nullptr, 0});
}

extern "C" int32_t rt_scalar_contiguous(rt_ctx* ctx, int32_t dtype, int32_t op, void* buf, uint64_t buf_len, const void* value,
                                        uint64_t start, uint64_t len) {
    const int64_t one = 1;
    return scalar_any(ctx, dtype, op, ViewArg{buf, buf_len, start, 1, &len, &one, nullptr, 0}, value);
}
extern "C" int32_t rt_scalar_1d_strided(rt_ctx* ctx, int32_t dtype, int32_t op, void* buf, uint64_t buf_len, const void* value,
                                        uint64_t offset, int64_t stride, uint64_t len) {
    return scalar_any(ctx, dtype, op, ViewArg{buf, buf_len, offset, 1, &len, &stride, nullptr, 0}, value);
}
extern "C" int32_t rt_scalar_nd(rt_ctx* ctx, int32_t dtype, int32_t op, void* buf, uint64_t buf_len, const void* value, uint64_t offset,
                                int32_t rank, const uint64_t* shape, const int64_t* strides) {
    return scalar_any(ctx, dtype, op, ViewArg{buf, buf_len, offset, rank, shape, strides, nullptr, 0}, value);
}

// Out-of-place forms: dst[0 .. len) = op(src[start .. start + len)).  The source is only read.
extern "C" int32_t rt_unary_to(rt_ctx* ctx, int32_t dtype, int32_t op, const void* src, uint64_t src_len, uint64_t start, uint64_t len, void* dst,
                               uint64_t dst_len) {
    const int64_t one = 1;
    if (!dst && len) return rt_fail(RT_E_INVALID, "unary: null destination");
    return unary_any(ctx, dtype, op, ViewArg{const_cast<void*>(src), src_len, start, 1, &len, &one, dst, dst_len});
}
extern "C" int32_t rt_scalar_to(rt_ctx* ctx, int32_t dtype, int32_t op, const void* src, uint64_t src_len, const void* value, uint64_t start,
                                uint64_t len, void* dst, uint64_t dst_len) {
    const int64_t one = 1;
    if (!dst && len) return rt_fail(RT_E_INVALID, "scalar: null destination");
    return scalar_any(ctx, dtype, op, ViewArg{const_cast<void*>(src), src_len, start, 1, &len, &one, dst, dst_len}, value);
}

// Fused chain: dst[dst_start + i] = step_{n-1}(... step_0(inputs[0][starts[0] + i]) ...) for i < len.
extern "C" int32_t rt_fused_chain(rt_ctx* ctx, int32_t dtype, int32_t n_inputs, const void* const* inputs, const uint64_t* input_lens,
                                  const uint64_t* input_starts, uint64_t len, int32_t n_steps, const rt_chain_step* steps, void* dst, uint64_t dst_len,
                                  uint64_t dst_start) {
    RT_TRY(rt_ctx_enter(ctx));
    const int es = rt_elem_size(dtype);
    if (!es) return no_dtype("fused chain", dtype);
    if (n_inputs < 1 || n_inputs > RT_CHAIN_MAX_INPUTS) return rt_fail(RT_E_INVALID, "fused chain: %d inputs (1..%d)", n_inputs, RT_CHAIN_MAX_INPUTS);
    if (n_steps < 1 || n_steps > RT_CHAIN_MAX_STEPS) return rt_fail(RT_E_INVALID, "fused chain: %d steps (1..%d)", n_steps, RT_CHAIN_MAX_STEPS);
    if (!inputs || !input_lens || !input_starts || !steps) return rt_fail(RT_E_INVALID, "fused chain: null argument");
    if (dst_start > dst_len || len > dst_len - dst_start)
        return rt_fail(RT_E_OUT_OF_BOUNDS, "fused chain: %llu results from element %llu of a buffer of %llu", (unsigned long long)len, (unsigned long long)dst_start,
                       (unsigned long long)dst_len);
    for (int k = 0; k < n_inputs; ++k)
        if (input_starts[k] > input_lens[k] || len > input_lens[k] - input_starts[k])
            return rt_fail(RT_E_OUT_OF_BOUNDS, "fused chain: input %d is shorter than start + len", k);
    if (dtype == RT_BOOL || es == 16) return rt_fail(RT_E_DTYPE, "fused chain: bool and 128-bit integers are not built (issue the separate ops instead)");
    if (len == 0) return RT_OK;
    if (!dst) return rt_fail(RT_E_INVALID, "fused chain: null destination");
    const ByteSpan ds = rt_run_span(dst, es, dst_start, len);
    for (int k = 0; k < n_inputs; ++k) {
        if (!inputs[k]) return rt_fail(RT_E_INVALID, "fused chain: null input %d", k);
        // the destination may be the very run of an input (every lane reads its elements before it writes them), nothing else
        const bool same = inputs[k] == dst && input_starts[k] == dst_start;
        if (!same && rt_spans_meet(ds, rt_run_span(inputs[k], es, input_starts[k], len)))
            return rt_fail(RT_E_INVALID, "fused chain: the destination overlaps input %d without being the same run", k);
    }
    RT_FOR_DTYPE(dtype, {
        if constexpr (!is_bool<T>::value && sizeof(T) <= 8) return chain_typed<T>(ctx, n_inputs, inputs, input_starts, len, n_steps, steps, dst, dst_start);
    });
    return no_dtype("fused chain", dtype);
}
