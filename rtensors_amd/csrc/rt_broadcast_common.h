// Shared by the broadcast translation units (rt_broadcast.hip: planning, contiguous / row / generic kernels;
// rt_broadcast_tile.hip: the LDS-transpose kernel): element types, the binary op on T, 16-byte vectors, operand access modes.
#pragma once

#include "rt_common.h"
#include "rt_div128.h"

#include <limits>
#include <type_traits>

namespace rtb {

struct boolean_t { uint8_t v; };
template <class T> struct is_flt : std::integral_constant<bool, std::is_same<T, float>::value || std::is_same<T, double>::value> {};
template <class T> struct is_bool : std::is_same<T, boolean_t> {};

typedef unsigned __int128 u128_t;
typedef __int128 i128_t;              // only division tells the two 128-bit types apart; + - * run on u128_t
template <class T> struct is_int128 : std::integral_constant<bool, std::is_same<T, u128_t>::value || std::is_same<T, i128_t>::value> {};
template <class T, class E = void> struct carrier { typedef T type; };
template <> struct carrier<i128_t, void> { typedef u128_t type; };
template <class T> struct carrier<T, typename std::enable_if<std::is_integral<T>::value && sizeof(T) <= 4>::type> { typedef uint32_t type; };
template <class T> struct carrier<T, typename std::enable_if<std::is_integral<T>::value && sizeof(T) == 8>::type> { typedef uint64_t type; };

// ops/base.rs:27-37 on T; integers wrap (release build), integer division truncates toward zero
constexpr int kOpCopy = 4;      // internal: dst = left (strided gather); right is ignored

// `fault`: where integer division reports what the reference answers with a panic (ops/base.rs:27-37: `/` on a zero divisor, and
// MIN / -1, which overflows): the lane stores 1 there -- a plain store, every lane that meets a fault writes the same value -- and
// the host turns a set word into RT_E_ARITH at the next call that waits for the stream.  The element itself becomes 0 (MIN for
// MIN / -1).
template <int OP, class T> __device__ __forceinline__ T bin_apply(T a, T b, int32_t* fault = nullptr) {
    if constexpr (OP == kOpCopy) {
        return a;
    } else if constexpr (is_flt<T>::value) {
        if constexpr (OP == RT_ADD) return a + b;
        else if constexpr (OP == RT_SUB) return a - b;
        else if constexpr (OP == RT_MUL) return a * b;
        else return a / b;
    } else if constexpr (is_bool<T>::value) {
        if constexpr (OP == RT_ADD) return boolean_t{(uint8_t)(a.v | b.v)};            // core/value.rs:708-713 (OR)
        else if constexpr (OP == RT_SUB) return boolean_t{(uint8_t)(a.v ^ b.v)};       // core/value.rs:715-720 (XOR)
        else return boolean_t{(uint8_t)(a.v & b.v)};                                   // core/value.rs:722-727 (AND)
    } else {
        typedef typename carrier<T>::type W;
        if constexpr (OP == RT_ADD) return (T)(W)((W)a + (W)b);
        else if constexpr (OP == RT_SUB) return (T)(W)((W)a - (W)b);
        else if constexpr (OP == RT_MUL) return (T)(W)((W)a * (W)b);
        else if constexpr (is_int128<T>::value) {
            // hand-written long division (rt_div128.h); MIN / -1 wraps to MIN there
            if (b == 0) {
                if (fault) *fault = 1;
                return (T)0;
            }
            if constexpr (std::is_same<T, i128_t>::value) {
                if (b == (T)-1 && a == (T)((u128_t)1 << 127) && fault) *fault = 1;
                return rt_idiv128(a, b);
            } else {
                return rt_udiv128(a, b);
            }
        } else {
            if (b == 0) {
                if (fault) *fault = 1;
                return (T)0;
            }
            if constexpr (std::is_signed<T>::value) {
                if (b == (T)-1) {
                    if (a == std::numeric_limits<T>::min() && fault) *fault = 1;
                    return (T)(W)((W)0 - (W)a);
                }
            }
            if constexpr (sizeof(T) <= 2) return rt_div_narrow<T>(a, b);
            else if constexpr (sizeof(T) == 4) return rt_div32<T>(a, b);
            else return rt_div64<T>(a, b);
        }
    }
}

template <class T> struct alignas(16) Vec16 { T e[16 / sizeof(T)]; };

// x = x OP y on a whole vector.  1-byte add / subtract (and every bool op) run on four elements per 32-bit word.
template <int OP, class T> __device__ __forceinline__ void bin_apply_vec(Vec16<T>& x, const Vec16<T>& y, int32_t* fault = nullptr) {
    if constexpr (sizeof(T) == 1 && (OP == RT_ADD || OP == RT_SUB || (OP == RT_MUL && is_bool<T>::value))) {
        rt_words4 a = __builtin_bit_cast(rt_words4, x);
        const rt_words4 b = __builtin_bit_cast(rt_words4, y);
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            if constexpr (is_bool<T>::value) a.w[j] = OP == RT_ADD ? (a.w[j] | b.w[j]) : (OP == RT_SUB ? (a.w[j] ^ b.w[j]) : (a.w[j] & b.w[j]));
            else a.w[j] = OP == RT_ADD ? rt_add_4x8(a.w[j], b.w[j]) : rt_sub_4x8(a.w[j], b.w[j]);
        }
        x = __builtin_bit_cast(Vec16<T>, a);
    } else if constexpr (OP == RT_DIV && std::is_integral<T>::value && sizeof(T) == 2) {
        // 16-bit division without a branch per element, so that the eight quotients of a vector are computed side by side: a zero
        // divisor is replaced by 1 and its result selected afterwards, the fault word is written once per vector.  (Measured on the
        // config-3 shapes: i16 0.37 -> 0.48 of peak against a branch per element, u16 level; 1-byte and 32-bit elements lose.)
        bool bad = false;
#pragma unroll
        for (int j = 0; j < 8; ++j) {
            const T a = x.e[j], b = y.e[j];
            const bool zero = b == (T)0;
            const int32_t q = rt_div_narrow_wide<T>(a, zero ? (T)1 : b);
            bad |= zero;
            if constexpr (std::is_signed<T>::value) bad |= q > (int32_t)std::numeric_limits<T>::max();      // MIN / -1
            x.e[j] = zero ? (T)0 : (T)q;
        }
        if (bad && fault) *fault = 1;
    } else if constexpr (OP == RT_DIV && std::is_integral<T>::value && sizeof(T) == 4) {
        // 32-bit division, likewise without a branch per element
        bool bad = false;
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const T a = x.e[j], b = y.e[j];
            const bool zero = b == (T)0;
            const double q = rt_div32_real<T>(a, zero ? (T)1 : b);
            bad |= zero;
            if constexpr (std::is_signed<T>::value) {
                const bool ovf = q >= 2147483648.0;                                                        // MIN / -1
                bad |= ovf;
                x.e[j] = zero ? (T)0 : (ovf ? std::numeric_limits<T>::min() : (T)(int32_t)q);
            } else {
                x.e[j] = zero ? (T)0 : (T)(uint32_t)q;
            }
        }
        if (bad && fault) *fault = 1;
    } else {
#pragma unroll
        for (int j = 0; j < (int)(16 / sizeof(T)); ++j) x.e[j] = bin_apply<OP, T>(x.e[j], y.e[j], fault);
    }
}

// ---- division of 1-byte integers through a table of multipliers ---------------------------------------------------------------------
// For 0 <= a < 256 and 1 <= b < 256 the quotient a / b equals (a * M[b]) >> 16 with M[b] = 65536 / b + 1: the product overshoots
// a / b by a * (M[b] - 65536 / b) / 65536 < 256 / 65536, less than the 1 / b that separates a / b from the next integer.  Signed
// bytes use the same multipliers with the divisor's sign on them: p = a * Ms[b] has the sign of the quotient and a magnitude that is
// never a whole multiple of 65536 unless it is 0, so the truncating quotient is (p >> 16) + (p < 0) (all 256 x 255 pairs of either
// type checked against integer arithmetic).  The 256 multipliers live in LDS, one computed per lane when the block starts; per
// element that is a lookup, a 24-bit multiply and a shift, against two conversions, a quarter-rate reciprocal, a multiply and a
// conversion back on the float path -- which stays for the kernels without the table.  M[0] = 0: the quotient of a zero divisor is 0.
template <class T, int OP> struct uses_div8 : std::integral_constant<bool, OP == RT_DIV && sizeof(T) == 1 && std::is_integral<T>::value> {};

template <class T> __device__ __forceinline__ void div8_table_init(int32_t* tbl) {          // 256 lanes; caller synchronises
    const uint32_t byte = threadIdx.x & 255u;
    const int32_t v = std::is_signed<T>::value ? (int32_t)(int8_t)byte : (int32_t)byte;
    const int32_t mag = v < 0 ? -v : v;
    // floor of the correctly rounded f32 quotient: exact, the true quotient is at least 1 / 255 away from the next integer
    const int32_t m = mag ? (int32_t)(65536.0f / (float)mag) + 1 : 0;
    tbl[byte] = v < 0 ? -m : m;
}

template <class T> __device__ __forceinline__ void div8_vec(Vec16<T>& x, const Vec16<T>& y, const int32_t* tbl, int32_t* fault) {
    rt_words4 a = __builtin_bit_cast(rt_words4, x);
    const rt_words4 b = __builtin_bit_cast(rt_words4, y);
    bool bad = false;
#pragma unroll
    for (int w = 0; w < 4; ++w) {
        const uint32_t bw = b.w[w];
        bad |= ((bw - 0x01010101u) & ~bw & 0x80808080u) != 0;                         // a zero byte among the four divisors
        uint32_t out = 0;
#pragma unroll
        for (int k = 0; k < 4; ++k) {
            const int32_t m = tbl[(bw >> (8 * k)) & 0xffu];
            if constexpr (std::is_signed<T>::value) {
                const int32_t av = (int32_t)(int8_t)(a.w[w] >> (8 * k));
                const int32_t p = av * m;
                const int32_t q = (p >> 16) + (int32_t)((uint32_t)p >> 31);
                bad |= q == 128;                                                          // MIN / -1
                out |= ((uint32_t)q & 0xffu) << (8 * k);
            } else {
                const uint32_t av = (a.w[w] >> (8 * k)) & 0xffu;
                out |= ((av * (uint32_t)m) >> 16) << (8 * k);
            }
        }
        a.w[w] = out;
    }
    if (bad && fault) *fault = 1;
    x = __builtin_bit_cast(Vec16<T>, a);
}

// x = x OP y on a whole vector, for the kernels that hold the 1-byte division table (`tbl`: 256 words of LDS, filled by
// div8_table_init, when uses_div8<T, OP>; ignored otherwise)
template <int OP, class T> __device__ __forceinline__ void bin_apply_vec_t(Vec16<T>& x, const Vec16<T>& y, int32_t* fault, const int32_t* tbl) {
    if constexpr (uses_div8<T, OP>::value) div8_vec<T>(x, y, tbl, fault);
    else bin_apply_vec<OP, T>(x, y, fault);
}

// The fault word of the context for a launch that can raise an integer-division fault (and a note for the host to look at it at
// the next synchronising call); null for every other launch.
template <class T, int OP> static inline int32_t* fault_of(rt_ctx* ctx) {
    if constexpr (OP == RT_DIV && (std::is_integral<T>::value || is_int128<T>::value)) {
        ctx->fault_pending = true;
        return ctx->fault_dev;
    } else {
        return nullptr;
    }
}

constexpr int kBlock = 256;     // generic kernels
constexpr int kRBlock = 128;    // contig / rows kernels: small blocks, one 16-byte vector per lane per step

// M_VEC: unit stride along the row (16-byte accesses at element alignment), M_BCAST: stride 0, M_ELEM: any other stride
enum Mode : int { M_VEC = 0, M_BCAST = 1, M_ELEM = 2 };

// One 16-byte vector of an operand's row as four 32-bit words (the form that crosses selects and loops without being split into
// per-element registers), and the same as elements.
template <class T, int MODE>
__device__ __forceinline__ rt_u32x4 load_raw(const T* __restrict__ rowp, uint32_t c, int64_t istride) {
    constexpr int N = 16 / sizeof(T);
    if constexpr (MODE == M_VEC) {
        // Unit stride along the row; the row may start at any element.  Plain (cached) loads: right for operands that are re-read
        // (broadcast along some dim).  Kernels that know an operand is read once load it with rt_ld16u<T, true> themselves -- the
        // choice has to be made at compile time, because two loads that differ only in the hint are merged and the hint is lost.
        return rt_ld16u<T, false>(rowp + c);
    } else {
        Vec16<T> v;
        if constexpr (MODE == M_BCAST) {
            T x = rowp[0];
#pragma unroll
            for (int j = 0; j < N; ++j) v.e[j] = x;
        } else {
#pragma unroll
            for (int j = 0; j < N; ++j) v.e[j] = rowp[(int64_t)(c + j) * istride];
        }
        return __builtin_bit_cast(rt_u32x4, v);
    }
}
template <class T, int MODE>
__device__ __forceinline__ Vec16<T> load_vec(const T* __restrict__ rowp, uint32_t c, int64_t istride) {
    return __builtin_bit_cast(Vec16<T>, load_raw<T, MODE>(rowp, c, istride));
}

static inline bool mult_of(int64_t v, int64_t n) { return v % n == 0; }

// Launches the LDS-transpose kernel when the operation fits it: exactly one input is "transposed" (its inner stride is
// neither 0 nor 1 and it has unit |stride| along another dim) and there is no long stride-0 dim over which the row kernel
// could hoist it.  Returns true when the operation was taken (then *status is its result), false when another kernel
// should run it.  Instantiated in rt_broadcast_tile.hip for every (T, OP) that rt_broadcast.hip uses.
template <class T, int OP>
bool tile_try(rt_ctx* ctx, const NdDesc& dsc, uint64_t count, const T* l, const T* r, T* d, int32_t* status);

// Row-major copy of a view whose second-to-last dim is short (2..64) and unit-stride in the source while the last dim steps
// by exactly that extent: interleaved -> planar, e.g. (H*W, C) pixels into (C, H*W) planes.  Returns true when taken.
// Instantiated in rt_broadcast_tile.hip for the four word sizes the gather uses.
template <class T>
bool planar_copy_try(rt_ctx* ctx, const NdDesc& dsc, uint64_t count, const T* src, T* dst, int32_t* status);

// Row-major copy of a view through N-d tiles in LDS (rt_permute.hip): for views whose contiguous pieces are short in src, in dst or
// in both.  Returns false when the copy is not for it (`force`: take every view the plan can handle, not only those it is the
// fastest kernel for); instantiated for the four word sizes the gather uses.
template <class T>
bool permute_try(rt_ctx* ctx, const NdDesc& dsc, uint64_t count, const T* src, T* dst, int32_t* status, bool force = false);

// dst = xt (op) xo, or xo (op) xt, through the same N-d tiles: xt is the permuted input (dsc.stride[0], dsc.offset[0]); xo and dst
// point at their first elements and are both laid out row-major over dsc.shape (dsc.stride[2]); dst may be xo.  Instantiated for
// float and double with the four ops and for the 32- and 64-bit carriers with + - * (PermBinFused below).
template <class T, int OP>
bool permute_bin_try(rt_ctx* ctx, const NdDesc& dsc, uint64_t count, const T* xt, const T* xo, T* dst, bool tile_is_left, int32_t* status);
template <class T, int OP> struct PermBinFused {
    static constexpr bool value = std::is_same<T, float>::value || std::is_same<T, double>::value ||
                                  ((std::is_same<T, uint32_t>::value || std::is_same<T, uint64_t>::value) && OP != RT_DIV && OP != kOpCopy);
};

}  // namespace rtb
