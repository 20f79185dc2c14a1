// Buffer equality (PartialEq of Backend::Buf) and dtype conversion (Backend::convert).
#include "rt_common.h"

#include <type_traits>
#include <limits>

namespace {

constexpr int kBlock = 256;

__global__ void set_flag_kernel(int32_t* flag, int32_t v) { *flag = v; }

template <class T> struct alignas(16) Vec16 { T e[16 / sizeof(T)]; };
constexpr int kVBlock = 256;    // vector kernels: one 16-byte vector (or one group of vectors) per lane, tiled traversal (see TileMap)

// `==` per element: NaN != NaN, -0.0 == 0.0 (what Box<[T]> == Box<[T]> gives; the reference's device version is
// K/kernels/utils/buffer_equal.cu:7-39).  All lanes that see a mismatch store the same value.  Both buffers are read
// exactly once: one 16-byte vector per lane, non-temporal loads.
template <class T>
__global__ __launch_bounds__(kVBlock) void equal_vec_kernel(const Vec16<T>* __restrict__ a, const Vec16<T>* __restrict__ b, size_t nvec, int32_t* flag,
                                                            TileMap m) {
    constexpr int N = 16 / sizeof(T);
    size_t i;
    if (!rt_tile_index(m, blockIdx.x, kVBlock, threadIdx.x, nvec, &i)) return;
    const Vec16<T> x = rt_ld16_nt(a + i), y = rt_ld16_nt(b + i);
    bool bad = false;
#pragma unroll
    for (int j = 0; j < N; ++j) bad = bad || !(x.e[j] == y.e[j]);
    if (bad) *flag = 0;
}
template <class T>
__global__ __launch_bounds__(kBlock) void equal_kernel(const T* __restrict__ a, const T* __restrict__ b, size_t n, int32_t* flag) {
    size_t i = (size_t)blockIdx.x * kBlock + threadIdx.x;
    const size_t step = (size_t)gridDim.x * kBlock;
    bool bad = false;
    for (; i < n; i += step) bad = bad || !(a[i] == b[i]);
    if (bad) *flag = 0;
}

template <class T>
int32_t equal_typed(rt_ctx* ctx, const void* a, const void* b, size_t n) {
    constexpr size_t N = 16 / sizeof(T);
    const bool aligned = ((reinterpret_cast<uintptr_t>(a) | reinterpret_cast<uintptr_t>(b)) & 15) == 0;
    const size_t nvec = aligned ? n / N : 0;
    if (nvec) {
        const TileMap m = rt_make_tilemap(a, nvec, kVBlock);
        const size_t blocks = rt_tilemap_blocks(m, nvec, kVBlock);
        if (blocks > 0x7fffffffull) return rt_fail(RT_E_INVALID, "rt_equal: %zu elements is too long for one launch", n);
        hipLaunchKernelGGL((equal_vec_kernel<T>), dim3((unsigned)blocks), dim3(kVBlock), 0, ctx->stream, (const Vec16<T>*)a, (const Vec16<T>*)b, nvec,
                           ctx->flag_dev, m);
    }
    const size_t rest = n - nvec * N;
    if (rest) {
        size_t blocks = (rest + kBlock - 1) / kBlock;
        size_t cap = (size_t)ctx->num_cus * 32;
        hipLaunchKernelGGL((equal_kernel<T>), dim3((unsigned)(blocks > cap ? cap : blocks)), dim3(kBlock), 0, ctx->stream,
                           (const T*)a + nvec * N, (const T*)b + nvec * N, rest, ctx->flag_dev);
    }
    RT_HIP(hipGetLastError());
    return RT_OK;
}

// ---- convert: `T::convert::<N>` (core/value.rs:255-462) ---------------------------------------------------------------
// float -> int : round half away from zero, then Rust's saturating `as` (NaN -> 0)
// int   -> int : Rust `as` (truncate / sign-extend)
// any   -> bool: x != 0;   bool -> any: 0 / 1
struct boolean_t { uint8_t v; };
template <class T> struct is_flt : std::integral_constant<bool, std::is_same<T, float>::value || std::is_same<T, double>::value> {};
template <class T> struct is_bool : std::is_same<T, boolean_t> {};

typedef unsigned __int128 u128_t;
typedef __int128 i128_t;
template <class T> struct is_128 : std::integral_constant<bool, std::is_same<T, u128_t>::value || std::is_same<T, i128_t>::value> {};

// u128 -> f32 / f64, correctly rounded (Rust `as`): the 64 leading bits go through the hardware's u64 conversion with the bits
// shifted out folded into the lowest one (it lies far below the rounding position), then an exact power-of-two scaling.  A value
// of 2^128 - 2^103 and above becomes +inf in f32, as in Rust.
template <class F> __device__ __forceinline__ F u128_to_float(u128_t x) {
    const uint64_t hi = (uint64_t)(x >> 64), lo = (uint64_t)x;
    if (hi == 0) return (F)lo;
    const int lz = __builtin_clzll(hi);
    const u128_t v = x << lz;
    uint64_t m = (uint64_t)(v >> 64);
    if ((uint64_t)v != 0) m |= 1;
    if constexpr (std::is_same<F, float>::value) return ldexpf((float)m, 64 - lz);
    else return ldexp((double)m, 64 - lz);
}
// f32 / f64 (already rounded to an integer, finite, 0 <= r < 2^128) -> u128, exact
template <class F> __device__ __forceinline__ u128_t float_to_u128(F r) {
    const F two64 = (F)18446744073709551616.0;
    if (r < two64) return (u128_t)(uint64_t)r;
    const uint64_t hi = (uint64_t)(r / two64);                  // a power-of-two quotient: exact, then truncated
    const uint64_t lo = (uint64_t)(r - (F)hi * two64);
    return ((u128_t)hi << 64) | lo;
}

template <class D, class S> __device__ __forceinline__ D convert_one(S x) {
    if constexpr (is_128<D>::value && is_flt<S>::value) {
        // round half away from zero, then Rust's saturating `as` (NaN -> 0)
        S r = std::is_same<S, float>::value ? (S)roundf((float)x) : (S)round((double)x);
        if (r != r) return (D)0;
        const S two127 = (S)170141183460469231731687303715884105728.0;
        if constexpr (std::is_same<D, u128_t>::value) {
            if (r <= (S)0) return (D)0;
            if (r >= two127 * (S)2) return ~(u128_t)0;          // also +inf (2^128 itself is not finite in f32)
            return float_to_u128<S>(r);
        } else {
            if (r <= -two127) return (i128_t)((u128_t)1 << 127);
            if (r >= two127) return (i128_t)(~(u128_t)0 >> 1);
            return r < (S)0 ? -(i128_t)float_to_u128<S>(-r) : (i128_t)float_to_u128<S>(r);
        }
    } else if constexpr (is_128<S>::value && is_flt<D>::value) {
        if constexpr (std::is_same<S, u128_t>::value) return u128_to_float<D>(x);
        else return x < 0 ? -u128_to_float<D>((u128_t)0 - (u128_t)x) : u128_to_float<D>((u128_t)x);
    } else
    if constexpr (is_bool<D>::value) {
        if constexpr (is_bool<S>::value) return x;
        else return boolean_t{(uint8_t)(x != (S)0)};
    } else if constexpr (is_bool<S>::value) {
        return (D)(x.v ? 1 : 0);
    } else if constexpr (is_flt<S>::value && !is_flt<D>::value) {
        S r = std::is_same<S, float>::value ? (S)roundf((float)x) : (S)round((double)x);
        if (r != r) return (D)0;
        // bounds as doubles/floats: lowest is exact; max+1 is a power of two and exact
        const S lo = (S)std::numeric_limits<D>::lowest();
        const S hi_p1 = (S)2 * (S)((std::numeric_limits<D>::max() >> 1) + 1);
        if (r <= lo) return std::numeric_limits<D>::lowest();
        if (r >= hi_p1) return std::numeric_limits<D>::max();
        return (D)r;
    } else {
        return (D)x;
    }
}

template <class S, class D>
__global__ __launch_bounds__(kBlock) void convert_kernel(const S* __restrict__ s, D* __restrict__ d, size_t n) {
    size_t i = (size_t)blockIdx.x * kBlock + threadIdx.x;
    const size_t step = (size_t)gridDim.x * kBlock;
    for (; i < n; i += step) d[i] = convert_one<D, S>(s[i]);
}

// Non-temporal access of a naturally aligned pack of 1, 2, 4, 8 or 16 bytes.
template <int BYTES> struct pack_word;
template <> struct pack_word<1> { typedef uint8_t type; };
template <> struct pack_word<2> { typedef uint16_t type; };
template <> struct pack_word<4> { typedef uint32_t type; };
template <> struct pack_word<8> { typedef uint64_t type; };
template <> struct pack_word<16> { typedef rt_u32x4 type; };
template <class P> __device__ __forceinline__ P pack_ld_nt(const P* p) {
    typedef typename pack_word<sizeof(P)>::type W;
    return __builtin_bit_cast(P, __builtin_nontemporal_load(reinterpret_cast<const W*>(p)));
}
template <class P> __device__ __forceinline__ void pack_st_nt(P* p, const P& v) {
    typedef typename pack_word<sizeof(P)>::type W;
    __builtin_nontemporal_store(__builtin_bit_cast(W, v), reinterpret_cast<W*>(p));
}

// A lane converts E = 16 / max(sizeof S, sizeof D) elements: one 16-byte vector of the wider type and one 16-, 8-, 4-, 2-
// or 1-byte pack of the narrower one, so that every load and every store instruction of a wave covers one contiguous run.
// (Giving each lane 16 bytes of the narrower type and several vectors of the wider one leaves every wide access
// half-coalesced: f32 -> f64 measured 4.0 TB/s that way against 4.8 TB/s for one element per lane.)
template <class S, class D>
__global__ __launch_bounds__(kVBlock) void convert_vec_kernel(const S* __restrict__ s, D* __restrict__ d, size_t ngroups, TileMap m) {
    constexpr int E = 16 / (sizeof(S) > sizeof(D) ? sizeof(S) : sizeof(D));
    struct alignas(E * sizeof(S)) SP { S e[E]; };
    struct alignas(E * sizeof(D)) DP { D e[E]; };
    size_t i;
    if (!rt_tile_index(m, blockIdx.x, kVBlock, threadIdx.x, ngroups, &i)) return;
    const SP in = pack_ld_nt(reinterpret_cast<const SP*>(s) + i);
    DP out;
#pragma unroll
    for (int k = 0; k < E; ++k) out.e[k] = convert_one<D, S>(in.e[k]);
    pack_st_nt(reinterpret_cast<DP*>(d) + i, out);
}

template <class S, class D>
int32_t convert_go(rt_ctx* ctx, const void* s, void* d, size_t n) {
    constexpr size_t E = 16 / (sizeof(S) > sizeof(D) ? sizeof(S) : sizeof(D));
    const bool aligned = ((reinterpret_cast<uintptr_t>(s) | reinterpret_cast<uintptr_t>(d)) & 15) == 0;
    const size_t ngroups = aligned ? n / E : 0;
    if (ngroups) {
        // the map walks the wider type's 16-byte vectors; the narrower side follows in proportionally smaller pieces
        const TileMap m = rt_make_tilemap(sizeof(S) >= sizeof(D) ? s : (const void*)d, ngroups, kVBlock);
        const size_t blocks = rt_tilemap_blocks(m, ngroups, kVBlock);
        if (blocks > 0x7fffffffull) return rt_fail(RT_E_INVALID, "convert: %zu elements is too long for one launch", n);
        hipLaunchKernelGGL((convert_vec_kernel<S, D>), dim3((unsigned)blocks), dim3(kVBlock), 0, ctx->stream, (const S*)s, (D*)d, ngroups, m);
    }
    const size_t rest = n - ngroups * E;
    if (rest) {
        size_t blocks = (rest + kBlock - 1) / kBlock;
        size_t cap = (size_t)ctx->num_cus * 32;
        hipLaunchKernelGGL((convert_kernel<S, D>), dim3((unsigned)(blocks > cap ? cap : blocks)), dim3(kBlock), 0, ctx->stream,
                           (const S*)s + ngroups * E, (D*)d + ngroups * E, rest);
    }
    RT_HIP(hipGetLastError());
    return RT_OK;
}

#define RT_DST_CASES(S)                                                            \
    switch (dd) {                                                                  \
        case RT_U8: return convert_go<S, uint8_t>(ctx, s, d, n);                   \
        case RT_I8: return convert_go<S, int8_t>(ctx, s, d, n);                    \
        case RT_U16: return convert_go<S, uint16_t>(ctx, s, d, n);                 \
        case RT_I16: return convert_go<S, int16_t>(ctx, s, d, n);                  \
        case RT_U32: return convert_go<S, uint32_t>(ctx, s, d, n);                 \
        case RT_I32: return convert_go<S, int32_t>(ctx, s, d, n);                  \
        case RT_U64: return convert_go<S, uint64_t>(ctx, s, d, n);                 \
        case RT_I64: return convert_go<S, int64_t>(ctx, s, d, n);                  \
        case RT_F32: return convert_go<S, float>(ctx, s, d, n);                    \
        case RT_F64: return convert_go<S, double>(ctx, s, d, n);                   \
        case RT_BOOL: return convert_go<S, boolean_t>(ctx, s, d, n);               \
        case RT_U128: return convert_go<S, u128_t>(ctx, s, d, n);                  \
        case RT_I128: return convert_go<S, i128_t>(ctx, s, d, n);                  \
    }                                                                              \
    break;

int32_t convert_any(rt_ctx* ctx, int sd, const void* s, int dd, void* d, size_t n) {
    switch (sd) {
        case RT_U8: RT_DST_CASES(uint8_t)
        case RT_I8: RT_DST_CASES(int8_t)
        case RT_U16: RT_DST_CASES(uint16_t)
        case RT_I16: RT_DST_CASES(int16_t)
        case RT_U32: RT_DST_CASES(uint32_t)
        case RT_I32: RT_DST_CASES(int32_t)
        case RT_U64: RT_DST_CASES(uint64_t)
        case RT_I64: RT_DST_CASES(int64_t)
        case RT_F32: RT_DST_CASES(float)
        case RT_F64: RT_DST_CASES(double)
        case RT_BOOL: RT_DST_CASES(boolean_t)
        case RT_U128: RT_DST_CASES(u128_t)
        case RT_I128: RT_DST_CASES(i128_t)
    }
    return rt_fail(RT_E_DTYPE, "convert: dtype pair (%d -> %d) is not built for the device", sd, dd);
}

}  // namespace

extern "C" int32_t rt_equal(rt_ctx* ctx, int32_t dtype, const void* a, uint64_t a_len, const void* b, uint64_t b_len, int32_t* out_equal) {
    RT_TRY(rt_ctx_enter(ctx));
    if (!out_equal) return rt_fail(RT_E_INVALID, "rt_equal: null out");
    int es = rt_elem_size(dtype);
    if (!es) return rt_fail(RT_E_DTYPE, "rt_equal: unknown dtype code %d", dtype);
    if (a_len != b_len) { *out_equal = 0; return RT_OK; }
    if (a_len == 0) { *out_equal = 1; return RT_OK; }
    if (!a || !b) return rt_fail(RT_E_INVALID, "rt_equal: null buffer");
    CtxGuard g(ctx);
    hipLaunchKernelGGL(set_flag_kernel, dim3(1), dim3(1), 0, ctx->stream, ctx->flag_dev, 1);
    int32_t rc;
    switch (dtype) {
        // integers and bool: bitwise equality of the element is `==`
        case RT_U8: case RT_I8: case RT_BOOL: rc = equal_typed<uint8_t>(ctx, a, b, a_len); break;
        case RT_U16: case RT_I16: rc = equal_typed<uint16_t>(ctx, a, b, a_len); break;
        case RT_U32: case RT_I32: rc = equal_typed<uint32_t>(ctx, a, b, a_len); break;
        case RT_U64: case RT_I64: rc = equal_typed<uint64_t>(ctx, a, b, a_len); break;
        case RT_U128: case RT_I128: rc = equal_typed<uint64_t>(ctx, a, b, a_len * 2); break;
        case RT_F32: rc = equal_typed<float>(ctx, a, b, a_len); break;
        default: rc = equal_typed<double>(ctx, a, b, a_len); break;
    }
    if (rc != RT_OK) return rc;
    int32_t host = 0;
    RT_HIP(hipMemcpyAsync(&host, ctx->flag_dev, sizeof(host), hipMemcpyDeviceToHost, ctx->stream));
    RT_HIP(hipStreamSynchronize(ctx->stream));
    *out_equal = host;
    return rt_take_fault(ctx);
}

extern "C" int32_t rt_convert(rt_ctx* ctx, int32_t src_dtype, const void* src, uint64_t src_len, int32_t dst_dtype, void* dst, uint64_t dst_len) {
    RT_TRY(rt_ctx_enter(ctx));
    if (!rt_elem_size(src_dtype) || !rt_elem_size(dst_dtype)) return rt_fail(RT_E_DTYPE, "convert: unknown dtype code");
    if (src_len != dst_len)
        return rt_fail(RT_E_SIZE_MISMATCH, "Buffer size mismatch in convert: src size %llu, dst size %llu", (unsigned long long)src_len,
                       (unsigned long long)dst_len);
    if (src_len == 0) return RT_OK;
    if (!src || !dst) return rt_fail(RT_E_INVALID, "convert: null buffer");
    if (rt_spans_meet(rt_run_span(src, rt_elem_size(src_dtype), 0, src_len), rt_run_span(dst, rt_elem_size(dst_dtype), 0, dst_len)))
        return rt_fail(RT_E_INVALID, "convert: the destination overlaps the source");
    CtxGuard g(ctx);
    return convert_any(ctx, src_dtype, src, dst_dtype, dst, (size_t)src_len);
}
