// Internal definitions shared by the translation units of librt_hip.so (gfx950 only).
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>
#include <type_traits>
#include <stdarg.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>

#include <map>
#include <mutex>
#include <vector>

#include "../../include/rt_hip.h"

// ---- error plumbing ---------------------------------------------------------------------------------------------
int32_t rt_fail(int32_t status, const char* fmt, ...) __attribute__((format(printf, 2, 3)));
int32_t rt_hip_fail(hipError_t e, const char* what);

#define RT_HIP(call)                                              \
    do {                                                          \
        hipError_t e__ = (call);                                  \
        if (e__ != hipSuccess) return rt_hip_fail(e__, #call);    \
    } while (0)

#define RT_TRY(call)                                   \
    do {                                               \
        int32_t s__ = (call);                          \
        if (s__ != RT_OK) return s__;                  \
    } while (0)

// ---- context ------------------------------------------------------------------------------------------------------
// One stream per context; every launch and copy is enqueued on it, so a block returned to the free lists by
// rt_free can be handed out again immediately: its next user runs after its previous user in stream order.
struct rt_ctx {
    int device = 0;
    hipStream_t stream = nullptr;
    std::mutex mu;
    // caching allocator: exact-size-class free lists
    std::multimap<size_t, void*> free_blocks;      // capacity -> block
    std::map<void*, size_t> live;                  // block -> capacity
    uint64_t bytes_in_use = 0, bytes_cached = 0, device_allocs = 0;
    // scratch for two-stage reductions (partials), grown on demand, reused across calls
    void* scratch = nullptr;
    size_t scratch_bytes = 0;
    // While `fixed_only` is set (for the duration of one call of the entry point that allocates nothing, under `mu`) rt_scratch hands
    // out `fixed_scratch` (fixed_scratch_bytes long) and refuses anything larger instead of growing `scratch`.
    void* fixed_scratch = nullptr;
    size_t fixed_scratch_bytes = 0;
    bool fixed_only = false;
    void* static_scratch = nullptr;                // this device's copy of the library's built-in workspace (rt_static_scratch_init)
    // pinned staging ring for large host<->device transfers (allocated by the first one), one event per slot
    void* stage[4] = {nullptr, nullptr, nullptr, nullptr};
    hipEvent_t stage_ev[4] = {nullptr, nullptr, nullptr, nullptr};
    // rocBLAS handle bound to `stream` (created by the first f32/f64 matmul) and the function that destroys it
    void* blas = nullptr;
    int (*blas_destroy)(void*) = nullptr;
    // device flag written by the equality kernel and read back by rt_equal
    int32_t* flag_dev = nullptr;
    // device word set by integer-division kernels that met a zero divisor or MIN / -1 (the reference panics there); looked at by
    // the next call that waits for the stream, and only when such a kernel was launched since the last look
    int32_t* fault_dev = nullptr;
    bool fault_pending = false;
    int num_cus = 256;
};

struct CtxGuard {
    rt_ctx* c;
    std::unique_lock<std::mutex> lk;
    explicit CtxGuard(rt_ctx* ctx) : c(ctx), lk(ctx->mu) {}
};

int32_t rt_ctx_enter(rt_ctx* ctx);                                   // validates ctx and makes its device current
int32_t rt_alloc_bytes(rt_ctx* ctx, size_t bytes, void** out);       // caller holds ctx->mu
int32_t rt_free_locked(rt_ctx* ctx, void* p);
int32_t rt_scratch(rt_ctx* ctx, size_t bytes, void** out);           // caller holds ctx->mu; growth counts as a device allocation
// Device address of the built-in workspace of rt_reduce_nd_static on `device`, which must be current (looked up once per device).
int32_t rt_static_scratch_init(int device, void** out);
// After the stream has been waited for: RT_E_ARITH if an integer division launched since the last look met a fault, and the fault
// word is cleared.  Caller holds ctx->mu.
int32_t rt_take_fault(rt_ctx* ctx);

// Validation shared by the reduce and argmax entry points.  *run == false after RT_OK: there are no outputs, launch nothing.
int32_t rt_check_reduce_flat(uint64_t src_len, const void* src, const void* dst, uint64_t dst_len, uint64_t start, uint64_t len);
int32_t rt_check_reduce_nd(uint64_t src_len, const void* src, uint64_t offset, int32_t rank, const uint64_t* shape, const int64_t* strides,
                           const void* dst, uint64_t dst_len, int32_t dim, uint64_t* outer, uint64_t* inner, bool* run);
int32_t rt_reduce_rows(rt_ctx* ctx, int dtype, int op, const void* src, void* out, uint64_t rows, uint64_t R);     // caller holds ctx->mu
int32_t rt_reduce_cols(rt_ctx* ctx, int dtype, int op, const void* src, void* out, uint64_t R, uint64_t inner);
// variance / stdev / logsumexp / norms (out: T*) and argmax / argmin (out: uint64_t*) of src viewed as (outer, R, inner); caller
// holds ctx->mu
int32_t rt_reduce_stat(rt_ctx* ctx, int dtype, int op, const void* src, void* out, uint64_t outer, uint64_t R, uint64_t inner);

static inline int rt_elem_size(int dtype) {
    switch (dtype) {
        case RT_U8: case RT_I8: case RT_BOOL: return 1;
        case RT_U16: case RT_I16: return 2;
        case RT_U32: case RT_I32: case RT_F32: return 4;
        case RT_U64: case RT_I64: case RT_F64: return 8;
        case RT_U128: case RT_I128: return 16;
    }
    return 0;
}

// The contiguous kernels hand the `head` elements before their 16-byte vector body and the `tail` elements after it to lanes of the
// first and the last block, which compare those counts with the lane index.  A count of a block size or more, or pieces that do not
// add up to the run, would make lanes store past the run: checked on the host before every such launch.
inline int32_t rt_check_edges(const char* what, size_t head, size_t nvec, size_t per_vec, size_t tail, size_t n, unsigned block) {
    if (head >= block || tail >= block || tail >= per_vec || nvec > (SIZE_MAX - head - tail) / per_vec || head + nvec * per_vec + tail != n)
        return rt_fail(RT_E_INVALID, "%s: launch geometry does not cover the run (head %zu, %zu vectors of %zu, tail %zu, run %zu, block %u)", what, head, nvec,
                       per_vec, tail, n, block);
    return RT_OK;
}

// ---- descriptor validation and canonicalisation (host) -----------------------------------------------------------
// check_extent of the reference's remote server (backend/remote/server.rs:241-270): lowest and highest addressed
// element must lie inside [0, len).  Returns the element count through *count (0 when any dim is 0).
int32_t rt_check_extent(const char* what, uint64_t offset, int rank, const uint64_t* shape, const int64_t* strides,
                        uint64_t len, uint64_t* count);

// Byte range [lo, hi) that a non-empty, already validated view touches in its buffer.
struct ByteSpan { uintptr_t lo, hi; };
ByteSpan rt_view_span(const void* base, int elem_size, uint64_t offset, int rank, const uint64_t* shape, const int64_t* strides);
inline ByteSpan rt_run_span(const void* base, int elem_size, uint64_t start, uint64_t len) {
    const uintptr_t lo = reinterpret_cast<uintptr_t>(base) + (uintptr_t)start * (uintptr_t)elem_size;
    return ByteSpan{lo, lo + (uintptr_t)len * (uintptr_t)elem_size};
}
inline bool rt_spans_meet(ByteSpan a, ByteSpan b) { return a.lo < b.hi && b.lo < a.hi; }
// The one aliasing an output may have with an input: the very same elements in the same order (what the in-place operators
// pass).  Every lane then reads its elements before it writes them.  Any other overlap makes the result depend on block order.
bool rt_same_view(const void* a, uint64_t a_offset, const int64_t* a_strides, const void* b, uint64_t b_offset, const int64_t* b_strides,
                  int rank, const uint64_t* shape);

// The one-wave-per-row kernels (ew_rows4_kernel, bin_rows4_kernel) put a wave's 64 vectors on the 128-byte line grid of memory: the
// lane's column is moved back by the row's phase, the distance in elements from the line boundary at or below the row's first element,
// so that a wave writes eight whole lines whatever the row's start.  Tiles of 64 vectors a row needs for the largest phase its rows can
// have, and whether rows have ends that do not fill a 16-byte vector.  `first` = address of the view's first element in elements;
// `strides` = the strides of the dims outside the row.
struct RowTiling { uint32_t tiles; bool ragged; };
inline RowTiling rt_row_tiling(uint64_t first, const int64_t* strides, int nstrides, uint32_t L, uint32_t esize) {
    const uint32_t N = 16 / esize, LN = 128 / esize;
    bool line_uniform = true, vec_uniform = true;
    for (int k = 0; k < nstrides; ++k) {
        if (strides[k] % (int64_t)LN != 0) line_uniform = false;
        if (strides[k] % (int64_t)N != 0) vec_uniform = false;
    }
    const uint32_t vphase = (uint32_t)(first % N);
    const uint32_t max_phase = line_uniform ? (uint32_t)(first % LN) : (vec_uniform ? LN - N + vphase : LN - 1);
    RowTiling t;
    t.tiles = (uint32_t)((((uint64_t)L + max_phase + N - 1) / N + 63) / 64);
    t.ragged = !vec_uniform || vphase != 0 || (vphase + L) % N != 0;
    return t;
}

// LDS pitch, in elements, of the rows that the short-row reductions stage in a tile.  Lanes (or lane groups) walk different rows, so
// two rows whose starts are a multiple of 32 words apart meet in one bank.  The row length itself is the pitch -- the tile is then a
// plain copy of the run, written with 16-byte stores -- when that puts at most two rows on a bank (R words with gcd(R, 32) <= 2:
// rows of 10 f32 staged this way instead of element by element: logsumexp 0.65 -> see the measured table), and always for 1- and
// 2-byte elements; other lengths are padded to an odd pitch.
inline uint32_t rt_tile_pitch(uint32_t R, uint32_t esize) {
    if (esize < 4) return R;
    const uint64_t words = (uint64_t)R * (esize / 4);
    uint64_t g = words, h = 32;
    while (h) { const uint64_t t = g % h; g = h; h = t; }
    return g <= 2 ? R : (R | 1u);
}

// Launches whose index arithmetic is 32-bit take fewer than 2^31 elements.  A larger N-d descriptor is cut along its outermost dim into
// slices below that bound (`fn(sub, count_of_sub)` is called for each, in order); when one index of that dim alone is too large the
// dim is dropped and every index becomes a descriptor of its own, to be cut further by the callee.  Returns the first non-zero status.
struct NdDesc;
template <class Fn> int32_t rt_for_slices_below_2g(const NdDesc& d, uint64_t count, Fn fn);

// A view over up to three operands sharing one shape, after removal of size-1 dims and merging of adjacent dims
// that are mergeable in every operand.  Dim 0 is outermost.
struct NdDesc {
    int rank;
    int64_t shape[RT_MAX_RANK];
    int64_t stride[3][RT_MAX_RANK];
    int64_t offset[3];
};

template <class Fn> int32_t rt_for_slices_below_2g(const NdDesc& d, uint64_t count, Fn fn) {
    const uint64_t n0 = (uint64_t)d.shape[0], per = count / n0;
    const bool drop = per >= (1ull << 31);                        // one index alone is too large: a descriptor per index, dim 0 removed
    const uint64_t step = drop ? 1 : ((1ull << 31) - 1) / per;
    for (uint64_t i0 = 0; i0 < n0; i0 += step) {
        const uint64_t take = n0 - i0 < step ? n0 - i0 : step;
        NdDesc sub = d;
        for (int o = 0; o < 3; ++o) sub.offset[o] += (int64_t)i0 * d.stride[o][0];
        if (take == 1) {
            for (int k = 1; k < d.rank; ++k) {
                sub.shape[k - 1] = d.shape[k];
                for (int o = 0; o < 3; ++o) sub.stride[o][k - 1] = d.stride[o][k];
            }
            sub.rank = d.rank - 1;
        } else {
            sub.shape[0] = (int64_t)take;
        }
        const int32_t st = fn(sub, take * per);
        if (st != 0) return st;
    }
    return 0;
}

// Collapses `nops` operands (1..3).  When `reorder` is set (allowed whenever the visiting order of elements is
// irrelevant, i.e. for every elementwise op), dims are first flipped so operand `key`'s strides are non-negative
// and sorted by that operand's stride, largest first, which maximises merging and makes its accesses ascend.
int32_t rt_collapse(int nops, int rank, const uint64_t* shape, const int64_t* const* strides, const uint64_t* offsets,
                    bool reorder, int key, NdDesc* out);

// A collapsed layout of any rank with its descriptor in device memory: words[0 .. rank) = shape, words[(o + 1) * rank + i] = stride
// of operand o along dim i (dim 0 outermost).  Used when more than RT_MAX_RANK dims remain after collapsing.
struct BigDesc {
    int rank;
    const int64_t* words;           // device pointer (the context's scratch buffer; valid until the next call that uses scratch)
    int64_t offset[3];
};
int32_t rt_collapse_big(rt_ctx* ctx, int nops, int rank, const uint64_t* shape, const int64_t* const* strides, const uint64_t* offsets,
                        bool reorder, int key, BigDesc* out);

// ---- device helpers ------------------------------------------------------------------------------------------------
#define RT_WAVE 64

// A dynamic-LDS size that lets four 256-lane blocks share a CU's 160 KiB of LDS (each block also holds a few hundred bytes of
// static LDS).  Passed as the launch's dynamic LDS by long streaming reductions to cap their occupancy; the memory is not used.
constexpr size_t kRtFourBlocksLds = 40000;
constexpr size_t kRtThreeBlocksLds = 54000;      // likewise, three resident blocks

// 16-byte global accesses.  The non-temporal forms mark data that is touched once (streamed operands, outputs):
// measured on MI355X they lift a read-modify-write pass from ~5.5 to ~6.7 TB/s and a read-only pass from ~5.5 to
// ~7.0 TB/s, because streamed lines no longer displace each other in L2 / Infinity Cache.
typedef uint32_t rt_u32x4 __attribute__((ext_vector_type(4)));
template <class V> __device__ __forceinline__ V rt_ld16(const V* p) {
    static_assert(sizeof(V) == 16, "16-byte vector expected");
    return *p;
}
template <class V> __device__ __forceinline__ V rt_ld16_nt(const V* p) {
    static_assert(sizeof(V) == 16, "16-byte vector expected");
    rt_u32x4 r = __builtin_nontemporal_load(reinterpret_cast<const rt_u32x4*>(p));
    return __builtin_bit_cast(V, r);
}
template <class V> __device__ __forceinline__ void rt_st16_nt(V* p, const V& v) {
    static_assert(sizeof(V) == 16, "16-byte vector expected");
    __builtin_nontemporal_store(__builtin_bit_cast(rt_u32x4, v), reinterpret_cast<rt_u32x4*>(p));
}

// 16-byte accesses at element alignment.  The hardware runs in unaligned-access mode: the same global_load / global_store
// dwordx4 serves any address, so a row that starts 4 bytes past a 16-byte boundary (a column slice `m[:, 1:]`, an odd row length)
// still moves one vector per lane; a wave's 1 KiB then touches nine 128-byte lines instead of eight.  The pointee types below
// only tell the compiler not to assume more than the element's own alignment.
typedef uint32_t rt_u32x4_a1 __attribute__((ext_vector_type(4), aligned(1)));
typedef uint32_t rt_u32x4_a2 __attribute__((ext_vector_type(4), aligned(2)));
typedef uint32_t rt_u32x4_a4 __attribute__((ext_vector_type(4), aligned(4)));
template <int ES> struct rt_uvec { typedef rt_u32x4_a4 type; };
template <> struct rt_uvec<1> { typedef rt_u32x4_a1 type; };
template <> struct rt_uvec<2> { typedef rt_u32x4_a2 type; };
// NT is a compile-time choice on purpose (see rt_ld16_dyn for why a plain ternary will not do).
template <class T, bool NT> __device__ __forceinline__ rt_u32x4 rt_ld16u(const T* p) {
    typedef typename rt_uvec<(int)sizeof(T)>::type U;
    const U* q = reinterpret_cast<const U*>(p);
    U r;
    if constexpr (NT) r = __builtin_nontemporal_load(q); else r = *q;
    return rt_u32x4{r.x, r.y, r.z, r.w};
}
template <class T> __device__ __forceinline__ void rt_st16u(T* p, rt_u32x4 v) {
    typedef typename rt_uvec<(int)sizeof(T)>::type U;
    U r = {v.x, v.y, v.z, v.w};
    *reinterpret_cast<U*>(p) = r;
}
template <class T> __device__ __forceinline__ void rt_st16u_nt(T* p, rt_u32x4 v) {
    typedef typename rt_uvec<(int)sizeof(T)>::type U;
    U r = {v.x, v.y, v.z, v.w};
    __builtin_nontemporal_store(r, reinterpret_cast<U*>(p));
}

// Aligned 16-byte load whose non-temporal hint is a wave-uniform run-time flag: two real branches.  The pointer of the
// non-temporal branch passes through an empty asm statement, because written as `nt ? nontemporal_load(q) : *q` the two loads of
// one address can be merged into a single plain load.
template <class V> __device__ __forceinline__ V rt_ld16_dyn(const V* p, bool nt) {
    if (nt) {
        const V* q = p;
        asm volatile("" : "+v"(q));
        return rt_ld16_nt(q);
    }
    return rt_ld16(p);
}

// Truncating division of integers of at most 16 bits through the float unit (the compiler's 32-bit integer expansion is about three
// times as long).  With |a|, |b| < 2^16 the value (|a| + 0.5) / |b| lies at least 0.5 / |b| away from every integer, while
// (|a| + 0.5) * rcp(|b|) is off by less than 0.02 / |b| (the reciprocal to one ulp, the product to half an ulp, of a value below
// 2^16 / |b|): truncating it gives the exact quotient.  Signed operands keep their signs through the float arithmetic (the half is
// given the dividend's sign, the conversion truncates toward zero).  b != 0.  Returns the quotient before narrowing: MIN / -1 is the
// one pair whose quotient does not fit T.
template <class T> __device__ __forceinline__ int32_t rt_div_narrow_wide(T a, T b) {
    static_assert(sizeof(T) <= 2, "operands below 2^16 in magnitude");
    if constexpr (std::is_signed<T>::value) {
        const float fa = (float)(int32_t)a;
        return (int32_t)((fa + __builtin_copysignf(0.5f, fa)) * __builtin_amdgcn_rcpf((float)(int32_t)b));
    } else {
        return (int32_t)(uint32_t)(((float)(uint32_t)a + 0.5f) * __builtin_amdgcn_rcpf((float)(uint32_t)b));
    }
}
template <class T> __device__ __forceinline__ T rt_div_narrow(T a, T b) { return (T)rt_div_narrow_wide<T>(a, b); }

// Truncating division of 32-bit integers through the f64 unit.  r = 1 / b after one Newton step on the hardware reciprocal is good
// to better than 2^-40; (|a| + 0.5) / |b| lies at least 0.5 / |b| away from every integer and (|a| + 0.5) * r is off by less than
// 2^32 / |b| * 2^-40, so truncation gives the exact quotient.  b != 0; rt_div32_real returns the biased quotient before truncation (MIN / -1: 2^31 + 0.5, which does not fit).
template <class T> __device__ __forceinline__ double rt_div32_real(T a, T b) {
    static_assert(sizeof(T) == 4, "32-bit operands");
    const double fb = (double)b;
    double r = __builtin_amdgcn_rcp(fb);
    r = __builtin_fma(__builtin_fma(-fb, r, 1.0), r, r);
    const double fa = (double)a;
    if constexpr (std::is_signed<T>::value) return (fa + __builtin_copysign(0.5, fa)) * r;
    else return (fa + 0.5) * r;
}
template <class T> __device__ __forceinline__ T rt_div32(T a, T b) {
    if constexpr (std::is_signed<T>::value) return (T)(int32_t)rt_div32_real<T>(a, b);
    else return (T)(uint32_t)rt_div32_real<T>(a, b);
}

// Truncating division of 64-bit integers, b != 0 (and not MIN / -1).  Magnitudes that both fit 32 bits -- nearly every 64-bit integer
// tensor in practice: counts, indices, small values -- take the exact f64 path of rt_div32, about 15 operations; anything larger
// takes the compiler's 64-bit expansion (some 80 operation slots with its quarter-rate 32-bit multiplies, ALU-bound at any layout).
// Signed operands divide as magnitudes: the compiler's own signed expansion measured 0.34 of peak on the config-3 shapes where the
// unsigned one reaches 0.84.
__device__ __forceinline__ uint64_t rt_udiv64(uint64_t a, uint64_t b) {
    if (((a | b) >> 32) == 0) return (uint64_t)rt_div32<uint32_t>((uint32_t)a, (uint32_t)b);
    return a / b;
}
template <class T> __device__ __forceinline__ T rt_div64(T a, T b) {
    static_assert(sizeof(T) == 8, "64-bit operands");
    if constexpr (std::is_signed<T>::value) {
        const uint64_t ua = a < 0 ? (uint64_t)0 - (uint64_t)a : (uint64_t)a, ub = b < 0 ? (uint64_t)0 - (uint64_t)b : (uint64_t)b;
        const uint64_t q = rt_udiv64(ua, ub);
        return (T)((a < 0) != (b < 0) ? (uint64_t)0 - q : q);
    } else {
        return (T)rt_udiv64((uint64_t)a, (uint64_t)b);
    }
}

// Four 1-byte integers packed in a 32-bit word, wrapping add / subtract of every byte at once: the low seven bits are
// combined with the top bits masked so that no carry or borrow crosses a byte, then the top bits are restored by xor.
// Per-byte code (sub-dword selects and re-packing) costs about twice the vector instructions per 16-byte vector, enough
// to pull a streaming pass over 1-byte elements from ~6.55 down to ~6.1 TB/s on MI355X.
__device__ __forceinline__ uint32_t rt_add_4x8(uint32_t a, uint32_t b) {
    return ((a & 0x7f7f7f7fu) + (b & 0x7f7f7f7fu)) ^ ((a ^ b) & 0x80808080u);
}
__device__ __forceinline__ uint32_t rt_sub_4x8(uint32_t a, uint32_t b) {
    return ((a | 0x80808080u) - (b & 0x7f7f7f7fu)) ^ ((a ^ ~b) & 0x80808080u);
}
// bytes with the sign bit set -> 0xff, others -> 0x00
__device__ __forceinline__ uint32_t rt_negmask_4x8(uint32_t a) {
    uint32_t s = (a >> 7) & 0x01010101u;
    return (s << 8) - s;
}
struct rt_words4 { uint32_t w[4]; };

// ---- tiled traversal of a contiguous run ------------------------------------------------------------------------------------------
// The streaming kernels give lane i of the grid the i-th 16-byte vector of a run.  Walking the run in that order, a block of 256
// lanes owns one whole 4 KiB page.  Measured on MI355X, the same kernels are 4-6 % faster when a block instead owns the same
// 1 KiB quarter of four neighbouring pages (and the next block the next quarter of those pages): 1 GiB f32, in-place op 0.82 ->
// 0.87 of the 8 TB/s peak, copy 0.81 -> 0.87, c = a + b 0.82 -> 0.86, and a fill with 512-lane blocks owning 1 KiB pieces of
// pages 64 KiB apart 0.84 -> 0.89.  Blocks are dealt to the eight XCDs in turn, so in this order every XCD keeps to its own slice
// of each page instead of all eight sweeping the same address bits together.  The map is a permutation of the vector indices inside
// windows of `rows` pieces at a pitch of `stride` bytes; the vectors before the first 4 KiB boundary and after the last whole window
// keep their plain order.
struct TileMap {
    uint64_t lead;                  // vectors before the first window (plain order)
    uint64_t bulk;                  // vectors inside whole windows
    uint32_t pad;                   // idle lanes at the front of the grid, so that windows start on block boundaries
    uint32_t lp, lr, lc;            // log2 of: vectors per piece, pieces (rows) per block column, pieces per row of the window
};
static inline TileMap rt_make_tilemap(const void* body, size_t nvec, uint32_t nthreads, uint32_t piece_bytes = 1024, uint32_t rows = 4,
                                      uint32_t stride_bytes = 4096) {
    TileMap m;
    const uintptr_t addr = reinterpret_cast<uintptr_t>(body);
    size_t lead = ((4096 - (addr & 4095)) & 4095) / 16;
    if (lead > nvec) lead = nvec;
    const size_t window = (size_t)rows * stride_bytes / 16;
    m.lead = lead;
    m.bulk = (nvec - lead) / window * window;
    m.pad = (uint32_t)((nthreads - lead % nthreads) % nthreads);
    m.lp = (uint32_t)__builtin_ctz(piece_bytes / 16);
    m.lr = (uint32_t)__builtin_ctz(rows);
    m.lc = (uint32_t)__builtin_ctz(stride_bytes / piece_bytes);
    return m;
}
static inline size_t rt_tilemap_blocks(const TileMap& m, size_t nvec, uint32_t nthreads) { return (nvec + m.pad + nthreads - 1) / nthreads; }
// The vector that lane `tid` of block `block` owns; false when the lane has none.  Lane by lane, from the lane's own position: the form
// of the kernels that do a few instructions per element (every lane starts its load after one short chain of vector arithmetic).
__host__ __device__ __forceinline__ bool rt_tile_index(const TileMap& m, uint32_t block, uint32_t nthreads, uint32_t tid, size_t nvec, size_t* out) {
    const int64_t i = (int64_t)block * nthreads + tid - (int64_t)m.pad;
    if (i < 0 || (size_t)i >= nvec) return false;
    size_t j = (size_t)i - m.lead;                      // wraps to a huge value for i < lead
    if (j < m.bulk) {
        const size_t within = j & (((size_t)1 << m.lp) - 1);
        size_t t = j >> m.lp;
        const size_t r = t & (((size_t)1 << m.lr) - 1);
        t >>= m.lr;
        const size_t c = t & (((size_t)1 << m.lc) - 1);
        const size_t w = t >> m.lc;
        j = ((((w << m.lr) + r) << (m.lc + m.lp)) + (c << m.lp)) + within;
    }
    *out = m.lead + j;
    return true;
}
// The same answer with the block's share of the arithmetic kept apart from the lane's.  Windows start on block boundaries (`pad`), so a
// block that lies inside the windows owns whole pieces of one piece column: window, column and first row are the same for all of its
// lanes -- 64-bit arithmetic on the block index, which the compiler keeps on the scalar unit -- and a lane adds its row and its place
// in the piece, two 32-bit operations, instead of walking the whole decomposition in 64-bit vector arithmetic (17 vector instructions
// per vector, a tenth of the vector work of the heavier maps).  Blocks that hold the vectors before the first window or after the
// last one take the lane-by-lane form.  For the kernels whose arithmetic shows: measured on 1 GiB maps, f32 tanh 0.76 -> 0.81 of the
// memory rate, f32 log1p_b 0.71 -> 0.78, f64 asinh 0.70 -> 0.74; the cheap maps lose 2 % with it (the scalar chain delays a wave's first
// load) and keep the lane form.
__host__ __device__ __forceinline__ bool rt_tile_index_block(const TileMap& m, uint32_t block, uint32_t nthreads, uint32_t tid, size_t nvec, size_t* out) {
    const int64_t jb = (int64_t)block * nthreads - (int64_t)m.pad - (int64_t)m.lead;      // position of lane 0 counted from the first window
    const uint32_t pieces = nthreads >> m.lp;                                            // pieces a block owns: consecutive rows of one column
    if (jb >= 0 && (uint64_t)jb + nthreads <= m.bulk && pieces <= (1u << m.lr) && (pieces << m.lp) == nthreads) {
        const uint64_t tb = (uint64_t)jb >> m.lp;                                        // a multiple of `pieces`
        const uint64_t r0 = tb & (((uint64_t)1 << m.lr) - 1);
        const uint64_t c = (tb >> m.lr) & (((uint64_t)1 << m.lc) - 1);
        const uint64_t w = tb >> (m.lr + m.lc);
        const uint64_t base = m.lead + ((((w << m.lr) + r0) << (m.lc + m.lp)) + (c << m.lp));
        const uint32_t lane = ((tid >> m.lp) << (m.lc + m.lp)) + (tid & ((1u << m.lp) - 1));
        *out = base + lane;
        return true;
    }
    return rt_tile_index(m, block, nthreads, tid, nvec, out);
}

// Column reductions: into how many segments to split the rows of `tiles` column tiles (a tile is what one block covers of a row), when
// `want` blocks fill the chip (one or two per CU, by the kernel) and a segment should keep at least a few dozen rows (`by_size` = the
// most segments the row count allows).
// The plain rule: as many segments as keep the blocks within `want`; when that leaves a quarter of the places unused, twice as many.
static inline uint32_t rt_cols_splits_plain(uint64_t tiles, uint64_t want, uint64_t by_size) {
    if (tiles == 0 || tiles >= want) return 1;
    if (by_size < 1) by_size = 1;
    uint64_t sp = want / tiles;
    if (sp > by_size) sp = by_size;
    if (sp < 1) sp = 1;
    if (tiles * sp * 4 < want * 3) {
        const uint64_t by_need = (2 * want + tiles - 1) / tiles;
        sp = by_need < by_size ? by_need : by_size;
    }
    return (uint32_t)(sp > 1024 ? 1024 : sp);
}
// Rows of 64 KiB and more (64 tiles; such rows are never regrouped) meet that rule badly: 129 tiles get one segment and half the CUs,
// 274 tiles 1.07 rounds.  With x = blocks / want, a forced-split sweep (1 GiB f32 sums over axis 0, 98 ... 1024 tiles, 1 ... 16
// segments, rate relative to the best) reads: up to one round the rate grows as 0.2 + 1.05 x and is at its best from x = 0.77; just
// past a whole number of rounds it falls off a cliff (x = 1.008: 0.70, 2.016: 0.77, 3.05: 0.84), because the few CUs with one block
// more finish late, and recovers as the last round fills (1.53: 0.92, 1.84: 0.95, 3.83: 0.95); many rounds cost a little each (smaller
// segments, more partials).  The split with the best estimate is taken; an unsplit launch spares the second stage, which costs the
// statistics (`lean` = false: states instead of values, and more arithmetic per element, so that they also gain from every further
// block up to a full round and take the plain ramp x there) more than the plain reductions.  Against the plain rule, on one machine,
// of peak -- sum, 129 tiles: 0.70 -> 0.82, 157: 0.80 -> 0.85, 274: 0.66 -> 0.83, 586: 0.78 -> 0.83; variance, 98: 0.75 -> 0.85, 129:
// 0.68 -> 0.80, 196: 0.75 -> 0.83; f64 sum over 20000 columns 0.81 -> 0.86.
static inline double rt_cols_launch_rate(uint64_t blocks, uint64_t want, bool lean) {
    const double x = (double)blocks / (double)want;
    if (x <= 1.0) {
        if (!lean) return 0.1 + 0.9 * x;
        const double r = 0.2 + 1.05 * x;
        return (r < 1.0 ? r : 1.0) * (0.9 + 0.1 * x);                // among equals the fuller launch
    }
    const double k = (double)(blocks / want), fr = x - k;
    const double time = k + (fr > 0.0 ? 0.35 + 0.6 * fr : 0.0);
    return 0.95 * x / time * (1.0 - 0.012 * (k - 1.0));
}
static inline uint32_t rt_cols_splits_wide(uint64_t tiles, uint64_t want, uint64_t by_size, bool lean) {
    if (tiles == 0 || want == 0) return 1;
    if (tiles < 64) return rt_cols_splits_plain(tiles, want, by_size);
    if (by_size < 1) by_size = 1;
    uint64_t best = 1;
    double best_score = 0.0;
    uint64_t limit = by_size > 1024 ? 1024 : by_size;
    const uint64_t enough = (8 * want + tiles - 1) / tiles;                      // beyond eight rounds nothing new happens
    if (limit > enough) limit = enough;
    for (uint64_t sp = 1; sp <= limit; ++sp) {
        double score = rt_cols_launch_rate(tiles * sp, want, lean);
        if (sp > 1) score *= lean ? 0.985 : 0.95;
        if (score > best_score * 1.002) { best_score = score; best = sp; }
    }
    return (uint32_t)best;
}

// Column reductions over short rows: how many consecutive rows to read as one (1 = as they are).  The kernels that reduce over rows
// with lanes along the columns (a wave covers 1 KiB of a row, the rows are split over blocks until the launch has about `want`
// blocks) run at 0.72 ... 0.89 of peak on the same 1 GiB depending on how the row length meets that shape; joining g consecutive
// rows into one changes the row length without changing the result (the g partial results per column are folded with the partials
// of the split).  Among the g that divide the row count, leave at least 2048 joined rows and keep the joined row within 128 KiB, the
// one with the best product of what the sweeps showed to matter (f32 sums over axis 0, 1 GiB):
//   how full the launch is under the plain split rule: 1000 columns, g = 20 (79 tiles x 3 segments = 237 blocks) 0.89, g = 24 (94 tiles) 0.74;
//   joined rows that are whole 128-byte lines: 500 columns, g = 8 / 16 / 24 0.87 / 0.87 / 0.88, g = 10 / 20 0.80 / 0.82;
//   how full the last tile of a row is;
//   longer rows, mildly: 2048 columns, g = 1 / 3 / 10 / 16 0.85 / 0.87 / 0.88 / 0.89 (rows of one tile need no help: 256 columns 0.89).
static inline uint64_t rt_cols_regroup(uint64_t rows, uint64_t row_bytes, uint64_t want) {
    if (row_bytes == 0 || row_bytes > 64 * 1024 || want == 0) return 1;
    uint64_t best = 1;
    double best_score = 0.0;
    for (uint64_t g = 1; g * row_bytes <= 128 * 1024; ++g) {
        if (rows % g != 0 || (g > 1 && rows / g < 2048)) continue;
        const uint64_t bytes = g * row_bytes, tiles = (bytes + 1023) / 1024;
        const double lane_fill = (double)bytes / (double)(tiles * 1024);
        const uint64_t blocks = tiles * rt_cols_splits_plain(tiles, want, ~0ull);
        const double launch = (double)blocks / (double)(((blocks + want - 1) / want) * want);
        const double aligned = bytes % 128 == 0 ? 1.0 : 0.92;
        const double length = tiles == 1 ? 1.0 : (bytes < (16u << 10) ? 0.96 : (bytes < (32u << 10) ? 0.98 : (bytes < (64u << 10) ? 0.99 : (bytes < (128u << 10) ? 0.995 : 1.0))));
        const double score = lane_fill * launch * aligned * length;
        if (score > best_score * 1.005) { best_score = score; best = g; }               // a larger g has to earn its extra partials
    }
    return best;
}

// Division of a 32-bit numerator by a runtime-constant divisor via multiply-high (round-up method); exact for
// every n < 2^31 and 1 <= d < 2^31.
struct FastDiv32 {
    uint32_t d, mul, shift;
};
static inline FastDiv32 make_fastdiv(uint32_t d) {
    FastDiv32 f;
    f.d = d;
    if (d == 1) { f.mul = 1; f.shift = 0; return f; }             // (umulhi(n, 1) + n) >> 0 == n: no special case on the device
    uint32_t l = 32 - __builtin_clz(d - 1);                       // ceil(log2 d)
    uint64_t m = (((uint64_t)1 << 32) * (((uint64_t)1 << l) - d)) / d + 1;
    f.mul = (uint32_t)m;
    f.shift = l;
    return f;
}
__device__ __forceinline__ uint32_t fd_div(uint32_t n, const FastDiv32& f) {
    uint32_t t = __umulhi(n, f.mul);
    return (uint32_t)(((uint64_t)t + n) >> f.shift);
}

// Keeps a wave-uniform value that came from the kernel arguments in a scalar register from this point on.  Kernel arguments are
// fetched with scalar loads where they are first used; a kernel that uses them one after another behind branches waits for scalar
// memory once per use.  Pinning everything a short-lived wave needs at the top of the kernel makes all those loads one batch with
// one wait.  (A wave of the one-vector-per-lane kernels has about a microsecond to live if the chip is to stay at full bandwidth.)
#define RT_PIN(x) asm volatile("" : "+s"(x))
// The same for pointers: as an input only, so that the compiler still knows they point to global memory (a pointer that comes out
// of an asm statement is accessed with the slower flat instructions).
#define RT_TOUCH(x) asm volatile("" : : "s"(x))

// blockIdx remainder -> element offsets of NOPS operands over the outer dims of a launch (outermost first, the entries from
// `nouter` on hold shape 1).  Branch-free over a fixed number of dims: written as a loop that tests `k < nouter`, every dim costs
// a chain of dependent scalar loads of the kernel arguments (load the shape, wait, branch, load the divisor, wait, ...), some thirty
// waits before a wave issues its first global load.  Launches with at most two outer dims, nearly all of them, take the short form.
template <int NOPS>
__device__ __forceinline__ void rt_outer_offsets(uint32_t rem, int nouter, const uint32_t (&oshape)[RT_MAX_RANK], const FastDiv32 (&odiv)[RT_MAX_RANK],
                                                 const int64_t (&ostride)[NOPS][RT_MAX_RANK], int64_t (&off)[NOPS]) {
#pragma unroll
    for (int o = 0; o < NOPS; ++o) off[o] = 0;
    if (nouter <= 2) {
#pragma unroll
        for (int k = 1; k >= 0; --k) {
            const uint32_t q = fd_div(rem, odiv[k]);
            const uint32_t c = rem - q * oshape[k];
#pragma unroll
            for (int o = 0; o < NOPS; ++o) off[o] += (int64_t)c * ostride[o][k];
            rem = q;
        }
    } else {
#pragma unroll
        for (int k = RT_MAX_RANK - 1; k >= 0; --k) {
            const uint32_t q = fd_div(rem, odiv[k]);
            const uint32_t c = rem - q * oshape[k];
#pragma unroll
            for (int o = 0; o < NOPS; ++o) off[o] += (int64_t)c * ostride[o][k];
            rem = q;
        }
    }
}
