// Reductions whose running state is more than one value of T: variance / standard deviation, logsumexp, L1 / L2 norm, argmax /
// argmin, full (flat) and along one axis of a row-major contiguous tensor viewed as (outer, R, inner).  The reference offers them
// on its Cuda backend only (K/kernels/reduction/reduce.cu: Welford states 167-213 and 324-460, logsumexp 641-735, norms 66-97 and
// 291-321, argmax 843-990); its Cpu backend panics or has todo!() for them (ops/reduction/mod.rs:185, backend/cpu.rs:451-471).
//
// Every kernel is written once over a state type S with init / push / push_block / merge / result:
//   MomentState   (mean, m2, n)   blocks of 8-16 elements are folded exactly (mean of the block, squared deviations from it) and
//                                 merged into the running state with Chan's update -- the reference's welford_combine; one
//                                 division per block instead of one per element
//   LseState      (max, sum)      sum of exp(x - max), rescaled when the maximum moves; one exp per element plus one per block
//   NormState     (sum)           sum |x| or sum x^2
//   ArgState      (value, index)  strict comparison against T::MIN / T::MAX, smallest index among equals
// Kernels (HBM-bound, algorithmic traffic N_in * sizeof(T) + N_out * sizeof(out)):
//   rows  (inner == 1): block per row segment / wave per row / LDS-staged short rows, as in rt_reduce.hip
//   cols  (inner  > 1): lanes along `inner` with 16-byte loads; a narrow `inner` is streamed as one contiguous run instead
//   Partial states of split reductions go to the context's scratch buffer and a merge kernel folds them (two launches, no atomics).
#include "rt_common.h"
#include "rt_math64.h"

#include <limits>
#include <type_traits>

namespace {

constexpr int kBlock = 256;
constexpr int kWaves = kBlock / RT_WAVE;

template <class T> struct is_flt : std::integral_constant<bool, std::is_same<T, float>::value || std::is_same<T, double>::value> {};
template <class T> struct alignas(16) Vec16 { T e[16 / sizeof(T)]; };

__device__ __forceinline__ float m_exp(float x) { return expf(x); }
__device__ __forceinline__ double m_exp(double x) { return exp(x); }
__device__ __forceinline__ float m_log(float x) { return logf(x); }
__device__ __forceinline__ double m_log(double x) { return log(x); }
__device__ __forceinline__ float m_sqrt(float x) { return sqrtf(x); }
__device__ __forceinline__ double m_sqrt(double x) { return sqrt(x); }
__device__ __forceinline__ float m_abs(float x) { return fabsf(x); }
__device__ __forceinline__ double m_abs(double x) { return fabs(x); }
__device__ __forceinline__ float m_max(float a, float b) { return fmaxf(a, b); }
__device__ __forceinline__ double m_max(double a, double b) { return fmax(a, b); }

// ---- states -----------------------------------------------------------------------------------------------------------
// push(x, pos): one element at position `pos` of the reduced axis; push_block<K>(x, pos0, step): K elements at positions pos0,
// pos0 + step, ...; merge(o): another partial state, any relative order; result(flags): the output value.

// 1 / x for a weight: the hardware reciprocal (1 ulp) is enough for f32, where a correctly rounded division costs ~10 instructions
__device__ __forceinline__ float m_recip(float x) { return __builtin_amdgcn_rcpf(x); }
__device__ __forceinline__ double m_recip(double x) { return 1.0 / x; }

template <class T> struct MomentState {
    typedef T Out;
    // column kernel: resident blocks per CU and loads in flight per lane.  1 GiB f32 over axis 0: 0.90 of peak with one fat block and
    // eight loads (the plain column sum's shape), 0.86 with two blocks and four loads, 0.80 with four blocks
    static constexpr int kColsBlocksPerCU = 1;
    static constexpr int kColsLoads = 8;
    static constexpr int kNarrowBlocksPerCU = 2;   // narrow-column kernel: resident blocks per CU (1 GiB over 3 and 100 columns: 0.85 .. 0.88 of peak with 2, 0.79 .. 0.81 with 4)
    T mean, m2;
    double n;                                                   // a count, exact up to 2^53; as a double it converts to T in one instruction
    __device__ __forceinline__ void init() { mean = (T)0; m2 = (T)0; n = 0.0; }
    // welford_combine, reduce.cu:191-213.  An empty receiver needs no special case: delta = omean, w = 1, n * w = 0.
    __device__ __forceinline__ void absorb(T omean, T om2, double on) {
        if (on == 0.0) return;
        const double nn = n + on;
        const T delta = omean - mean;
        const T w = (T)on * m_recip((T)nn);
        mean = mean + delta * w;
        m2 = m2 + om2 + (delta * delta) * ((T)n * w);
        n = nn;
    }
    __device__ __forceinline__ void push(T x, uint64_t) { absorb(x, (T)0, 1.0); }
    template <int K> __device__ __forceinline__ void push_block(const T* x, uint64_t, uint64_t) {
        T s = (T)0;
#pragma unroll
        for (int i = 0; i < K; ++i) s = s + x[i];
        const T bm = s * ((T)1 / (T)K);                                              // K is a power of two: exact scaling
        T q = (T)0;
#pragma unroll
        for (int i = 0; i < K; ++i) { const T d = x[i] - bm; q = q + d * d; }
        absorb(bm, q, (double)K);
    }
    __device__ __forceinline__ void merge(const MomentState& o) { absorb(o.mean, o.m2, o.n); }
    __device__ __forceinline__ T result(int flags) const {                          // finalize_var_kernel_ptr, reduce.cu:385-402
        const T denom = (flags & RT_R_FLAG_UNBIASED) ? (T)(n - 1.0) : (T)n;
        const T v = m2 / denom;
        return (flags & RT_R_FLAG_STD) ? m_sqrt(v) : v;
    }
};

template <class T> struct LseState {
    typedef T Out;
    // one exp per element: two blocks of four loads (0.87 of peak; one fat block 0.78, four blocks 0.82)
    static constexpr int kColsBlocksPerCU = 2;
    static constexpr int kColsLoads = 4;
    static constexpr int kNarrowBlocksPerCU = 2;
    T m, s;
    __device__ __forceinline__ void init() { m = -std::numeric_limits<T>::infinity(); s = (T)0; }
    // exp(x - top), with x == top giving 1 also when both are infinite.  The argument is never positive, so for f32 the hardware
    // exponential (2^(x log2 e), a few ulp for the arguments near 0 that carry the sum) stays inside the 1e-5 of the result; the
    // library routine costs about four times the instructions and made short-row logsumexp compute-bound.
    // f64: the exponential written for non-positive arguments (rt_math64.h, within 1.5 ulp, half the library routine's instructions),
    // computed for every lane in straight-line code.  It has no case for x == top: a finite x == top gives exp(0) = 1 exactly, and
    // under an infinite top the sum does not reach the result (result() returns m = +-inf for s = 0 and for s > 0 alike).  It turns
    // a NaN argument into 0, so NaN elements are noted apart and make the sum NaN, which every later step keeps.
    static __device__ __forceinline__ T term(T x, T top) {
        if constexpr (std::is_same<T, float>::value) return x == top ? 1.0f : __expf(x - top);
        else return rt_exp_nonpos_f64(x - top);
    }
    static constexpr bool kNoteNan = !std::is_same<T, float>::value;
    __device__ __forceinline__ void push(T x, uint64_t) {
        const T top = m_max(m, x);
        s = s * term(m, top) + term(x, top);
        if constexpr (kNoteNan) s = x != x ? x : s;
        m = top;
    }
    template <int K> __device__ __forceinline__ void push_block(const T* x, uint64_t, uint64_t) {
        T top = m;
#pragma unroll
        for (int i = 0; i < K; ++i) top = m_max(top, x[i]);
        T acc = s * term(m, top);
        bool bad = false;
#pragma unroll
        for (int i = 0; i < K; ++i) {
            acc = acc + term(x[i], top);
            if constexpr (kNoteNan) bad |= x[i] != x[i];
        }
        if constexpr (kNoteNan) acc = bad ? std::numeric_limits<T>::quiet_NaN() : acc;
        s = acc;
        m = top;
    }
    __device__ __forceinline__ void merge(const LseState& o) {                      // lse_combine, reduce.cu:660-673
        const T top = m_max(m, o.m);
        s = s * term(m, top) + o.s * term(o.m, top);
        m = top;
    }
    __device__ __forceinline__ T result(int) const { return s == (T)0 ? m : m + m_log(s); }
    // a whole row by one lane: the maximum first, then one exponential per element (the running form above pays one more per block
    // of four for rescaling the sum: 14 instead of 10 on rows of 10)
    __device__ __forceinline__ void fold_row(const T* row, uint32_t R) {
        T top = row[0];
        for (uint32_t k = 1; k < R; ++k) top = m_max(top, row[k]);
        T acc = (T)0;
        bool bad = false;
        for (uint32_t k = 0; k < R; ++k) {
            acc = acc + term(row[k], top);
            if constexpr (kNoteNan) bad |= row[k] != row[k];
        }
        if constexpr (kNoteNan) acc = bad ? std::numeric_limits<T>::quiet_NaN() : acc;
        m = top;
        s = acc;
    }
};

template <class T, bool SQ> struct NormState {
    typedef T Out;
    static constexpr int kColsBlocksPerCU = 1;                  // as MomentState
    static constexpr int kColsLoads = 8;
    static constexpr int kNarrowBlocksPerCU = 2;
    T s;
    __device__ __forceinline__ void init() { s = (T)0; }
    __device__ __forceinline__ void push(T x, uint64_t) { s = s + (SQ ? x * x : m_abs(x)); }
    template <int K> __device__ __forceinline__ void push_block(const T* x, uint64_t, uint64_t) {
        T b = (T)0;
#pragma unroll
        for (int i = 0; i < K; ++i) b = b + (SQ ? x[i] * x[i] : m_abs(x[i]));
        s = s + b;
    }
    __device__ __forceinline__ void merge(const NormState& o) { s = s + o.s; }
    __device__ __forceinline__ T result(int) const { return SQ ? m_sqrt(s) : s; }
};

template <class T, bool MAX> struct ArgState {
    typedef uint64_t Out;
    static constexpr int kColsBlocksPerCU = 2;                  // 0.85 of peak; one fat block 0.76, four blocks 0.80
    static constexpr int kColsLoads = 4;
    static constexpr int kNarrowBlocksPerCU = 3;   // narrow columns: 0.80 with 3 or 4, 0.71 with 2
    T v;
    uint64_t idx;
    __device__ __forceinline__ void init() {
        v = MAX ? std::numeric_limits<T>::lowest() : std::numeric_limits<T>::max();
        idx = ~0ull;
    }
    static __device__ __forceinline__ bool beats(T a, T b) { return MAX ? a > b : a < b; }
    __device__ __forceinline__ void push(T x, uint64_t pos) {
        if (beats(x, v)) { v = x; idx = pos; }                                      // NaN never wins, the first of equals stays
    }
    template <int K> __device__ __forceinline__ void push_block(const T* x, uint64_t pos0, uint64_t step) {
#pragma unroll
        for (int i = 0; i < K; ++i) push(x[i], pos0 + (uint64_t)i * step);
    }
    __device__ __forceinline__ void merge(const ArgState& o) {
        if (beats(o.v, v) || (o.v == v && o.idx < idx)) { v = o.v; idx = o.idx; }
    }
    __device__ __forceinline__ uint64_t result(int) const { return idx == ~0ull ? 0 : idx; }
};

// a state moved between lanes as 32-bit words
template <class S> struct is_arg_state : std::false_type {};
template <class T, bool MAX> struct is_arg_state<ArgState<T, MAX>> : std::true_type {};

template <class S> __device__ __forceinline__ S shfl_down_state(const S& s, int d) {
    static_assert(sizeof(S) % 4 == 0, "state is a whole number of words");
    constexpr int W = sizeof(S) / 4;
    uint32_t w[W];
    __builtin_memcpy(w, &s, sizeof(S));                                             // states may hold padding: no bit_cast
#pragma unroll
    for (int i = 0; i < W; ++i) w[i] = (uint32_t)__shfl_down((int)w[i], d, RT_WAVE);
    S r;
    __builtin_memcpy(&r, w, sizeof(S));
    return r;
}

// lanes [0, width) of each aligned group of `width` lanes fold into the group's first lane (width: power of two <= 64)
template <class S> __device__ __forceinline__ void group_reduce(S& a, uint32_t width, uint32_t lane_in_group) {
    for (uint32_t d = width / 2; d >= 1; d >>= 1) {
        S o = shfl_down_state(a, (int)d);
        if (lane_in_group + d < width) a.merge(o);
    }
}

// ---- sums and maxima over a group of lanes without the LDS crossbar -----------------------------------------------------------------
// A group is an aligned run of `width` lanes, width a power of two <= 64, all lanes of the wave active.  Inside a row of 16 lanes the
// data-parallel-primitive lane patterns move the operand as part of an ordinary vector instruction: swap neighbours, swap pairs (after
// which the four lanes of a quad agree), mirror the halves of 8, mirror the row.  Across rows the four row results are read into scalar
// registers.  Every lane ends with the group's result.  (The permute instruction these replace goes through the LDS unit, about a
// hundred cycles a step, six steps per value: variance over rows of 512 f32 spent a sixth of its time there.)
template <int CTRL> __device__ __forceinline__ float dpp_get(float v) {
    const int w = __builtin_bit_cast(int, v);
    return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(w, w, CTRL, 0xf, 0xf, false));
}
template <int CTRL> __device__ __forceinline__ double dpp_get(double v) {
    const uint64_t w = __builtin_bit_cast(uint64_t, v);
    const int lo = (int)(uint32_t)w, hi = (int)(uint32_t)(w >> 32);
    const uint32_t l2 = (uint32_t)__builtin_amdgcn_update_dpp(lo, lo, CTRL, 0xf, 0xf, false);
    const uint32_t h2 = (uint32_t)__builtin_amdgcn_update_dpp(hi, hi, CTRL, 0xf, 0xf, false);
    return __builtin_bit_cast(double, (uint64_t)l2 | ((uint64_t)h2 << 32));
}
__device__ __forceinline__ float lane_get(float v, int lane) { return __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, v), lane)); }
__device__ __forceinline__ double lane_get(double v, int lane) {
    const uint64_t w = __builtin_bit_cast(uint64_t, v);
    const uint32_t lo = (uint32_t)__builtin_amdgcn_readlane((int)(uint32_t)w, lane), hi = (uint32_t)__builtin_amdgcn_readlane((int)(uint32_t)(w >> 32), lane);
    return __builtin_bit_cast(double, (uint64_t)lo | ((uint64_t)hi << 32));
}
struct OpSum { template <class T> static __device__ __forceinline__ T f(T a, T b) { return a + b; } };
struct OpMax { template <class T> static __device__ __forceinline__ T f(T a, T b) { return m_max(a, b); } };
template <class Op, class T> __device__ __forceinline__ T group_all(T v, uint32_t width) {
    if (width >= 2) v = Op::f(v, dpp_get<0xB1>(v));              // quad_perm [1, 0, 3, 2]
    if (width >= 4) v = Op::f(v, dpp_get<0x4E>(v));              // quad_perm [2, 3, 0, 1]
    if (width >= 8) v = Op::f(v, dpp_get<0x141>(v));             // row_half_mirror
    if (width >= 16) v = Op::f(v, dpp_get<0x140>(v));            // row_mirror
    if (width >= 32) {
        const T lo = Op::f(lane_get(v, 0), lane_get(v, 16)), hi = Op::f(lane_get(v, 32), lane_get(v, 48));
        if (width >= 64) v = Op::f(lo, hi);
        else v = (threadIdx.x & 32) ? hi : lo;
    }
    return v;
}

// Norms: one sum.
template <class T, bool SQ> __device__ __forceinline__ void group_reduce(NormState<T, SQ>& a, uint32_t width, uint32_t) {
    if (width == 1) return;
    a.s = group_all<OpSum>(a.s, width);
}
// The two states whose merge is expensive (two exponentials; a reciprocal), in phases that need one of those per lane instead of one
// or two per step.  logsumexp: the group's maximum, every lane's sum rescaled to it once, the sums added.
template <class T> __device__ __forceinline__ void group_reduce(LseState<T>& a, uint32_t width, uint32_t) {
    if (width == 1) return;
    const T top = group_all<OpMax>(a.m, width);
    a.s = group_all<OpSum>(a.s * LseState<T>::term(a.m, top), width);       // an empty lane (m = -inf, s = 0) contributes 0
    a.m = top;
}
// moments: with d_i = mean_i - c the distances from a common reference (the largest of the lanes' means), the group's mean is c + D,
// D = sum(n_i d_i) / sum(n_i), and its m2 = sum(m2_i + n_i (d_i - D)^2): sums and one reciprocal.  The distances are differences
// of nearby values, so nothing is lost to the size of the mean itself.
template <class T> __device__ __forceinline__ void group_reduce(MomentState<T>& a, uint32_t width, uint32_t) {
    if (width == 1) return;
    const T ninf = -std::numeric_limits<T>::infinity();
    T c = group_all<OpMax>(a.n > 0.0 ? a.mean : ninf, width);
    c = c == ninf ? (T)0 : c;                                       // no lane holds anything (or nothing but NaN)
    const T d = a.n > 0.0 ? a.mean - c : (T)0;
    const T cnt = (T)a.n;                                           // a lane's own count is small enough to be exact in T
    const double n = group_all<OpSum>(a.n, width);
    const T w = group_all<OpSum>(cnt * d, width);
    const T D = n > 0.0 ? w * m_recip((T)n) : (T)0;
    const T e = d - D;
    a.m2 = group_all<OpSum>(a.m2 + cnt * (e * e), width);
    a.mean = c + D;
    a.n = n;
}

template <class S> __device__ __forceinline__ void block_reduce(S& a) {
    __shared__ S part[kWaves];
    const uint32_t lane = threadIdx.x & (RT_WAVE - 1), w = threadIdx.x / RT_WAVE;
    group_reduce(a, RT_WAVE, lane);
    if (lane == 0) part[w] = a;
    __syncthreads();
    if (threadIdx.x == 0) {
#pragma unroll
        for (int k = 1; k < kWaves; ++k) a.merge(part[k]);
    }
}

// fold elements [begin, end) of the contiguous run `p`; positions are relative to `p`
template <class S, class T, int U = 4>
__device__ __forceinline__ void fold_run(S& a, const T* __restrict__ p, uint64_t begin, uint64_t end, uint32_t tid, uint32_t nthreads) {
    constexpr uint32_t N = 16 / sizeof(T);
    if (begin >= end) return;
    uint64_t head = ((16 - (reinterpret_cast<uintptr_t>(p + begin) & 15)) & 15) / sizeof(T);
    if (head > end - begin) head = end - begin;
    if (tid < head) a.push(p[begin + tid], begin + tid);
    const uint64_t vb = begin + head;
    const uint64_t nvec = (end - vb) / N;
    const Vec16<T>* pv = reinterpret_cast<const Vec16<T>*>(p + vb);
    uint64_t i = tid;
    for (; i + (uint64_t)(U - 1) * nthreads < nvec; i += (uint64_t)U * nthreads) {
        Vec16<T> v[U];
#pragma unroll
        for (int u = 0; u < U; ++u) v[u] = rt_ld16_nt(pv + i + (uint64_t)u * nthreads);
        if constexpr (std::is_same<typename S::Out, uint64_t>::value) {
#pragma unroll
            for (int u = 0; u < U; ++u) a.template push_block<N>(v[u].e, vb + (i + (uint64_t)u * nthreads) * N, 1);
        } else {
            T x[U * N];                                                             // positions are irrelevant: one block of U * N
#pragma unroll
            for (int u = 0; u < U; ++u) {
#pragma unroll
                for (uint32_t j = 0; j < N; ++j) x[u * N + j] = v[u].e[j];
            }
            a.template push_block<U * N>(x, 0, 0);
        }
    }
    if (i < nvec) {                                             // the last 1 .. U-1 vectors of this lane, loads first
        Vec16<T> v[U - 1];
#pragma unroll
        for (int u = 0; u < U - 1; ++u)
            if (i + (uint64_t)u * nthreads < nvec) v[u] = rt_ld16_nt(pv + i + (uint64_t)u * nthreads);
#pragma unroll
        for (int u = 0; u < U - 1; ++u)
            if (i + (uint64_t)u * nthreads < nvec) a.template push_block<N>(v[u].e, vb + (i + (uint64_t)u * nthreads) * N, 1);
    }
    const uint64_t tb = vb + nvec * N;
    if (tb + tid < end) a.push(p[tb + tid], tb + tid);
}

// ---- rows -------------------------------------------------------------------------------------------------------------
// grid.x = rows * splits; block b folds segment (b % splits) of row (b / splits) -> part[b] (state) or out[row] (result)
template <class S, class T, int U = 4>
__global__ __launch_bounds__(kBlock) void st_rows_block_kernel(const T* __restrict__ src, typename S::Out* __restrict__ out, S* __restrict__ part,
                                                               uint64_t R, uint32_t splits, uint64_t seglen, int flags) {
    const uint64_t row = blockIdx.x / splits;
    const uint32_t seg = blockIdx.x - (uint32_t)(row * splits);
    const uint64_t begin = (uint64_t)seg * seglen;
    uint64_t end = begin + seglen;
    if (end > R) end = R;
    S a;
    a.init();
    fold_run<S, T, U>(a, src + row * R, begin, end, threadIdx.x, kBlock);
    block_reduce(a);
    if (threadIdx.x == 0) {
        if (part) part[blockIdx.x] = a;
        else out[row] = a.result(flags);
    }
}

// G lanes per row, G = 16, 32 or 64 (a quarter of a wave, half a wave, a wave): the fold over the lanes of a row costs the same per row
// whatever its length, so rows of 2 ... 4 KiB get 16 lanes (eight vectors per lane) and rows of 4 ... 8 KiB 32
template <class S, class T, int G>
__global__ __launch_bounds__(kBlock) void st_rows_wave_kernel(const T* __restrict__ src, typename S::Out* __restrict__ out, uint64_t rows, uint64_t R, int flags) {
    const uint64_t row = ((uint64_t)blockIdx.x * kBlock + threadIdx.x) / G;
    const uint32_t lane = threadIdx.x & (G - 1);
    S a;
    a.init();
    // (a group past the last row folds nothing: the lanes of a wave stay together for the exchange below)
    if (row < rows) fold_run<S, T>(a, src + row * R, 0, R, lane, G);
    group_reduce(a, G, lane);
    if (lane == 0 && row < rows) out[row] = a.result(flags);
}

// short rows (1 <= R <= 1024): the block's rows are one contiguous run, copied into LDS with coalesced 16-byte loads (row pitch R | 1
// keeps lanes that walk different rows on different banks), then groups of G lanes fold one row each.
// 24 KiB: six resident blocks per CU.  Measured on 1 GiB of f32 rows against 32 KiB (five blocks): logsumexp over rows of 10
// 0.69 -> 0.76 of peak, variance 0.71 -> 0.77, sum 0.71 -> 0.76; rows of 100: 0.67 -> 0.73, 0.73 -> 0.79, 0.73 -> 0.81; 16, 20, 22 and
// 26 KiB lie between, 48 KiB (three blocks) loses 10 %.
constexpr uint32_t kTileBytes = 24576;
constexpr uint64_t kTileMaxR = 1024;
// (also for small slabs with a few columns, as the plain reductions' tiled kernel: a row of the tile is then the slab of one outer
// index, L = R * inner elements, and a group of lanes folds one of its columns)
struct TileArgs {
    uint64_t rows;
    uint32_t R, L, inner, pitch, rpb, G;
    FastDiv32 l_div, inner_div;
};

template <class S, class T>
__global__ __launch_bounds__(kBlock) void st_rows_tile_kernel(const T* __restrict__ src, typename S::Out* __restrict__ out, TileArgs a, int flags) {
    constexpr uint32_t N = 16 / sizeof(T);
    __shared__ alignas(16) T tile[kTileBytes / sizeof(T)];
    const uint64_t row0 = (uint64_t)blockIdx.x * a.rpb;
    const uint32_t nrows = (uint32_t)(a.rows - row0 < a.rpb ? a.rows - row0 : a.rpb);
    const uint32_t ne = nrows * a.L;
    const T* p = src + row0 * a.L;
    // pitch == R: the run is copied as it lies, with 16-byte LDS stores; `mis` keeps the 16-byte phase of the global address.  Always
    // for 1- and 2-byte elements (an element-wise scatter would issue 8 or 16 sub-word stores per vector: u8 rows of 100 ran at
    // 1.9 TB/s), and for wider elements whenever rows at that pitch meet at most two to a bank (see tile_pitch); otherwise rows go
    // to a padded pitch element by element, an index division per element.
    const bool verbatim = a.pitch == a.L;
    const uint32_t mis = verbatim ? (uint32_t)((reinterpret_cast<uintptr_t>(p) & 15) / sizeof(T)) : 0u;
    auto put = [&](uint32_t e, T v) {
        if (verbatim) {
            tile[mis + e] = v;
        } else {
            const uint32_t r = fd_div(e, a.l_div);
            tile[r * a.pitch + (e - r * a.L)] = v;
        }
    };
    uint32_t head = (uint32_t)(((16 - (reinterpret_cast<uintptr_t>(p) & 15)) & 15) / sizeof(T));
    if (head > ne) head = ne;
    if (threadIdx.x < head) put(threadIdx.x, p[threadIdx.x]);
    const uint32_t nvec = (ne - head) / N;
    const Vec16<T>* pv = reinterpret_cast<const Vec16<T>*>(p + head);
    constexpr int U = 8;                                           // the whole tile in flight at once (six vectors per lane at 24 KiB)
    for (uint32_t v0 = threadIdx.x; v0 < nvec; v0 += U * kBlock) {
        Vec16<T> x[U];
#pragma unroll
        for (int u = 0; u < U; ++u)
            if (v0 + u * kBlock < nvec) x[u] = rt_ld16_nt(pv + v0 + u * kBlock);
#pragma unroll
        for (int u = 0; u < U; ++u) {
            if (v0 + u * kBlock < nvec) {
                if (verbatim) {
                    *reinterpret_cast<Vec16<T>*>(&tile[mis + head + (v0 + u * kBlock) * N]) = x[u];
                } else {
#pragma unroll
                    for (uint32_t j = 0; j < N; ++j) put(head + (v0 + u * kBlock) * N + j, x[u].e[j]);
                }
            }
        }
    }
    const uint32_t tb = head + nvec * N;
    if (tb + threadIdx.x < ne) put(tb + threadIdx.x, p[tb + threadIdx.x]);
    __syncthreads();
    const uint32_t g = threadIdx.x / a.G, j = threadIdx.x & (a.G - 1), groups = kBlock / a.G;
    // f64 logsumexp reads its rows twice (see below): there the exponentials set the time (rows of 100: 0.49 -> 0.56 of peak); for f32,
    // whose exponential is one instruction, the second round of LDS reads costs more than the rescaling it saves (rows of 256: 0.70 -> 0.67)
    constexpr bool kTwoPass = std::is_same<S, LseState<T>>::value && sizeof(T) == 8;
    const uint32_t nout = nrows * a.inner, in = a.inner;
    for (uint32_t q0 = 0; q0 < nout; q0 += groups) {                // every lane runs every trip: the exchanges below need the whole wave
        const uint32_t q = q0 + g;
        const bool live = q < nout;
        const uint32_t r = in == 1 ? q : fd_div(q, a.inner_div);
        const uint32_t c = q - r * in;
        const T* col = tile + mis + (live ? r * a.pitch + c : 0u);  // pitch == L in the verbatim layout; element k of the column at col[k * in]
        S acc;
        acc.init();
        if (live) {
            uint32_t k = j;
            if constexpr (std::is_same<S, LseState<T>>::value) {
                if (a.G == 1 && in == 1) { acc.fold_row(col, a.R); k = a.R; }
            }
            if constexpr (!kTwoPass) {
                for (; k + 3 * a.G < a.R; k += 4 * a.G) {
                    T x[4];
#pragma unroll
                    for (int u = 0; u < 4; ++u) x[u] = col[(k + u * a.G) * in];
                    acc.template push_block<4>(x, k, a.G);
                }
                for (; k < a.R; k += a.G) acc.push(col[k * in], k);
            }
        }
        if constexpr (kTwoPass) {
            // the column lies in LDS: its maximum first (the lanes' maxima, then the group's), then one exponential per element and no
            // rescaling of running sums (the running form pays one more per four elements and one per lane at the end)
            if (a.G > 1 || in > 1) {
                T top = -std::numeric_limits<T>::infinity();
                if (live) {
                    uint32_t k = j;
                    for (; k + 3 * a.G < a.R; k += 4 * a.G) {     // four LDS reads in flight
                        T x[4];
#pragma unroll
                        for (int u = 0; u < 4; ++u) x[u] = col[(k + u * a.G) * in];
                        top = m_max(m_max(top, x[0]), m_max(x[1], m_max(x[2], x[3])));
                    }
                    for (; k < a.R; k += a.G) top = m_max(top, col[k * in]);
                }
                top = group_all<OpMax>(top, a.G);
                T sum = (T)0;
                bool bad = false;
                if (live) {
                    uint32_t k = j;
                    for (; k + 3 * a.G < a.R; k += 4 * a.G) {
                        T x[4];
#pragma unroll
                        for (int u = 0; u < 4; ++u) x[u] = col[(k + u * a.G) * in];
#pragma unroll
                        for (int u = 0; u < 4; ++u) { sum = sum + S::term(x[u], top); bad |= x[u] != x[u]; }
                    }
                    for (; k < a.R; k += a.G) {
                        const T x = col[k * in];
                        sum = sum + S::term(x, top);
                        bad |= x != x;
                    }
                }
                if (S::kNoteNan && bad) sum = std::numeric_limits<T>::quiet_NaN();
                sum = group_all<OpSum>(sum, a.G);
                acc.m = top;
                acc.s = sum;
            }
        } else {
            group_reduce(acc, a.G, j);
        }
        if (j == 0 && live) out[(row0 + r) * in + c] = acc.result(flags);
    }
}

// rows of 1, 2 or 4 aligned 16-byte vectors: no staging, lane t reads vector t of the block's run (four loads in flight) and the
// lanes of a row, neighbours inside a wave, merge with one or two shuffle steps
template <class S, class T>
__global__ __launch_bounds__(kBlock) void st_rows_pow2_kernel(const T* __restrict__ src, typename S::Out* __restrict__ out, uint64_t nvec, uint32_t VR,
                                                              uint32_t vr_shift, int flags) {
    constexpr uint32_t N = 16 / sizeof(T);
    constexpr int U = 4;
    const uint64_t v0 = (uint64_t)blockIdx.x * (kBlock * U) + threadIdx.x;           // the run may start at any element
    Vec16<T> x[U];
#pragma unroll
    for (int u = 0; u < U; ++u)
        if (v0 + (uint64_t)u * kBlock < nvec) x[u] = __builtin_bit_cast(Vec16<T>, rt_ld16u<T, true>(src + (v0 + (uint64_t)u * kBlock) * N));
    const uint32_t j = threadIdx.x & (VR - 1);
#pragma unroll
    for (int u = 0; u < U; ++u) {
        const uint64_t v = v0 + (uint64_t)u * kBlock;
        S a;
        a.init();
        if constexpr (std::is_same<S, LseState<T>>::value) {
            // the row's maximum before any exponential: N of them per lane and no rescaling
            T top = -std::numeric_limits<T>::infinity();
            if (v < nvec) {
#pragma unroll
                for (uint32_t e = 0; e < N; ++e) top = m_max(top, x[u].e[e]);
            }
            top = group_all<OpMax>(top, VR);
            T sum = (T)0;
            bool bad = false;
            if (v < nvec) {
#pragma unroll
                for (uint32_t e = 0; e < N; ++e) {
                    sum = sum + S::term(x[u].e[e], top);
                    bad |= x[u].e[e] != x[u].e[e];
                }
            }
            if (S::kNoteNan && bad) sum = std::numeric_limits<T>::quiet_NaN();
            sum = group_all<OpSum>(sum, VR);
            a.m = top;
            a.s = sum;
        } else {
            if (v < nvec) a.template push_block<N>(x[u].e, (uint64_t)j * N, 1);
            group_reduce(a, VR, j);
        }
        if (j == 0 && v < nvec) out[v >> vr_shift] = a.result(flags);
    }
}

// ---- cols -------------------------------------------------------------------------------------------------------------
// src viewed as (outer, R, inner).  blockIdx.x -> (o, seg, tile); lane tx covers columns (tile * 64 + tx) * VW ..; wave ty takes
// k = begin + ty, + kWaves, ...  Results go to out[o * inner + col], partial states to part[(seg * outer + o) * inner + col].
template <class S, class T, int VW, int U = 4>
__global__ __launch_bounds__(kBlock) void st_cols_kernel(const T* __restrict__ src, typename S::Out* __restrict__ out, S* __restrict__ part, uint64_t R,
                                                         uint64_t inner, uint64_t outer, uint32_t tiles, uint32_t splits, uint64_t seglen, int flags,
                                                         uint32_t regroup, uint64_t inner_out) {
    struct alignas(sizeof(T) * VW) VecW { T e[VW]; };
    uint64_t b = blockIdx.x;
    const uint32_t tile = (uint32_t)(b % tiles);
    b /= tiles;
    const uint32_t seg = (uint32_t)(b % splits);
    const uint64_t o = b / splits;
    const uint32_t tx = threadIdx.x & (RT_WAVE - 1), ty = threadIdx.x / RT_WAVE;
    const uint64_t col0 = ((uint64_t)tile * RT_WAVE + tx) * VW;
    const bool active = col0 < inner;
    // The last lane of a row whose length is not a multiple of VW moves back to the row's last VW columns (VW <= inner here), so
    // that it too loads whole vectors: it folds `skip` columns of the lane before it a second time and does not write them.
    // (Element loads in that one lane doubled the time of its block, and with two resident blocks per CU the slowest block is
    // the kernel's time: 1 GiB f32 sum over axis 0 with 32767 columns 0.42 ms.)
    const uint64_t col = (active && inner - col0 < (uint64_t)VW) ? inner - VW : col0;
    const uint32_t skip = (uint32_t)(col0 - col);
    // rows may start at any element: unaligned 16-byte loads
    auto load = [](const T* q) -> VecW {
        if constexpr (sizeof(VecW) == 16) {
            return __builtin_bit_cast(VecW, rt_ld16u<T, true>(q));
        } else {
            VecW w;
            w.e[0] = __builtin_nontemporal_load(q);
            return w;
        }
    };
    const uint64_t begin = (uint64_t)seg * seglen;
    uint64_t end = begin + seglen;
    if (end > R) end = R;

    S a[VW];
#pragma unroll
    for (int j = 0; j < VW; ++j) a[j].init();
    if (active) {
        const T* p = src + o * R * inner + col;
        uint64_t k = begin + ty;
        for (; k + (uint64_t)(U - 1) * kWaves < end; k += (uint64_t)U * kWaves) {
            VecW v[U];
#pragma unroll
            for (int u = 0; u < U; ++u) v[u] = load(p + (k + (uint64_t)u * kWaves) * inner);
#pragma unroll
            for (int j = 0; j < VW; ++j) {
                T x[U];
#pragma unroll
                for (int u = 0; u < U; ++u) x[u] = v[u].e[j];
                a[j].template push_block<U>(x, k, kWaves);
            }
        }
        for (; k < end; k += kWaves) {
            VecW v = load(p + k * inner);
#pragma unroll
            for (int j = 0; j < VW; ++j) a[j].push(v.e[j], k);
        }
    }
    __shared__ S sm[kWaves - 1][RT_WAVE][VW];
    if (ty > 0) {
#pragma unroll
        for (int j = 0; j < VW; ++j) sm[ty - 1][tx][j] = a[j];
    }
    __syncthreads();
    if (ty == 0 && active) {
        const uint64_t at = ((uint64_t)seg * outer + o) * inner + col;
#pragma unroll
        for (int j = 0; j < VW; ++j) {
#pragma unroll
            for (int w = 0; w < kWaves - 1; ++w) a[j].merge(sm[w][tx][j]);
            if ((uint32_t)j < skip) continue;
            if constexpr (is_arg_state<S>::value) {
                // regrouped rows: column c of the joined row k is column c % inner_out of row k * regroup + c / inner_out
                if (regroup > 1 && a[j].idx != ~0ull) a[j].idx = a[j].idx * regroup + (col + j) / inner_out;
            }
            if (part) part[at + j] = a[j];
            else out[at + j] = a[j].result(flags);
        }
    }
}

// Narrow inner (fewer columns than a wave of vectors covers): the (R, inner) slab of one outer index is read as one contiguous stream
// in tiles of Tn * VW elements, a multiple of inner, so that lane t always meets the same VW columns (element t * VW + j of every
// tile, column (t * VW + j) % inner) in rows tile * L + (t * VW + j) / inner, L rows per tile, ascending.  The lanes that share a
// column are merged through LDS at the end.
struct NarrowArgs {
    uint64_t R, outer, seg_tiles;       // tiles per segment
    uint32_t inner, Tn, L, splits, G;   // columns, active lanes, rows per tile, segments per outer index, lanes per column in the final merge
    FastDiv32 inner_div;
};

template <class S, class T, int VW>
__global__ __launch_bounds__(kBlock) void st_cols_narrow_kernel(const T* __restrict__ src, typename S::Out* __restrict__ out, S* __restrict__ part, NarrowArgs a,
                                                                int flags) {
    struct alignas(sizeof(T) * VW) VecW { T e[VW]; };
    constexpr int U = 4;
    __shared__ S sm[kBlock * VW];
    const uint64_t o = blockIdx.x / a.splits;
    const uint32_t seg = (uint32_t)(blockIdx.x - o * a.splits);
    const uint32_t t = threadIdx.x;
    const uint32_t tile_elems = a.Tn * VW;
    const uint64_t slab = a.R * a.inner;
    const T* base = src + o * slab;
    S acc[VW];
    uint32_t krow[VW];
#pragma unroll
    for (int j = 0; j < VW; ++j) { acc[j].init(); krow[j] = fd_div(t * VW + j, a.inner_div); }
    if (t < a.Tn) {
        const uint64_t tile_begin = (uint64_t)seg * a.seg_tiles;
        uint64_t tile_end = tile_begin + a.seg_tiles;
        const uint64_t ntiles = (a.R + a.L - 1) / a.L;
        if (tile_end > ntiles) tile_end = ntiles;
        auto load = [&](uint64_t e) -> VecW {
            if constexpr (sizeof(VecW) == 16) {
                return __builtin_bit_cast(VecW, rt_ld16u<T, true>(base + e));          // any phase
            } else {
                VecW w;
                w.e[0] = __builtin_nontemporal_load(base + e);
                return w;
            }
        };
        uint64_t tl = tile_begin;
        // batches of U tiles that this lane's vector lies inside completely
        for (; tl + U <= tile_end && (tl + U - 1) * tile_elems + (uint64_t)t * VW + VW <= slab; tl += U) {
            VecW x[U];
#pragma unroll
            for (int u = 0; u < U; ++u) x[u] = load((tl + u) * tile_elems + (uint64_t)t * VW);
#pragma unroll
            for (int j = 0; j < VW; ++j) {
                T col[U];
#pragma unroll
                for (int u = 0; u < U; ++u) col[u] = x[u].e[j];
                acc[j].template push_block<U>(col, tl * a.L + krow[j], a.L);
            }
        }
        for (; tl < tile_end; ++tl) {                          // the last tiles, element by element where the slab ends inside a vector
            const uint64_t e = tl * tile_elems + (uint64_t)t * VW;
#pragma unroll
            for (int j = 0; j < VW; ++j)
                if (e + j < slab) acc[j].push(base[e + j], tl * a.L + krow[j]);
        }
    }
#pragma unroll
    for (int j = 0; j < VW; ++j) sm[t * VW + j] = acc[j];
    __syncthreads();
    // column c is held by the L states c, c + inner, ...: G lanes per column (a power of two, inner * G <= kBlock) share them
    const uint32_t c = t / a.G, j = t & (a.G - 1);
    S r;
    r.init();
    if (c < a.inner) {
        for (uint32_t q = j; q < a.L; q += a.G) r.merge(sm[c + q * a.inner]);
    }
    group_reduce(r, a.G, j);
    if (c < a.inner && j == 0) {
        const uint64_t at = ((uint64_t)seg * a.outer + o) * a.inner + c;
        if (part) part[at] = r;
        else out[at] = r.result(flags);
    }
}

// Short reduced axis (at most 32 rows, or a slab of at most 8 KiB): a lane per VW neighbouring outputs walks their R inputs, four rows
// in flight; consecutive lanes read consecutive addresses and one outer index is one contiguous slab, so every line is fetched once.
// (The column kernel gives such a slab a block of its own: variance over the middle axis of (2^20, 4, 64) f32 ran at 0.09 of peak.)
template <class S, class T, int VW>
__global__ __launch_bounds__(kBlock) void st_cols_short_kernel(const T* __restrict__ src, typename S::Out* __restrict__ out, uint32_t R, uint64_t inner,
                                                               uint32_t inner_vecs, FastDiv32 iv_div, uint64_t nvec_out, int flags) {
    struct alignas(sizeof(T) * VW) VecW { T e[VW]; };
    const uint64_t idx = (uint64_t)blockIdx.x * kBlock + threadIdx.x;
    if (idx >= nvec_out) return;
    const uint32_t o = fd_div((uint32_t)idx, iv_div);           // nvec_out < 2^31 on this path
    const uint32_t iv = (uint32_t)idx - o * inner_vecs;
    // the last vector of a row whose length is not a multiple of VW moves back to the row's last VW columns (VW <= inner here): it
    // folds `skip` columns of its neighbour a second time and does not write them
    const uint64_t col0 = (uint64_t)iv * VW;
    const uint64_t col = inner - col0 < (uint64_t)VW ? inner - VW : col0;
    const uint32_t skip = (uint32_t)(col0 - col);
    const T* p = src + (uint64_t)o * R * inner + col;
    S acc[VW];
#pragma unroll
    for (int j = 0; j < VW; ++j) acc[j].init();
    constexpr int U = 4;
    uint32_t k = 0;
    for (; k + U <= R; k += U) {
        VecW x[U];
#pragma unroll
        for (int u = 0; u < U; ++u) {
            if constexpr (sizeof(VecW) == 16) x[u] = __builtin_bit_cast(VecW, rt_ld16u<T, true>(p + (uint64_t)(k + u) * inner));
            else x[u].e[0] = __builtin_nontemporal_load(p + (uint64_t)(k + u) * inner);
        }
#pragma unroll
        for (int j = 0; j < VW; ++j) {
            T col[U];
#pragma unroll
            for (int u = 0; u < U; ++u) col[u] = x[u].e[j];
            acc[j].template push_block<U>(col, k, 1);
        }
    }
    for (; k < R; ++k) {
        VecW x;
        if constexpr (sizeof(VecW) == 16) x = __builtin_bit_cast(VecW, rt_ld16u<T, true>(p + (uint64_t)k * inner));
        else x.e[0] = __builtin_nontemporal_load(p + (uint64_t)k * inner);
#pragma unroll
        for (int j = 0; j < VW; ++j) acc[j].push(x.e[j], k);
    }
    typename S::Out* q = out + (uint64_t)o * inner + col;
    if constexpr (VW * sizeof(typename S::Out) == 16) {
        if (skip == 0 && (reinterpret_cast<uintptr_t>(q) & 15) == 0) {          // a whole aligned vector: one store
            struct alignas(16) OutV { typename S::Out e[VW]; } r;
#pragma unroll
            for (int j = 0; j < VW; ++j) r.e[j] = acc[j].result(flags);
            *reinterpret_cast<OutV*>(q) = r;
            return;
        }
    }
#pragma unroll
    for (int j = 0; j < VW; ++j)
        if ((uint32_t)j >= skip) q[j] = acc[j].result(flags);
}

// ---- second stage -------------------------------------------------------------------------------------------------------
// Partial state k of output o lies at part[o * ostride + k * kstride] (rows: ostride = splits, kstride = 1; columns: ostride = 1,
// kstride = number of outputs).  One wave per output, the lanes spread over k: few outputs with many partials each must not be
// folded by one lane in one long chain of dependent loads.
template <class S>
__global__ __launch_bounds__(kBlock) void st_merge_wave_kernel(const S* __restrict__ part, typename S::Out* __restrict__ out, uint64_t nout, uint32_t splits,
                                                               uint64_t ostride, uint64_t kstride, int flags) {
    const uint64_t o = (uint64_t)blockIdx.x * kWaves + threadIdx.x / RT_WAVE;
    if (o >= nout) return;
    const uint32_t lane = threadIdx.x & (RT_WAVE - 1);
    S a;
    a.init();
    for (uint32_t k = lane; k < splits; k += RT_WAVE) a.merge(part[o * ostride + (uint64_t)k * kstride]);
    group_reduce(a, RT_WAVE, lane);
    if (lane == 0) out[o] = a.result(flags);
}
// few outputs with thousands of partials each (the flat statistics of a large buffer), row layout: one block per output, four
// partials in flight per lane, then the block's fold (a single wave walking 8192 partial states took 12 of the pass's 167 us)
template <class S>
__global__ __launch_bounds__(kBlock) void st_merge_block_kernel(const S* __restrict__ part, typename S::Out* __restrict__ out, uint32_t splits, int flags) {
    const S* p = part + (uint64_t)blockIdx.x * splits;
    S a;
    a.init();
    uint32_t k = threadIdx.x;
    for (; k + 3 * kBlock < splits; k += 4 * kBlock) {
        S q[4];
#pragma unroll
        for (int u = 0; u < 4; ++u) q[u] = p[k + u * kBlock];
#pragma unroll
        for (int u = 0; u < 4; ++u) a.merge(q[u]);
    }
    for (; k < splits; k += kBlock) a.merge(p[k]);
    block_reduce(a);
    if (threadIdx.x == 0) out[blockIdx.x] = a.result(flags);
}
// many outputs, few partials each (column layout): one lane per output, coalesced over the outputs
template <class S>
__global__ __launch_bounds__(kBlock) void st_merge_lane_kernel(const S* __restrict__ part, typename S::Out* __restrict__ out, uint64_t nout, uint32_t splits, int flags) {
    const uint64_t o = (uint64_t)blockIdx.x * kBlock + threadIdx.x;
    if (o >= nout) return;
    S a = part[o];
    uint32_t k = 1;
    for (; k + 4 <= splits; k += 4) {                           // four loads in flight
        S p[4];
#pragma unroll
        for (int u = 0; u < 4; ++u) p[u] = part[(uint64_t)(k + u) * nout + o];
#pragma unroll
        for (int u = 0; u < 4; ++u) a.merge(p[u]);
    }
    for (; k < splits; ++k) a.merge(part[(uint64_t)k * nout + o]);
    out[o] = a.result(flags);
}

// an output with nothing to fold (R == 0)
template <class S>
__global__ __launch_bounds__(kBlock) void st_empty_kernel(typename S::Out* __restrict__ out, uint64_t nout, int flags) {
    const uint64_t o = (uint64_t)blockIdx.x * kBlock + threadIdx.x;
    if (o >= nout) return;
    S a;
    a.init();
    out[o] = a.result(flags);
}

// ---- host planning ------------------------------------------------------------------------------------------------------
static int32_t too_many() { return rt_fail(RT_E_INVALID, "reduce: too many outputs for one launch"); }

template <class S>
int32_t merge_cols(rt_ctx* ctx, const S* part, typename S::Out* out, uint64_t nout, uint32_t splits, int flags) {
    if (splits >= 8 && nout <= 16384) {
        hipLaunchKernelGGL((st_merge_wave_kernel<S>), dim3((unsigned)((nout + kWaves - 1) / kWaves)), dim3(kBlock), 0, ctx->stream, part, out, nout, splits,
                           (uint64_t)1, nout, flags);
    } else {
        const uint64_t mb = (nout + kBlock - 1) / kBlock;
        if (mb >= (1ull << 31)) return too_many();
        hipLaunchKernelGGL((st_merge_lane_kernel<S>), dim3((unsigned)mb), dim3(kBlock), 0, ctx->stream, part, out, nout, splits, flags);
    }
    RT_HIP(hipGetLastError());
    return RT_OK;
}

// the LDS-tiled kernel over `rows` runs of R * inner elements (inner == 1: short rows; else small slabs with a few columns)
template <class S, class T>
int32_t tile_plan(rt_ctx* ctx, const T* src, typename S::Out* out, uint64_t rows, uint64_t R, uint64_t inner, int flags) {
    TileArgs a;
    a.rows = rows;
    a.R = (uint32_t)R;
    a.inner = (uint32_t)inner;
    a.L = (uint32_t)(R * inner);
    a.pitch = rt_tile_pitch(a.L, (uint32_t)sizeof(T));
    a.rpb = (uint32_t)(kTileBytes / sizeof(T) - (a.pitch == a.L ? 16 / sizeof(T) : 0)) / a.pitch;
    a.l_div = make_fastdiv(a.L);
    a.inner_div = make_fastdiv(a.inner);
    uint32_t g = 1;                                               // lanes per output: fill the block, at most one wave, at most R
    while (g < 64 && (uint64_t)g * 2 * a.rpb * inner <= (uint64_t)kBlock && g * 2 <= a.R) g <<= 1;
    a.G = g;
    const uint64_t blocks = (rows + a.rpb - 1) / a.rpb;
    if (blocks >= (1ull << 31)) return too_many();
    hipLaunchKernelGGL((st_rows_tile_kernel<S, T>), dim3((unsigned)blocks), dim3(kBlock), 0, ctx->stream, src, out, a, flags);
    RT_HIP(hipGetLastError());
    return RT_OK;
}

template <class S, class T>
int32_t rows_plan(rt_ctx* ctx, const T* src, typename S::Out* out, uint64_t rows, uint64_t R, int flags) {
    hipStream_t s = ctx->stream;
    {
        constexpr uint64_t N = 16 / sizeof(T);
        const uint64_t vr = R / N;
        if (R % N == 0 && (vr == 1 || vr == 2 || vr == 4) && rows * vr >= 4096) {
            const uint64_t nvec = rows * vr;
            const uint64_t blocks = (nvec + (uint64_t)kBlock * 4 - 1) / ((uint64_t)kBlock * 4);
            if (blocks < (1ull << 31)) {
                hipLaunchKernelGGL((st_rows_pow2_kernel<S, T>), dim3((unsigned)blocks), dim3(kBlock), 0, s, src, out, nvec, (uint32_t)vr,
                                   vr == 1 ? 0u : (vr == 2 ? 1u : 2u), flags);
                RT_HIP(hipGetLastError());
                return RT_OK;
            }
        }
    }
    if (R <= kTileMaxR && R * sizeof(T) < 2048) {                // from 2 KiB per row a wave per row is faster (f32 rows of 1024: 0.194 / 0.157 ms)
        return tile_plan<S, T>(ctx, src, out, rows, R, 1, flags);
    }
    const uint64_t want = (uint64_t)ctx->num_cus * 8;
    if (R * sizeof(T) < 16384 && rows >= want / 2) {             // a block per row from 16 KiB on, as for the plain reductions
        const uint64_t row_bytes = R * sizeof(T);
        // 1 GiB, of peak, with 64 / 32 / 16 lanes per row -- f64 variance, rows of 2 KiB: 0.60 / - / 0.85, 3 KiB: 0.73 / - / 0.86; f32 variance,
        // rows of 2 KiB: 0.78 / - / 0.85, of 4000 B: 0.77 / - / 0.73, of 4 KiB: 0.87 / 0.85 / -; f64 logsumexp, whose exponentials make every
        // saved step count, rows of 2 KiB: 0.44 / - / 0.75, 4000 B: 0.46 / - / 0.68, 4 KiB: 0.63 / 0.73 / -
        constexpr bool kDear = std::is_same<S, LseState<double>>::value;
        const uint32_t g = kDear ? (row_bytes < 4096 ? 16 : (row_bytes < 8192 ? 32 : 64)) : (row_bytes <= 3072 ? 16 : 64);
        const uint64_t blocks = (rows * g + kBlock - 1) / kBlock;
        if (blocks >= (1ull << 31)) return too_many();
        if (g == 16) hipLaunchKernelGGL((st_rows_wave_kernel<S, T, 16>), dim3((unsigned)blocks), dim3(kBlock), 0, s, src, out, rows, R, flags);
        else if (g == 32) hipLaunchKernelGGL((st_rows_wave_kernel<S, T, 32>), dim3((unsigned)blocks), dim3(kBlock), 0, s, src, out, rows, R, flags);
        else hipLaunchKernelGGL((st_rows_wave_kernel<S, T, 64>), dim3((unsigned)blocks), dim3(kBlock), 0, s, src, out, rows, R, flags);
        RT_HIP(hipGetLastError());
        return RT_OK;
    }
    // the states that are cheap per element take the plain row reduction's fattest form: eight loads in flight per lane, three resident
    // blocks per CU, on rows or segments of 80 ... 256 KiB
    constexpr bool kCheap = std::is_same<S, MomentState<T>>::value || std::is_same<S, NormState<T, false>>::value || std::is_same<S, NormState<T, true>>::value;
    uint32_t splits = 1;
    if (rows < want) {
        const uint64_t min_seg = 16384;                           // elements; below this a split is not worth a second pass
        const uint64_t by_size = R / min_seg, by_need = (want + rows - 1) / rows;
        uint64_t sp = by_need < by_size ? by_need : by_size;
        if (sp > 4096) sp = 4096;
        if (kCheap) {
            // enough data for `want` segments of 128 KiB: segments of that size (variance of 1 GiB: 0.155 -> 0.149 ms for the first stage)
            const uint64_t by_fat = (R * sizeof(T) + (128u << 10) - 1) / (128u << 10);
            if (by_fat > sp && rows * by_fat >= want) sp = rows * by_fat <= 65536 ? by_fat : 65536 / rows;
        }
        if (sp > 1) splits = (uint32_t)sp;
    }
    if (rows * splits >= (1ull << 31)) return too_many();
    if (splits == 1) {
        // rows of 80 ... 256 KiB: eight loads in flight per lane and three resident blocks per CU, as in the plain row reduction, for
        // the states that are cheap per element (variance over rows of 32768 f32: 0.861 -> 0.892 of peak; logsumexp 0.860 -> 0.830 and
        // argmax 0.861 -> 0.600 with it: their arithmetic needs the fourth block's waves)
        if (kCheap && R * sizeof(T) >= 80 * 1024 && R * sizeof(T) <= 256 * 1024)
            hipLaunchKernelGGL((st_rows_block_kernel<S, T, 8>), dim3((unsigned)rows), dim3(kBlock), kRtThreeBlocksLds, s, src, out, (S*)nullptr, R, 1u, R, flags);
        else
        {
            // The cap of four resident blocks per CU (fewer, fatter streams) pays from rows of 32 KiB on -- 48 KiB for the index
            // states.  Below that a block is done after one trip and its fold of the states, which is long against the trip, needs the
            // other blocks' loads to hide behind: rows of 16 KiB ran at 0.62 - 0.70 of peak with the cap and run at 0.84 - 0.87 without.
            const size_t cap_from = is_arg_state<S>::value ? 48 * 1024 : 32 * 1024;
            const size_t lds = R * sizeof(T) >= cap_from ? kRtFourBlocksLds : 0;
            hipLaunchKernelGGL((st_rows_block_kernel<S, T>), dim3((unsigned)rows), dim3(kBlock), lds, s, src, out, (S*)nullptr, R, 1u, R, flags);
        }
        RT_HIP(hipGetLastError());
        return RT_OK;
    }
    constexpr uint64_t N = 16 / sizeof(T);
    uint64_t seglen = (R + splits - 1) / splits;
    seglen = (seglen + N * kBlock - 1) / (N * kBlock) * (N * kBlock);           // whole 16-byte vectors per lane
    splits = (uint32_t)((R + seglen - 1) / seglen);
    void* scratch = nullptr;
    RT_TRY(rt_scratch(ctx, (size_t)(rows * splits) * sizeof(S), &scratch));
    S* part = (S*)scratch;
    if (kCheap && seglen * sizeof(T) >= 80 * 1024 && seglen * sizeof(T) <= 256 * 1024)
        hipLaunchKernelGGL((st_rows_block_kernel<S, T, 8>), dim3((unsigned)(rows * splits)), dim3(kBlock), kRtThreeBlocksLds, s, src, out, part, R, splits, seglen,
                           flags);
    else
        hipLaunchKernelGGL((st_rows_block_kernel<S, T>), dim3((unsigned)(rows * splits)), dim3(kBlock), kRtFourBlocksLds, s, src, out, part, R, splits, seglen, flags);
    RT_HIP(hipGetLastError());
    if (splits >= 512 && rows <= 64)                              // few outputs with very many partials each: a block per output
        hipLaunchKernelGGL((st_merge_block_kernel<S>), dim3((unsigned)rows), dim3(kBlock), 0, s, part, out, splits, flags);
    else
        hipLaunchKernelGGL((st_merge_wave_kernel<S>), dim3((unsigned)((rows + kWaves - 1) / kWaves)), dim3(kBlock), 0, s, part, out, rows, splits,
                           (uint64_t)splits, (uint64_t)1, flags);
    RT_HIP(hipGetLastError());
    return RT_OK;
}

template <class S, class T, int VW>
int32_t cols_plan(rt_ctx* ctx, const T* src, typename S::Out* out, uint64_t outer, uint64_t R_all, uint64_t inner_out, int flags) {
    hipStream_t s = ctx->stream;
    const uint64_t per_tile = (uint64_t)RT_WAVE * VW;
    // Short rows are regrouped as in the plain column reduction (rt_cols_regroup): g consecutive rows are read as one, and the g
    // partial states per column join those of the split in the merge (the index states turn their positions back into row numbers).
    const uint64_t g = (outer == 1 && inner_out % VW == 0) ? rt_cols_regroup(R_all, inner_out * sizeof(T), (uint64_t)ctx->num_cus * S::kColsBlocksPerCU) : 1;
    const uint64_t R = R_all / g, inner = inner_out * g;
    const uint64_t tiles = (inner + per_tile - 1) / per_tile;
    const uint64_t want = (uint64_t)ctx->num_cus * S::kColsBlocksPerCU;
    uint32_t splits = 1;
    // whole rounds of `want` blocks (rounding the need up put 260 blocks on 256 CUs: 1 GiB f32 variance over axis 0 of 1000 columns 0.62 of
    // peak); wide rows by the estimate of rt_cols_splits_wide, except for the index states, which it did not help (391 tiles: 0.86 -> 0.77)
    splits = (g > 1 || is_arg_state<S>::value) ? rt_cols_splits_plain(outer * tiles, want, R / 64) : rt_cols_splits_wide(outer * tiles, want, R / 64, false);
    uint64_t seglen = (R + splits - 1) / splits;
    if (splits > 1) {
        seglen = (seglen + 8 * kWaves - 1) / (8 * kWaves) * (8 * kWaves);
        splits = (uint32_t)((R + seglen - 1) / seglen);
    }
    const uint64_t blocks = outer * splits * tiles;
    if (blocks >= (1ull << 31) || tiles >= (1ull << 31)) return too_many();
    S* part = nullptr;
    const bool staged = splits > 1 || g > 1;
    if (staged) {
        void* scratch = nullptr;
        RT_TRY(rt_scratch(ctx, (size_t)(splits * outer * inner) * sizeof(S), &scratch));
        part = (S*)scratch;
    }
    hipLaunchKernelGGL((st_cols_kernel<S, T, VW, S::kColsLoads>), dim3((unsigned)blocks), dim3(kBlock), 0, s, src, out, part, R, inner, outer, (uint32_t)tiles,
                       splits, seglen, flags, (uint32_t)g, inner_out);
    RT_HIP(hipGetLastError());
    if (staged) RT_TRY(merge_cols<S>(ctx, part, out, outer * inner_out, (uint32_t)(splits * g), flags));
    return RT_OK;
}

template <class S, class T>
int32_t narrow_plan(rt_ctx* ctx, const T* src, typename S::Out* out, uint64_t outer, uint64_t R, uint64_t inner, int flags) {
    constexpr uint32_t N = 16 / sizeof(T);
    // vector loads for 4- and 8-byte elements (more lanes' worth of states would not fit in LDS)
    const bool vec = sizeof(T) >= 4;
    const uint32_t vw = vec ? N : 1;
    uint32_t g = (uint32_t)inner, h = vw;                      // gcd(inner, vw)
    while (h) { uint32_t r = g % h; g = h; h = r; }
    const uint32_t innerp = (uint32_t)inner / g;               // lanes per period: Tn * vw must be a multiple of inner
    NarrowArgs a;
    a.R = R;
    a.outer = outer;
    a.inner = (uint32_t)inner;
    a.Tn = (uint32_t)kBlock / innerp * innerp;
    a.L = a.Tn * vw / (uint32_t)inner;
    a.inner_div = make_fastdiv((uint32_t)inner);
    a.G = 1;
    while (a.G < 64 && (uint64_t)a.G * 2 * inner <= (uint64_t)kBlock && a.G * 2 <= a.L) a.G <<= 1;
    const uint64_t ntiles = (R + a.L - 1) / a.L;
    const uint64_t want = (uint64_t)ctx->num_cus * S::kNarrowBlocksPerCU;
    uint64_t splits = outer >= want ? 1 : (want + outer - 1) / outer;
    if (splits > ntiles / 8) splits = ntiles / 8;              // at least 8 tiles per block
    if (splits < 1) splits = 1;
    a.seg_tiles = (ntiles + splits - 1) / splits;
    splits = (ntiles + a.seg_tiles - 1) / a.seg_tiles;
    a.splits = (uint32_t)splits;
    const uint64_t blocks = outer * splits;
    if (blocks >= (1ull << 31)) return too_many();
    S* part = nullptr;
    if (splits > 1) {
        void* scratch = nullptr;
        RT_TRY(rt_scratch(ctx, (size_t)(splits * outer * inner) * sizeof(S), &scratch));
        part = (S*)scratch;
    }
    if (vec) hipLaunchKernelGGL((st_cols_narrow_kernel<S, T, (sizeof(T) >= 4 ? (int)N : 1)>), dim3((unsigned)blocks), dim3(kBlock), 0, ctx->stream, src, out, part, a, flags);
    else hipLaunchKernelGGL((st_cols_narrow_kernel<S, T, 1>), dim3((unsigned)blocks), dim3(kBlock), 0, ctx->stream, src, out, part, a, flags);
    RT_HIP(hipGetLastError());
    if (splits > 1) RT_TRY(merge_cols<S>(ctx, part, out, outer * inner, (uint32_t)splits, flags));
    return RT_OK;
}

template <class S, class T>
int32_t plan(rt_ctx* ctx, const void* src_v, void* out_v, uint64_t outer, uint64_t R, uint64_t inner, int flags) {
    const T* src = (const T*)src_v;
    typename S::Out* out = (typename S::Out*)out_v;
    if (outer == 0 || inner == 0) return RT_OK;
    const uint64_t nout = outer * inner;
    if (R == 0) {
        const uint64_t blocks = (nout + kBlock - 1) / kBlock;
        if (blocks >= (1ull << 31)) return too_many();
        hipLaunchKernelGGL((st_empty_kernel<S>), dim3((unsigned)blocks), dim3(kBlock), 0, ctx->stream, out, nout, flags);
        RT_HIP(hipGetLastError());
        return RT_OK;
    }
    if (R == 1 && outer > 1) { inner *= outer; outer = 1; }       // an axis of one element: one run of outer * inner independent outputs
    if (inner == 1) return rows_plan<S, T>(ctx, src, out, outer, R, flags);
    constexpr int N = 16 / sizeof(T);
    // A short reduced axis goes to a lane per output vector, many small slabs with a few columns through LDS (see TileArgs) -- slabs of
    // up to a whole tile (variance over (89478, 1000, 3) f32: 0.28 of peak with a block streaming each slab, 0.69 through LDS).  Where both
    // apply, the lane-per-vector form when the rows of a slab are whole 128-byte lines, or at most four of them of 32 elements and more
    // (f32 variance over (.., 4, 64): 0.85 against 0.68; over (.., 8, 12): 0.42 against 0.74).
    // The lane-per-vector form: up to 16 rows (variance over the middle axis of (32768, 32, 256) f32 0.77 of peak on the column kernel,
    // 0.74 here), up to 32 for slabs within 24 KiB ((61440, 17, 257): 0.44 on the column kernel), up to 256 within 8 KiB; an axis of up to
    // four elements with any inner.
    const bool short_ok = (R <= 16 || (R <= 32 && R * inner * sizeof(T) <= 24576) || (R <= 256 && R * inner * sizeof(T) <= 8192)) && (inner <= 1024 || R <= 4);
    const bool slab_ok = inner <= 128 && R >= 2 && R * inner * sizeof(T) <= kTileBytes - 64 && outer >= 1024;
    const bool prefer_short = short_ok && ((inner * sizeof(T)) % 128 == 0 || (R <= 4 && inner >= 32));
    if (slab_ok && !prefer_short) return tile_plan<S, T>(ctx, src, out, outer, R, inner, flags);
    if (short_ok) {
        const bool v = inner >= (uint64_t)N;                                    // rows may start at any element and have any length
        const uint64_t ivecs = v ? (inner + N - 1) / N : inner;
        if (ivecs < (1ull << 31) && outer * ivecs < (1ull << 31)) {
            const uint64_t nvec_out = outer * ivecs;
            const uint64_t blocks = (nvec_out + kBlock - 1) / kBlock;
            if (v) hipLaunchKernelGGL((st_cols_short_kernel<S, T, N>), dim3((unsigned)blocks), dim3(kBlock), 0, ctx->stream, src, out, (uint32_t)R, inner,
                                      (uint32_t)ivecs, make_fastdiv((uint32_t)ivecs), nvec_out, flags);
            else hipLaunchKernelGGL((st_cols_short_kernel<S, T, 1>), dim3((unsigned)blocks), dim3(kBlock), 0, ctx->stream, src, out, (uint32_t)R, inner,
                                    (uint32_t)ivecs, make_fastdiv((uint32_t)ivecs), nvec_out, flags);
            RT_HIP(hipGetLastError());
            return RT_OK;
        }
    }
    // fewer columns than the vectors of one wave cover: stream the slab instead of leaving lanes idle
    if (inner < (uint64_t)RT_WAVE * (sizeof(T) >= 4 ? N : 1) && inner <= (uint64_t)kBlock && R * inner >= 1024 && outer * inner < (1ull << 31))
        return narrow_plan<S, T>(ctx, src, out, outer, R, inner, flags);
    const bool vec = inner >= (uint64_t)N;                      // one vector of columns per lane, whatever the alignment of the rows
    if (vec) return cols_plan<S, T, N>(ctx, src, out, outer, R, inner, flags);
    return cols_plan<S, T, 1>(ctx, src, out, outer, R, inner, flags);
}

template <class T>
int32_t stat_ops(rt_ctx* ctx, int op, const void* src, void* out, uint64_t outer, uint64_t R, uint64_t inner) {
    const int code = op & 0xff, flags = op & ~0xff;
    switch (code) {
        case RT_R_VARIANCE:
            if (flags & ~(RT_R_FLAG_UNBIASED | RT_R_FLAG_STD)) break;
            return plan<MomentState<T>, T>(ctx, src, out, outer, R, inner, flags);
        case RT_R_LOGSUMEXP:
            if (flags) break;
            return plan<LseState<T>, T>(ctx, src, out, outer, R, inner, flags);
        case RT_R_NORM:
            if (flags == RT_R_FLAG_L1) return plan<NormState<T, false>, T>(ctx, src, out, outer, R, inner, flags);
            if (flags == RT_R_FLAG_L2) return plan<NormState<T, true>, T>(ctx, src, out, outer, R, inner, flags);
            return rt_fail(RT_E_INVALID, "reduce: norm needs exactly one of RT_R_FLAG_L1 / RT_R_FLAG_L2 (op 0x%x)", op);
    }
    return rt_fail(RT_E_INVALID, "reduce: op 0x%x is not a reduction op code with valid flags", op);
}

template <class T>
int32_t arg_ops(rt_ctx* ctx, int op, const void* src, void* out, uint64_t outer, uint64_t R, uint64_t inner) {
    if (op == RT_R_ARGMAX) return plan<ArgState<T, true>, T>(ctx, src, out, outer, R, inner, 0);
    return plan<ArgState<T, false>, T>(ctx, src, out, outer, R, inner, 0);
}

}  // namespace

int32_t rt_reduce_stat(rt_ctx* ctx, int dtype, int op, const void* src, void* out, uint64_t outer, uint64_t R, uint64_t inner) {
    const int code = op & 0xff;
    if (code == RT_R_ARGMAX || code == RT_R_ARGMIN) {
        if (op != code) return rt_fail(RT_E_INVALID, "argmax: op 0x%x carries flags", op);
        switch (dtype) {
            case RT_U8: return arg_ops<uint8_t>(ctx, op, src, out, outer, R, inner);
            case RT_I8: return arg_ops<int8_t>(ctx, op, src, out, outer, R, inner);
            case RT_U16: return arg_ops<uint16_t>(ctx, op, src, out, outer, R, inner);
            case RT_I16: return arg_ops<int16_t>(ctx, op, src, out, outer, R, inner);
            case RT_U32: return arg_ops<uint32_t>(ctx, op, src, out, outer, R, inner);
            case RT_I32: return arg_ops<int32_t>(ctx, op, src, out, outer, R, inner);
            case RT_U64: return arg_ops<uint64_t>(ctx, op, src, out, outer, R, inner);
            case RT_I64: return arg_ops<int64_t>(ctx, op, src, out, outer, R, inner);
            case RT_F32: return arg_ops<float>(ctx, op, src, out, outer, R, inner);
            case RT_F64: return arg_ops<double>(ctx, op, src, out, outer, R, inner);
        }
        return rt_fail(RT_E_DTYPE, "argmax: dtype code %d has no order to search (f32/f64 in the reference, 8..64-bit integers added here)", dtype);
    }
    switch (dtype) {
        case RT_F32: return stat_ops<float>(ctx, op, src, out, outer, R, inner);
        case RT_F64: return stat_ops<double>(ctx, op, src, out, outer, R, inner);
    }
    return rt_fail(RT_E_DTYPE, "reduce: variance, logsumexp and norms are defined for f32 / f64 (the reference bounds them on WeightValue), not dtype code %d",
                   dtype);
}

extern "C" int32_t rt_argmax_flat(rt_ctx* ctx, int32_t dtype, int32_t op, const void* src, uint64_t src_len, uint64_t* dst, uint64_t dst_len,
                                  uint64_t start, uint64_t len) {
    RT_TRY(rt_ctx_enter(ctx));
    const int es = rt_elem_size(dtype);
    if (!es) return rt_fail(RT_E_DTYPE, "argmax: unknown dtype code %d", dtype);
    if (op != RT_R_ARGMAX && op != RT_R_ARGMIN) return rt_fail(RT_E_INVALID, "argmax: op code %d is neither argmax (9) nor argmin (10)", op);
    RT_TRY(rt_check_reduce_flat(src_len, src, dst, dst_len, start, len));
    CtxGuard g(ctx);
    return rt_reduce_stat(ctx, dtype, op, (const char*)src + start * es, dst, 1, len, 1);
}

extern "C" int32_t rt_argmax_nd(rt_ctx* ctx, int32_t dtype, int32_t op, const void* src, uint64_t src_len, uint64_t offset, int32_t rank,
                                const uint64_t* shape, const int64_t* strides, uint64_t* dst, uint64_t dst_len, int32_t dim) {
    RT_TRY(rt_ctx_enter(ctx));
    const int es = rt_elem_size(dtype);
    if (!es) return rt_fail(RT_E_DTYPE, "argmax: unknown dtype code %d", dtype);
    if (op != RT_R_ARGMAX && op != RT_R_ARGMIN) return rt_fail(RT_E_INVALID, "argmax: op code %d is neither argmax (9) nor argmin (10)", op);
    uint64_t outer = 0, inner = 0;
    bool run = false;
    RT_TRY(rt_check_reduce_nd(src_len, src, offset, rank, shape, strides, dst, dst_len, dim, &outer, &inner, &run));
    if (!run) return RT_OK;
    CtxGuard g(ctx);
    return rt_reduce_stat(ctx, dtype, op, (const char*)src + offset * es, dst, outer, shape[dim], inner);
}
