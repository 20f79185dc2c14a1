// Reductions: sum / prod / max / min / mean, full (flat) and along one axis of a row-major contiguous tensor viewed
// as (outer, R, inner).  Replaces Backend::apply_reduce_contiguous_flat / _nd (backend/mod.rs:357-409); element
// rules are the Cpu backend's accumulators (ops/reduction/mod.rs:9-137; loops backend/cpu.rs:397-449).  The
// reference's CUDA path (K/kernels/reduction/reduce.cu:239-274, 463-513) is CUB two-pass + one block per output.
//
// Kernels (all HBM-bound, algorithmic traffic (N_in + N_out) * sizeof(T)):
//   rows  (inner == 1): a block (or a wave, or a lane, depending on R) folds one contiguous row segment with
//                       16-byte loads, wave64 shuffle reduction, LDS across the waves of a block.
//   cols  (inner  > 1): lanes run along `inner` (coalesced, 16 bytes per lane), the four waves of a block take
//                       interleaved k, combined through LDS.
//   Both split R over several blocks when there are too few outputs to fill the chip; the partial results go to a
//   scratch buffer and a second launch of the same kernel folds them (two-stage grid reduction, deterministic:
//   no atomics, fixed combination order).  A single launch in which the last block to finish folds the partials
//   (ticket counter + device-scope fences) was measured and is not used: with the partials written on eight XCDs the
//   fences write back and invalidate whole L2s, about 0.7 us per block, which doubled the 1 GiB full sum to 0.35 ms.
//
// Exactness: integer sum/prod wrap, so any association gives the sequential result; max/min are order independent
// except for the sign of a zero result (-0.0 == 0.0, the sequential loop keeps the first).  Where lanes fold interleaved
// positions, the float max / min therefore run in two forms: a quick one that also notes whether a -0.0 was among the
// elements (a zero result without one is +0.0), and, only when a zero result did meet a -0.0, the same fold again with the
// position of the current extremum carried along.  Float sum/prod/mean are tree results.
#include "rt_common.h"

#include <type_traits>
#include <limits>

namespace {

template <class T> struct is_flt : std::integral_constant<bool, std::is_same<T, float>::value || std::is_same<T, double>::value> {};

template <class T, class E = void> struct carrier { typedef T type; };
template <class T> struct carrier<T, typename std::enable_if<std::is_integral<T>::value && sizeof(T) <= 4>::type> { typedef uint32_t type; };
template <class T> struct carrier<T, typename std::enable_if<std::is_integral<T>::value && sizeof(T) == 8>::type> { typedef uint64_t type; };

template <class T> __device__ __host__ constexpr T lowest_of() { return std::numeric_limits<T>::lowest(); }   // T::MIN
template <class T> __device__ __host__ constexpr T highest_of() { return std::numeric_limits<T>::max(); }     // T::MAX

constexpr int kBlock = 256;
constexpr int kWaves = kBlock / RT_WAVE;

template <class T> __device__ __forceinline__ T shfl_down_t(T v, int d) { return __shfl_down(v, d, RT_WAVE); }
template <> __device__ __forceinline__ uint8_t shfl_down_t<uint8_t>(uint8_t v, int d) { return (uint8_t)__shfl_down((int)v, d, RT_WAVE); }
template <> __device__ __forceinline__ int8_t shfl_down_t<int8_t>(int8_t v, int d) { return (int8_t)__shfl_down((int)v, d, RT_WAVE); }
template <> __device__ __forceinline__ uint16_t shfl_down_t<uint16_t>(uint16_t v, int d) { return (uint16_t)__shfl_down((int)v, d, RT_WAVE); }
template <> __device__ __forceinline__ int16_t shfl_down_t<int16_t>(int16_t v, int d) { return (int16_t)__shfl_down((int)v, d, RT_WAVE); }
template <> __device__ __forceinline__ uint32_t shfl_down_t<uint32_t>(uint32_t v, int d) { return (uint32_t)__shfl_down((int)v, d, RT_WAVE); }
template <> __device__ __forceinline__ uint64_t shfl_down_t<uint64_t>(uint64_t v, int d) { return (uint64_t)__shfl_down((unsigned long long)v, d, RT_WAVE); }
template <> __device__ __forceinline__ int64_t shfl_down_t<int64_t>(int64_t v, int d) { return (int64_t)__shfl_down((long long)v, d, RT_WAVE); }

// Accumulator state.  TRACK: the position of the current extremum is carried, so that partial folds over interleaved positions
// merge to the sequential result (float max / min only, see the header comment); without it a merge keeps its own value on ties,
// which is the sequential result when everything in `o` comes after everything folded so far.
template <int OP, class T, bool TRACK, class P = uint64_t> struct AccT {
    static constexpr bool kTrack = TRACK;
    T v;
    P pos;                  // P = uint32_t where a kernel's positions are known to fit (half the registers and shuffles)

    __device__ __forceinline__ void init() {
        if constexpr (OP == RT_R_SUM || OP == RT_R_MEAN) v = (T)0;
        else if constexpr (OP == RT_R_PROD) v = (T)1;
        else if constexpr (OP == RT_R_MAX) v = lowest_of<T>();
        else v = highest_of<T>();
        pos = (P)~(P)0;
    }
    // fold one element that comes after everything folded so far (ascending position)
    __device__ __forceinline__ void push(T x, P p) {
        if constexpr (OP == RT_R_SUM || OP == RT_R_MEAN) {
            if constexpr (is_flt<T>::value) v = v + x;
            else { typedef typename carrier<T>::type W; v = (T)(W)((W)v + (W)x); }
        } else if constexpr (OP == RT_R_PROD) {
            if constexpr (is_flt<T>::value) v = v * x;
            else { typedef typename carrier<T>::type W; v = (T)(W)((W)v * (W)x); }
        } else if constexpr (OP == RT_R_MAX) {
            if (x > v) { v = x; if constexpr (kTrack) pos = p; }            // NaN never wins; first of equals stays
        } else {
            if (x < v) { v = x; if constexpr (kTrack) pos = p; }
        }
    }
    // merge another partial state (any relative order when positions are tracked)
    __device__ __forceinline__ void merge(const AccT& o) {
        if constexpr (OP == RT_R_SUM || OP == RT_R_MEAN) {
            if constexpr (is_flt<T>::value) v = v + o.v;
            else { typedef typename carrier<T>::type W; v = (T)(W)((W)v + (W)o.v); }
        } else if constexpr (OP == RT_R_PROD) {
            if constexpr (is_flt<T>::value) v = v * o.v;
            else { typedef typename carrier<T>::type W; v = (T)(W)((W)v * (W)o.v); }
        } else if constexpr (OP == RT_R_MAX) {
            if constexpr (kTrack) { if (o.v > v || (o.v == v && o.pos < pos)) { v = o.v; pos = o.pos; } }
            else { if (o.v > v) v = o.v; }
        } else {
            if constexpr (kTrack) { if (o.v < v || (o.v == v && o.pos < pos)) { v = o.v; pos = o.pos; } }
            else { if (o.v < v) v = o.v; }
        }
    }
    __device__ __forceinline__ AccT shfl_down(int d) const {
        AccT o;
        o.v = shfl_down_t<T>(v, d);
        if constexpr (kTrack) o.pos = shfl_down_t<P>(pos, d); else o.pos = 0;
        return o;
    }
    __device__ __forceinline__ bool settled() const { return true; }
    __device__ __forceinline__ T value() const { return v; }
    // what a state carries besides its value, for the kernels that pass states through LDS as separate arrays
    static constexpr bool kExtra = TRACK;
    typedef P extra_t;
    __device__ __forceinline__ extra_t extra() const { return pos; }
    __device__ __forceinline__ static AccT make(T v, extra_t e) { AccT a; a.v = v; a.pos = e; return a; }
};
template <int OP, class T> struct needs_order : std::integral_constant<bool, is_flt<T>::value && (OP == RT_R_MAX || OP == RT_R_MIN)> {};
// the accumulator for folds over interleaved positions / for folds whose merges go in ascending order of position
template <int OP, class T> using Acc = AccT<OP, T, needs_order<OP, T>::value>;
template <int OP, class T> using AccOrd = AccT<OP, T, false>;

// The quick form of the float max / min over interleaved positions: no positions, but the signed minimum `m` of the elements' upper
// 32 bits, which is INT_MIN exactly when a -0.0 was folded (for f64 also for a negative denormal below 2^-1042: a rare false
// alarm).  A zero result with no -0.0 among the elements is +0.0 whatever the order; a zero result that met one is `unsettled`, and
// the caller folds again with AccT<OP, T, true>.
template <class T> __device__ __forceinline__ int32_t upper_bits(T x) {
    if constexpr (sizeof(T) == 4) return __builtin_bit_cast(int32_t, x);
    else return (int32_t)(__builtin_bit_cast(uint64_t, x) >> 32);
}
template <int OP, class T> struct AccQuick {
    static constexpr bool kTrack = false;
    T v;
    int32_t m;
    __device__ __forceinline__ void init() {
        v = OP == RT_R_MAX ? lowest_of<T>() : highest_of<T>();
        m = 0;
    }
    __device__ __forceinline__ void push(T x, uint64_t) {
        if constexpr (OP == RT_R_MAX) { if (x > v) v = x; } else { if (x < v) v = x; }
        const int32_t b = upper_bits<T>(x);
        m = b < m ? b : m;
    }
    __device__ __forceinline__ void merge(const AccQuick& o) {
        if constexpr (OP == RT_R_MAX) { if (o.v > v) v = o.v; } else { if (o.v < v) v = o.v; }
        m = o.m < m ? o.m : m;
    }
    __device__ __forceinline__ AccQuick shfl_down(int d) const {
        AccQuick o;
        o.v = shfl_down_t<T>(v, d);
        o.m = __shfl_down(m, d, RT_WAVE);
        return o;
    }
    __device__ __forceinline__ bool settled() const { return !(v == (T)0 && m == INT32_MIN); }
    __device__ __forceinline__ T value() const { return v == (T)0 ? (T)0 : v; }      // a settled zero is +0.0
    static constexpr bool kExtra = true;
    typedef int32_t extra_t;
    __device__ __forceinline__ extra_t extra() const { return m; }
    __device__ __forceinline__ static AccQuick make(T v, extra_t e) { AccQuick a; a.v = v; a.m = e; return a; }
};

// WeightValue::from_usize goes through f32 (core/value.rs:54-56); integers saturate like Rust's `as`.
template <class T> __device__ __forceinline__ T from_count(uint64_t n) {
    float f = (float)n;
    if constexpr (is_flt<T>::value) return (T)f;
    else {
        if (f >= (float)highest_of<T>()) return highest_of<T>();
        return (T)f;
    }
}

template <int OP, class T> __device__ __forceinline__ T finalize(T v, uint64_t count) {
    if constexpr (OP == RT_R_MEAN) {
        T c = from_count<T>(count);
        if constexpr (is_flt<T>::value) return v / c;
        else {
            if (c == 0) return (T)0;                          // refused on the host before launch
            if constexpr (std::is_signed<T>::value) { if (c == (T)-1) return (T)(0 - v); }
            return (T)(v / c);
        }
    } else {
        return v;
    }
}

// wave64 tree: after it lane 0 holds the fold of all 64 lanes
template <class A> __device__ __forceinline__ void wave_reduce(A& a) {
#pragma unroll
    for (int d = RT_WAVE / 2; d >= 1; d >>= 1) a.merge(a.shfl_down(d));
}

// block of kBlock lanes: result valid in thread 0
template <class A> __device__ __forceinline__ void block_reduce(A& a) {
    __shared__ A sa[kWaves];
    wave_reduce<A>(a);
    const int lane = threadIdx.x & (RT_WAVE - 1), w = threadIdx.x / RT_WAVE;
    if (lane == 0) sa[w] = a;
    __syncthreads();
    if (threadIdx.x == 0) {
#pragma unroll
        for (int k = 1; k < kWaves; ++k) a.merge(sa[k]);
    }
}

// the same with the result in every lane (one barrier; a decision taken on the result is then uniform without a second one)
template <class A> __device__ __forceinline__ void block_reduce_all(A& a) {
    __shared__ A sa[kWaves];
    wave_reduce<A>(a);
    const int lane = threadIdx.x & (RT_WAVE - 1), w = threadIdx.x / RT_WAVE;
    if (lane == 0) sa[w] = a;
    __syncthreads();
    a = sa[0];
#pragma unroll
    for (int k = 1; k < kWaves; ++k) a.merge(sa[k]);
}

template <class T> struct alignas(16) Vec16 { T e[16 / sizeof(T)]; };

// fold elements [begin, end) of the contiguous run `p`, lanes `tid` of `nthreads` cooperating; positions are
// reported relative to `p`
template <class A, class T, int U = 4>
__device__ __forceinline__ void fold_run(A& a, const T* __restrict__ p, uint64_t begin, uint64_t end, uint32_t tid, uint32_t nthreads) {
    constexpr uint32_t N = 16 / sizeof(T);
    if (begin >= end) return;
    // elements before the first 16-byte boundary
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
        // nothing may move across this point: left alone, the scheduler puts the first add (and with it a wait for the first
        // load) in front of the other three loads, and every trip then costs two memory latencies instead of one
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int u = 0; u < U; ++u) {
#pragma unroll
            for (uint32_t j = 0; j < N; ++j) a.push(v[u].e[j], vb + (i + (uint64_t)u * nthreads) * N + j);
        }
    }
    if (i < nvec) {
        // the last 1 .. U-1 vectors of this lane, again all loads issued before the first is used: a wave takes as long as its
        // slowest lane, and one load at a time here tripled the time of rows of 250 vectors
        Vec16<T> v[U - 1];
#pragma unroll
        for (int u = 0; u < U - 1; ++u)
            if (i + (uint64_t)u * nthreads < nvec) v[u] = rt_ld16_nt(pv + i + (uint64_t)u * nthreads);
#pragma unroll
        for (int u = 0; u < U - 1; ++u) {
            if (i + (uint64_t)u * nthreads < nvec) {
#pragma unroll
                for (uint32_t j = 0; j < N; ++j) a.push(v[u].e[j], vb + (i + (uint64_t)u * nthreads) * N + j);
            }
        }
    }
    const uint64_t tb = vb + nvec * N;
    if (tb + tid < end) a.push(p[tb + tid], tb + tid);
}

// ---- rows -------------------------------------------------------------------------------------------------------------
// grid.x = rows * splits.  Block b folds segment (b % splits) of row (b / splits); out[b] (stage 1 of 2) or out[row].
template <int OP, class T, int U = 4>
__global__ __launch_bounds__(kBlock) void reduce_rows_block_kernel(const T* __restrict__ src, T* __restrict__ out, uint64_t R, uint32_t splits,
                                                                   uint64_t seglen, uint64_t count, int last) {
    const uint64_t row = blockIdx.x / splits;
    const uint32_t seg = blockIdx.x - (uint32_t)(row * splits);
    const uint64_t begin = (uint64_t)seg * seglen;
    uint64_t end = begin + seglen;
    if (end > R) end = R;
    const T* p = src + row * R;
    if constexpr (Acc<OP, T>::kTrack) {
        // float max / min: the quick form first; the form with positions only when a zero result met a -0.0
        AccQuick<OP, T> q;
        q.init();
        fold_run<AccQuick<OP, T>, T, U>(q, p, begin, end, threadIdx.x, kBlock);
        block_reduce_all<AccQuick<OP, T> >(q);
        if (q.settled()) {
            if (threadIdx.x == 0) out[blockIdx.x] = last ? finalize<OP, T>(q.value(), count) : q.value();
            return;
        }
    }
    Acc<OP, T> a;
    a.init();
    fold_run<Acc<OP, T>, T, U>(a, p, begin, end, threadIdx.x, kBlock);
    block_reduce<Acc<OP, T> >(a);
    if (threadIdx.x == 0) out[blockIdx.x] = last ? finalize<OP, T>(a.v, count) : a.v;
}

// one wave per row (64 <= R < a few thousand): grid.x = ceil(rows / kWaves)
template <int OP, class T>
__global__ __launch_bounds__(kBlock) void reduce_rows_wave_kernel(const T* __restrict__ src, T* __restrict__ out, uint64_t rows, uint64_t R,
                                                                  uint64_t count, int last) {
    const uint64_t row = (uint64_t)blockIdx.x * kWaves + threadIdx.x / RT_WAVE;
    if (row >= rows) return;
    const uint32_t lane = threadIdx.x & (RT_WAVE - 1);
    if constexpr (Acc<OP, T>::kTrack) {
        AccQuick<OP, T> q;
        q.init();
        fold_run<AccQuick<OP, T>, T>(q, src + row * R, 0, R, lane, RT_WAVE);
        wave_reduce<AccQuick<OP, T> >(q);
        if (__builtin_amdgcn_readfirstlane((int)q.settled())) {             // lane 0 holds the row's result: the same branch for the whole wave
            if (lane == 0) out[row] = last ? finalize<OP, T>(q.value(), count) : q.value();
            return;
        }
    }
    Acc<OP, T> a;
    a.init();
    fold_run<Acc<OP, T>, T>(a, src + row * R, 0, R, lane, RT_WAVE);
    wave_reduce<Acc<OP, T> >(a);
    if (lane == 0) out[row] = last ? finalize<OP, T>(a.v, count) : a.v;
}

// one lane per row (R < 64)
template <int OP, class T>
__global__ __launch_bounds__(kBlock) void reduce_rows_lane_kernel(const T* __restrict__ src, T* __restrict__ out, uint64_t rows, uint32_t R,
                                                                  uint64_t count, int last) {
    const uint64_t row = (uint64_t)blockIdx.x * kBlock + threadIdx.x;
    if (row >= rows) return;
    AccOrd<OP, T> a;                                              // one lane folds its row in order
    a.init();
    const T* p = src + row * R;
    for (uint32_t k = 0; k < R; ++k) a.push(p[k], k);
    out[row] = last ? finalize<OP, T>(a.v, count) : a.v;
}

// ---- cols -------------------------------------------------------------------------------------------------------------
// src viewed as (outer, R, inner).  VW = elements per lane along `inner` (16 bytes worth when rows are aligned, else 1).
// blockIdx.x -> (o, seg, tile); lane tx covers columns (tile*64 + tx)*VW .., wave ty takes k = begin+ty, +kWaves, ...
// out index: ((seg * outer) + o) * inner + column   (seg = 0, splits = 1 when this is the only stage)
// One pass of the column kernel with accumulator class A; returns non-zero in a lane that wrote an unsettled result.
template <class A, int OP, class T, int VW, int U>
__device__ __forceinline__ int cols_pass(const T* __restrict__ src, T* __restrict__ out, uint64_t R, uint64_t inner, uint64_t outer, uint32_t tiles,
                                         uint32_t splits, uint64_t seglen, uint64_t count, int last, T (*sv)[RT_WAVE][VW], void* sx_raw) {
    struct alignas(sizeof(T) * VW) VecW { T e[VW]; };
    typedef typename A::extra_t X;
    X (*sx)[RT_WAVE][VW] = reinterpret_cast<X (*)[RT_WAVE][VW]>(sx_raw);
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
    // the source is read exactly once: non-temporal loads; rows may start at any element (unaligned 16-byte loads)
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

    A a[VW];
#pragma unroll
    for (int j = 0; j < VW; ++j) a[j].init();
    if (active) {
        const T* p = src + o * R * inner + col;
        uint64_t k = begin + ty;
        for (; k + (uint64_t)(U - 1) * kWaves < end; k += (uint64_t)U * kWaves) {
            VecW v[U];
#pragma unroll
            for (int u = 0; u < U; ++u) v[u] = load(p + (k + (uint64_t)u * kWaves) * inner);
            __builtin_amdgcn_sched_barrier(0);                    // all loads of a trip before the first add (see fold_run)
#pragma unroll
            for (int u = 0; u < U; ++u) {
#pragma unroll
                for (int j = 0; j < VW; ++j) a[j].push(v[u].e[j], k + (uint64_t)u * kWaves);
            }
        }
        for (; k < end; k += kWaves) {
            VecW v = load(p + k * inner);
#pragma unroll
            for (int j = 0; j < VW; ++j) a[j].push(v.e[j], k);
        }
    }
    // combine the kWaves interleaved partial folds of each column through LDS
#pragma unroll
    for (int j = 0; j < VW; ++j) {
        sv[ty][tx][j] = a[j].v;
        if constexpr (A::kExtra) sx[ty][tx][j] = a[j].extra();
    }
    __syncthreads();
    int unsettled = 0;
    if (ty == 0 && active) {
        T* q = out + ((uint64_t)seg * outer + o) * inner + col;
#pragma unroll
        for (int j = 0; j < VW; ++j) {
#pragma unroll
            for (int w = 1; w < kWaves; ++w) {
                X e = 0;
                if constexpr (A::kExtra) e = sx[w][tx][j];
                a[j].merge(A::make(sv[w][tx][j], e));
            }
            if ((uint32_t)j >= skip) {
                unsettled |= !a[j].settled();
                q[j] = last ? finalize<OP, T>(a[j].value(), count) : a[j].value();
            }
        }
    }
    return unsettled;
}

template <int OP, class T, int VW, int U = 4>
__global__ __launch_bounds__(kBlock) void reduce_cols_kernel(const T* __restrict__ src, T* __restrict__ out, uint64_t R, uint64_t inner, uint64_t outer,
                                                             uint32_t tiles, uint32_t splits, uint64_t seglen, uint64_t count, int last) {
    constexpr bool kTrack = Acc<OP, T>::kTrack;
    __shared__ T sv[kWaves][RT_WAVE][VW];
    __shared__ uint64_t sx[kTrack ? kWaves * RT_WAVE * VW : 1];
    if constexpr (kTrack) {
        // float max / min: the quick form first; the lanes whose column ended in an unsettled zero have written a provisional value,
        // and the whole block folds again with positions (every output is then written again by the same lane)
        if (!__syncthreads_or(cols_pass<AccQuick<OP, T>, OP, T, VW, U>(src, out, R, inner, outer, tiles, splits, seglen, count, last, sv, sx))) return;
    }
    cols_pass<Acc<OP, T>, OP, T, VW, U>(src, out, R, inner, outer, tiles, splits, seglen, count, last, sv, sx);
}

// ---- short rows: 1 <= R <= 1024 ----------------------------------------------------------------------------------------------
// One lane (or wave) per row reads a short row with a stride of R elements between lanes: at R = 32 that measured 0.32 TB/s.
// Here a block copies the contiguous run holding its rows into LDS with 16-byte coalesced loads (row r at pitch R | 1, so that
// lanes walking different rows hit different banks), then groups of T lanes fold one row each from LDS.
// 24 KiB: six resident blocks per CU.  Measured on 1 GiB of f32 rows against 32 KiB (five blocks): logsumexp over rows of 10
// 0.69 -> 0.76 of peak, variance 0.71 -> 0.77, sum 0.71 -> 0.76; rows of 100: 0.67 -> 0.73, 0.73 -> 0.79, 0.73 -> 0.81; 16, 20, 22 and
// 26 KiB lie between, 48 KiB (three blocks) loses 10 %.
constexpr uint32_t kRowsTileBytes = 24576;
// The same kernel takes small slabs with a few columns ((outer, R, inner) with inner <= 128 and R * inner elements in at most 8 KiB):
// a "row" of the tile is then the slab of one outer index, L = R * inner elements, and a group of lanes folds one of its columns,
// elements c, c + inner, ...  (A lane per output read such slabs from memory with a stride of one slab between lanes: 1 GiB f32
// summed over the middle axis of (2033601, 33, 2) ran at 0.11 of peak.)
struct RowsTileArgs {
    uint64_t rows;
    uint32_t R, L, inner, pitch, rpb, T;   // reduced length, elements per row of the tile (R * inner), columns, LDS pitch, rows per block, lanes per output (power of two <= 64)
    FastDiv32 l_div, inner_div;
};

template <int OP, class T>
__global__ __launch_bounds__(kBlock) void reduce_rows_tile_kernel(const T* __restrict__ src, T* __restrict__ out, RowsTileArgs a, uint64_t count) {
    constexpr uint32_t N = 16 / sizeof(T);
    __shared__ alignas(16) T tile[kRowsTileBytes / sizeof(T)];
    const uint64_t row0 = (uint64_t)blockIdx.x * a.rpb;
    const uint32_t nrows = (uint32_t)(a.rows - row0 < a.rpb ? a.rows - row0 : a.rpb);
    const uint32_t ne = nrows * a.L;
    const T* p = src + row0 * a.L;
    // pitch == L: the run is copied as it lies, with 16-byte LDS stores; `mis` keeps the 16-byte phase of the global address.  Always
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
    const uint32_t g = threadIdx.x / a.T, j = threadIdx.x & (a.T - 1), groups = kBlock / a.T;
    // the T lanes of a group take elements j, j + T, ... of their column: interleaved positions
    auto fold_row = [&](auto& acc, const T* col) {
        acc.init();
        for (uint32_t k = j; k < a.R; k += a.T) acc.push(col[k * a.inner], k);
        for (uint32_t d = a.T / 2; d >= 1; d >>= 1) {
            auto o = acc.shfl_down((int)d);
            if (j + d < a.T) acc.merge(o);
        }
    };
    const uint32_t nout = nrows * a.inner;
    for (uint32_t q = g; q < nout; q += groups) {
        const uint32_t r = a.inner == 1 ? q : fd_div(q, a.inner_div);
        const uint32_t c = q - r * a.inner;
        const T* col = tile + mis + r * a.pitch + c;              // pitch == L in the verbatim layout
        T* dst = out + (row0 + r) * a.inner + c;
        if constexpr (Acc<OP, T>::kTrack) {
            AccQuick<OP, T> qa;
            fold_row(qa, col);
            // one decision for the wave (its groups share the trip count of this loop up to the last trip, where the lanes of
            // finished groups are off): any group's unsettled zero sends all of them through the fold with positions
            if (!__builtin_amdgcn_ballot_w64(j == 0 && !qa.settled())) {
                if (j == 0) *dst = finalize<OP, T>(qa.value(), count);
                continue;
            }
        }
        Acc<OP, T> acc;
        fold_row(acc, col);
        if (j == 0) *dst = finalize<OP, T>(acc.v, count);
    }
}

// ---- short rows whose length is a power-of-two number of 16-byte vectors (16 B .. 1 KiB per row) -----------------------------------
// No staging: the rows of a block are one contiguous run, lane t reads vector t of it (four such loads in flight), the VR lanes
// that hold one row are neighbours inside a wave and fold with log2(VR) shuffles.
template <int OP, class T>
__global__ __launch_bounds__(kBlock) void reduce_rows_pow2_kernel(const T* __restrict__ src, T* __restrict__ out, uint64_t nvec, uint32_t VR, uint32_t vr_shift,
                                                                  uint64_t count) {
    constexpr uint32_t N = 16 / sizeof(T);
    constexpr int U = 4;
    const uint64_t v0 = (uint64_t)blockIdx.x * (kBlock * U) + threadIdx.x;           // the run may start at any element
    Vec16<T> x[U];
#pragma unroll
    for (int u = 0; u < U; ++u)
        if (v0 + (uint64_t)u * kBlock < nvec) x[u] = __builtin_bit_cast(Vec16<T>, rt_ld16u<T, true>(src + (v0 + (uint64_t)u * kBlock) * N));
    const uint32_t j = threadIdx.x & (VR - 1);                    // position of this lane's vector inside its row
#pragma unroll
    for (int u = 0; u < U; ++u) {
        const uint64_t v = v0 + (uint64_t)u * kBlock;
        // lane j holds elements j*N .. j*N+N-1 of its row, and with the distance doubling from 1 every merge joins a run of lanes
        // with the run right after it: in ascending order, so the float max / min need no positions here
        AccOrd<OP, T> a;
        a.init();
        if (v < nvec) {
#pragma unroll
            for (uint32_t e = 0; e < N; ++e) a.push(x[u].e[e], (uint64_t)j * N + e);
        }
        for (uint32_t d = 1; d < VR; d <<= 1) {
            AccOrd<OP, T> o = a.shfl_down((int)d);
            if (j + d < VR) a.merge(o);
        }
        if (j == 0 && v < nvec) out[v >> vr_shift] = finalize<OP, T>(a.v, count);
    }
}

// ---- narrow columns: inner < 128, long R ------------------------------------------------------------------------------------
// With lanes along `inner` only `inner` of 64 lanes would work.  Here the (R, inner) slab of one outer index is read as one
// contiguous stream in tiles of S = Tn * VW elements, S a multiple of inner, so that lane t always meets the same VW columns
// (element t*VW + j of every tile) and rows tile*L + (t*VW + j) / inner, L = S / inner rows per tile, in ascending order.  The
// lanes that share a column are combined through LDS at the end (ties by position, so the first extremum still wins).
struct ColsNarrowArgs {
    uint64_t R, outer;
    uint32_t inner, Tn, L, splits, G;   // columns, active lanes, rows per tile, segments per outer index, lanes per column in the final merge
    uint64_t seg_tiles;                 // tiles per segment
    FastDiv32 inner_div;
};

// One pass of the narrow-column kernel with accumulator class A; returns non-zero in a lane that wrote an unsettled result.
template <class A, int OP, class T, int VW>
__device__ __forceinline__ int cols_narrow_pass(const T* __restrict__ src, T* __restrict__ out, const ColsNarrowArgs& a, uint64_t count, int last, T* sv,
                                                void* sx_raw) {
    struct alignas(sizeof(T) * VW) VecW { T e[VW]; };
    typedef typename A::extra_t X;
    X* sx = reinterpret_cast<X*>(sx_raw);
    const uint64_t o = blockIdx.x / a.splits;
    const uint32_t seg = (uint32_t)(blockIdx.x - o * a.splits);
    const uint32_t t = threadIdx.x;
    const uint32_t S = a.Tn * VW;
    const uint64_t slab = a.R * a.inner;                       // elements of one outer index
    const T* base = src + o * slab;
    A acc[VW];
    uint32_t krow[VW];
#pragma unroll
    for (int j = 0; j < VW; ++j) { acc[j].init(); krow[j] = fd_div(t * VW + j, a.inner_div); }
    if (t < a.Tn) {
        const uint64_t tile_begin = (uint64_t)seg * a.seg_tiles;
        uint64_t tile_end = tile_begin + a.seg_tiles;
        const uint64_t ntiles = (a.R + a.L - 1) / a.L;
        if (tile_end > ntiles) tile_end = ntiles;
        constexpr int U = 4;
        for (uint64_t tl = tile_begin; tl < tile_end; tl += U) {
            VecW x[U];
            bool full[U];
#pragma unroll
            for (int u = 0; u < U; ++u) {
                const uint64_t e = (tl + u) * S + (uint64_t)t * VW;
                full[u] = tl + u < tile_end && e + VW <= slab;
                if (full[u]) {
                    if constexpr (sizeof(VecW) == 16) x[u] = __builtin_bit_cast(VecW, rt_ld16u<T, true>(base + e));     // any phase
                    else x[u].e[0] = __builtin_nontemporal_load(base + e);
                }
            }
#pragma unroll
            for (int u = 0; u < U; ++u) {
                const uint32_t k0 = (uint32_t)((tl + u - tile_begin) * a.L);       // row inside the segment: below 2^32 (checked on the host)
                if (full[u]) {
#pragma unroll
                    for (int j = 0; j < VW; ++j) acc[j].push(x[u].e[j], k0 + krow[j]);
                } else if (tl + u < tile_end) {                // the slab ends inside this lane's vector
                    const uint64_t e = (tl + u) * S + (uint64_t)t * VW;
#pragma unroll
                    for (int j = 0; j < VW; ++j)
                        if (e + j < slab) acc[j].push(base[e + j], k0 + krow[j]);
                }
            }
        }
    }
#pragma unroll
    for (int j = 0; j < VW; ++j) {
        sv[t * VW + j] = acc[j].v;
        if constexpr (A::kExtra) sx[t * VW + j] = acc[j].extra();
    }
    __syncthreads();
    // column c is held by the L values c, c + inner, ...: G lanes per column (a power of two, inner * G <= kBlock) share them
    const uint32_t c = t / a.G, j = t & (a.G - 1);
    A r;
    r.init();
    if (c < a.inner) {
        for (uint32_t q = j; q < a.L; q += a.G) {
            X e = 0;
            if constexpr (A::kExtra) e = sx[c + q * a.inner];
            r.merge(A::make(sv[c + q * a.inner], e));
        }
    }
    for (uint32_t d = a.G / 2; d >= 1; d >>= 1) {
        A x = r.shfl_down((int)d);
        if (j + d < a.G) r.merge(x);
    }
    if (c < a.inner && j == 0) {
        out[((uint64_t)seg * a.outer + o) * a.inner + c] = last ? finalize<OP, T>(r.value(), count) : r.value();
        return !r.settled();
    }
    return 0;
}

template <int OP, class T, int VW>
__global__ __launch_bounds__(kBlock) void reduce_cols_narrow_kernel(const T* __restrict__ src, T* __restrict__ out, ColsNarrowArgs a, uint64_t count,
                                                                    int last) {
    constexpr bool kTrack = Acc<OP, T>::kTrack;
    __shared__ T sv[kBlock * VW];
    __shared__ uint32_t sx[kTrack ? kBlock * VW : 1];
    if constexpr (kTrack) {
        // float max / min: the quick form first, the fold with positions only when a column's zero result met a -0.0
        if (!__syncthreads_or(cols_narrow_pass<AccQuick<OP, T>, OP, T, VW>(src, out, a, count, last, sv, sx))) return;
    }
    cols_narrow_pass<AccT<OP, T, kTrack, uint32_t>, OP, T, VW>(src, out, a, count, last, sv, sx);
}

// ---- short reduced axis: R <= 32, any inner -----------------------------------------------------------------------------------
// One lane per VW neighbouring outputs walks the R inputs of each (they are `inner` apart); consecutive lanes read consecutive
// addresses, and everything one outer index needs is one contiguous slab, so every cache line is fetched once.
template <int OP, class T, int VW>
__global__ __launch_bounds__(kBlock) void reduce_cols_short_kernel(const T* __restrict__ src, T* __restrict__ out, uint32_t R, uint64_t inner,
                                                                   uint32_t inner_vecs, FastDiv32 iv_div, uint64_t nvec_out, uint64_t count) {
    struct alignas(sizeof(T) * VW) VecW { T e[VW]; };
    const uint64_t idx = (uint64_t)blockIdx.x * kBlock + threadIdx.x;
    if (idx >= nvec_out) return;
    const uint32_t o = fd_div((uint32_t)idx, iv_div);           // nvec_out < 2^32 on this path
    const uint32_t iv = (uint32_t)idx - o * inner_vecs;
    // the last vector of a row whose length is not a multiple of VW moves back to the row's last VW columns (VW <= inner here): it
    // folds `skip` columns of its neighbour a second time and does not write them
    const uint64_t col0 = (uint64_t)iv * VW;
    const uint64_t col = inner - col0 < (uint64_t)VW ? inner - VW : col0;
    const uint32_t skip = (uint32_t)(col0 - col);
    const T* p = src + (uint64_t)o * R * inner + col;
    AccOrd<OP, T> acc[VW];                                      // each lane folds its columns in order
#pragma unroll
    for (int j = 0; j < VW; ++j) acc[j].init();
    constexpr int U = 4;
    for (uint32_t k = 0; k < R; k += U) {
        VecW x[U];
#pragma unroll
        for (int u = 0; u < U; ++u) {
            if (k + u < R) {
                if constexpr (sizeof(VecW) == 16) x[u] = __builtin_bit_cast(VecW, rt_ld16u<T, true>(p + (uint64_t)(k + u) * inner));
                else x[u].e[0] = __builtin_nontemporal_load(p + (uint64_t)(k + u) * inner);
            }
        }
#pragma unroll
        for (int u = 0; u < U; ++u) {
            if (k + u < R) {
#pragma unroll
                for (int j = 0; j < VW; ++j) acc[j].push(x[u].e[j], k + u);
            }
        }
    }
    T* q = out + (uint64_t)o * inner + col;
    if constexpr (VW * sizeof(T) == 16) {
        if (skip == 0 && (reinterpret_cast<uintptr_t>(q) & 15) == 0) {          // a whole aligned vector: one store
            Vec16<T> r;
#pragma unroll
            for (int j = 0; j < VW; ++j) r.e[j] = finalize<OP, T>(acc[j].v, count);
            *reinterpret_cast<Vec16<T>*>(q) = r;
            return;
        }
    }
#pragma unroll
    for (int j = 0; j < VW; ++j)
        if ((uint32_t)j >= skip) q[j] = finalize<OP, T>(acc[j].v, count);
}

constexpr uint64_t kRowsTileMaxR = 1024;

// ---- second stage of a split column reduction with few outputs ----------------------------------------------------------------
// part[k * nout + o], k < splits.  One wave per output with the lanes spread over k: a lane per output would walk its `splits`
// partials in one chain of dependent loads (1 GiB sum over 3 columns: 0.209 -> 0.17 ms).
template <int OP, class T>
__global__ __launch_bounds__(kBlock) void reduce_merge_wave_kernel(const T* __restrict__ part, T* __restrict__ out, uint64_t nout, uint32_t splits, uint64_t count) {
    const uint64_t o = (uint64_t)blockIdx.x * kWaves + threadIdx.x / RT_WAVE;
    if (o >= nout) return;
    const uint32_t lane = threadIdx.x & (RT_WAVE - 1);
    Acc<OP, T> a;
    a.init();
    for (uint32_t k = lane; k < splits; k += RT_WAVE) a.push(part[(uint64_t)k * nout + o], k);       // partials arrive in segment order
    wave_reduce<Acc<OP, T> >(a);
    if (lane == 0) out[o] = finalize<OP, T>(a.v, count);
}
// Second stage of a float max / min over regrouped rows (cols_launch): the partials of one column cover interleaved sets of rows,
// each holding the sequential result of its own set.  Their maximum is the column's; a zero maximum takes the sign that the zero
// partials share, and where they disagree the column itself is searched for its first zero (the wave walks the rows in order and
// stops at the first stretch that holds one).  One wave per output.
template <int OP, class T>
__global__ __launch_bounds__(kBlock) void reduce_merge_regroup_kernel(const T* __restrict__ part, T* __restrict__ out, const T* __restrict__ src, uint64_t nout,
                                                                      uint32_t nparts, uint64_t rows) {
    const uint64_t o = (uint64_t)blockIdx.x * kWaves + threadIdx.x / RT_WAVE;
    if (o >= nout) return;
    const uint32_t lane = threadIdx.x & (RT_WAVE - 1);
    AccOrd<OP, T> a;
    a.init();
    bool pz = false, nz = false;
    for (uint32_t k = lane; k < nparts; k += RT_WAVE) {
        const T x = part[(uint64_t)k * nout + o];
        a.push(x, k);
        if (x == (T)0) { if (upper_bits<T>(x) < 0) nz = true; else pz = true; }
    }
    wave_reduce<AccOrd<OP, T> >(a);
    const bool any_pz = __builtin_amdgcn_ballot_w64(pz) != 0, any_nz = __builtin_amdgcn_ballot_w64(nz) != 0;
    T v = __shfl(a.v, 0, RT_WAVE);
    if (v == (T)0) {
        bool neg = any_nz;
        if (any_nz && any_pz) {
            uint64_t first = ~0ull;
            for (uint64_t base = 0; base < rows; base += (uint64_t)RT_WAVE * 4) {
#pragma unroll
                for (int u = 3; u >= 0; --u) {
                    const uint64_t r = base + (uint64_t)u * RT_WAVE + lane;
                    if (r < rows && src[r * nout + o] == (T)0) first = r;
                }
                if (__builtin_amdgcn_ballot_w64(first != ~0ull)) break;
            }
#pragma unroll
            for (int d = RT_WAVE / 2; d >= 1; d >>= 1) {
                const uint64_t f2 = shfl_down_t<uint64_t>(first, d);
                first = f2 < first ? f2 : first;
            }
            first = __shfl(first, 0, RT_WAVE);
            neg = upper_bits<T>(src[first * nout + o]) < 0;
        }
        v = neg ? -(T)0 : (T)0;
    }
    if (lane == 0) out[o] = v;
}

template <int OP, class T>
bool merge_few_outputs(rt_ctx* ctx, const T* part, T* out, uint64_t nout, uint32_t splits, uint64_t count) {
    if (splits < 8 || nout > 16384) return false;
    hipLaunchKernelGGL((reduce_merge_wave_kernel<OP, T>), dim3((unsigned)((nout + kWaves - 1) / kWaves)), dim3(kBlock), 0, ctx->stream, part, out, nout, splits,
                       count);
    return true;
}

// ---- host planning ------------------------------------------------------------------------------------------------------
// the LDS-tiled kernel over `rows` runs of R * inner elements (inner == 1: short rows; else small slabs with a few columns)
template <int OP, class T>
int32_t tile_launch(rt_ctx* ctx, const T* src, T* out, uint64_t rows, uint64_t R, uint64_t inner, uint64_t count) {
    RowsTileArgs a;
    a.rows = rows;
    a.R = (uint32_t)R;
    a.inner = (uint32_t)inner;
    a.L = (uint32_t)(R * inner);
    a.pitch = rt_tile_pitch(a.L, (uint32_t)sizeof(T));
    a.rpb = (uint32_t)(kRowsTileBytes / sizeof(T) - (a.pitch == a.L ? 16 / sizeof(T) : 0)) / a.pitch;
    a.l_div = make_fastdiv(a.L);
    a.inner_div = make_fastdiv(a.inner);
    uint32_t t = 1;                                               // lanes per output: fill the block, at most one wave, at most R
    while (t < 64 && (uint64_t)t * 2 * a.rpb * inner <= (uint64_t)kBlock && t * 2 <= a.R) t <<= 1;
    a.T = t;
    const uint64_t blocks = (rows + a.rpb - 1) / a.rpb;
    if (blocks >= (1ull << 31)) return rt_fail(RT_E_INVALID, "reduce: too many rows for one launch");
    hipLaunchKernelGGL((reduce_rows_tile_kernel<OP, T>), dim3((unsigned)blocks), dim3(kBlock), 0, ctx->stream, src, out, a, count);
    RT_HIP(hipGetLastError());
    return RT_OK;
}

template <int OP, class T>
int32_t rows_stage(rt_ctx* ctx, const T* src, T* out, uint64_t rows, uint64_t R, uint64_t count, bool allow_split) {
    hipStream_t s = ctx->stream;
    if (rows == 0) return RT_OK;
    {
        constexpr uint64_t N = 16 / sizeof(T);
        const uint64_t vr = R / N;
        // (small inputs stay with the staged kernel, where few rows mean one lane per row: a sum in index order, bit for bit the
        // sequential result)
        const uint64_t vr_max = 64;
        if (count == R && R % N == 0 && vr >= 1 && vr <= vr_max && (vr & (vr - 1)) == 0 && rows * vr >= 4096) {
            const uint64_t nvec = rows * vr;
            const uint64_t blocks = (nvec + (uint64_t)kBlock * 4 - 1) / ((uint64_t)kBlock * 4);
            if (blocks < (1ull << 31)) {
                uint32_t shift = 0;
                while ((1ull << shift) < vr) ++shift;
                hipLaunchKernelGGL((reduce_rows_pow2_kernel<OP, T>), dim3((unsigned)blocks), dim3(kBlock), 0, s, src, out, nvec, (uint32_t)vr, shift, count);
                RT_HIP(hipGetLastError());
                return RT_OK;
            }
        }
    }
    // short rows (not the second stage of a split reduction).  From 2 KiB per row a wave per row is faster (f32 sum, 1 GiB: rows of
    // 512 elements 0.183 ms staged / 0.155 ms direct, 1024: 0.188 / 0.159; below that the staged form wins, 256: 0.185 / 0.222)
    if (R >= 1 && R <= kRowsTileMaxR && R * sizeof(T) < 2048 && count == R) {
        return tile_launch<OP, T>(ctx, src, out, rows, R, 1, count);
    }
    if (R < 64) {
        uint64_t blocks = (rows + kBlock - 1) / kBlock;
        if (blocks >= (1ull << 31)) return rt_fail(RT_E_INVALID, "reduce: too many rows for one launch");
        hipLaunchKernelGGL((reduce_rows_lane_kernel<OP, T>), dim3((unsigned)blocks), dim3(kBlock), 0, s, src, out, rows, (uint32_t)R, count, 1);
        RT_HIP(hipGetLastError());
        return RT_OK;
    }
    const uint64_t want = (uint64_t)ctx->num_cus * 8;
    // a wave per row up to 16 KiB, a block per row from there on (1 GiB, sum: rows of 8 KiB 0.86 of peak by waves / 0.56 by blocks, rows of
    // 16 KiB 0.85 / 0.91, of 32 KiB 0.81 / 0.90; the same for 1-, 2-, 4- and 8-byte elements)
    if (R * sizeof(T) < 16384 && rows >= want / 2) {
        uint64_t blocks = (rows + kWaves - 1) / kWaves;
        if (blocks >= (1ull << 31)) return rt_fail(RT_E_INVALID, "reduce: too many rows for one launch");
        hipLaunchKernelGGL((reduce_rows_wave_kernel<OP, T>), dim3((unsigned)blocks), dim3(kBlock), 0, s, src, out, rows, R, count, 1);
        RT_HIP(hipGetLastError());
        return RT_OK;
    }
    // block per (row, segment); split long rows when there are too few of them
    // The first-stage launches ask for kRtFourBlocksLds bytes of LDS they never touch, which holds a CU to four resident blocks
    // instead of eight: fewer concurrent streams keep more DRAM pages open.  1 GiB f32: full sum 0.167 -> 0.159 ms, sum and max
    // over rows of 32768 0.159 -> 0.158 and 0.163 -> 0.158 ms.  (The same cap on the one-vector-per-lane elementwise kernels,
    // which need every wave slot to cover latency, and on the wave-per-row kernel only lost time.)
    uint32_t splits = 1;
    if (allow_split && rows < want) {
        const uint64_t min_seg = 16384;                       // elements; below this a split is not worth a second pass
        uint64_t by_size = R / min_seg;
        uint64_t by_need = (want + rows - 1) / rows;
        uint64_t sp = by_need < by_size ? by_need : by_size;
        if (sp > 4096) sp = 4096;
        // enough data for `want` segments of 128 KiB: segments of that size, which stream fastest (see below); at most 65536 partials
        const uint64_t by_fat = (R * sizeof(T) + (128u << 10) - 1) / (128u << 10);
        if (by_fat > sp && rows * by_fat >= want) sp = rows * by_fat <= 65536 ? by_fat : 65536 / rows;
        if (sp > 1) splits = (uint32_t)sp;
    }
    if (rows * splits >= (1ull << 31)) return rt_fail(RT_E_INVALID, "reduce: too many rows for one launch");
    if (splits == 1) {
        // Rows of 80 ... 256 KiB: eight loads in flight per lane (a trip of the block covers 32 KiB) and three resident blocks per CU
        // instead of four loads and four blocks -- fewer, fatter streams.  1 GiB, rows of 32768 f32: sum 0.867 -> 0.895 of peak, max
        // 0.858 -> 0.877; f64 rows of 10000 ... 32768: 0.87 -> 0.89-0.90.  Shorter rows do not fill such trips (rows of 10000 f32:
        // 0.90 -> 0.77), longer ones lose 1-2 %.
        const uint64_t row_bytes = R * sizeof(T);
        if (row_bytes >= 80 * 1024 && row_bytes <= 256 * 1024)
            hipLaunchKernelGGL((reduce_rows_block_kernel<OP, T, 8>), dim3((unsigned)rows), dim3(kBlock), kRtThreeBlocksLds, s, src, out, R, 1u, R, count, 1);
        else
            hipLaunchKernelGGL((reduce_rows_block_kernel<OP, T>), dim3((unsigned)rows), dim3(kBlock), kRtFourBlocksLds, s, src, out, R, 1u, R, count, 1);
        RT_HIP(hipGetLastError());
        return RT_OK;
    }
    constexpr uint64_t N = 16 / sizeof(T);
    uint64_t seglen = (R + splits - 1) / splits;
    seglen = (seglen + N * kBlock - 1) / (N * kBlock) * (N * kBlock);       // whole 16-byte vectors per lane
    splits = (uint32_t)((R + seglen - 1) / seglen);
    void* scratch = nullptr;
    RT_TRY(rt_scratch(ctx, (size_t)(rows * splits) * sizeof(T), &scratch));
    T* part = (T*)scratch;
    if (seglen * sizeof(T) >= 80 * 1024 && seglen * sizeof(T) <= 256 * 1024)
        hipLaunchKernelGGL((reduce_rows_block_kernel<OP, T, 8>), dim3((unsigned)(rows * splits)), dim3(kBlock), kRtThreeBlocksLds, s, src, part, R, splits, seglen, count, 0);
    else
        hipLaunchKernelGGL((reduce_rows_block_kernel<OP, T>), dim3((unsigned)(rows * splits)), dim3(kBlock), kRtFourBlocksLds, s, src, part, R, splits, seglen, count, 0);
    RT_HIP(hipGetLastError());
    // second stage: each row of `splits` partials -> one output (mean divides by the original count)
    if (splits < 64) {
        uint64_t blocks = (rows + kBlock - 1) / kBlock;
        hipLaunchKernelGGL((reduce_rows_lane_kernel<OP, T>), dim3((unsigned)blocks), dim3(kBlock), 0, s, part, out, rows, splits, count, 1);
    } else {
        hipLaunchKernelGGL((reduce_rows_block_kernel<OP, T>), dim3((unsigned)rows), dim3(kBlock), 0, s, part, out, (uint64_t)splits, 1u, (uint64_t)splits, count, 1);
    }
    RT_HIP(hipGetLastError());
    return RT_OK;
}

template <int OP, class T, int VW>
int32_t cols_launch(rt_ctx* ctx, const T* src, T* out, uint64_t outer, uint64_t R_all, uint64_t inner_out, uint64_t count, bool allow_split) {
    hipStream_t s = ctx->stream;
    const uint64_t per_tile = (uint64_t)RT_WAVE * VW;
    // Short rows are regrouped (rt_cols_regroup): g consecutive rows of `inner_out` columns are read as one row of g * inner_out
    // columns, and the g partial results per column join the partials of the split in the second stage (the float max / min, whose
    // zero results follow row positions, have a second stage of their own for this).  Only for one outer index.
    const uint64_t g = (allow_split && outer == 1 && inner_out % VW == 0) ? rt_cols_regroup(R_all, inner_out * sizeof(T), (uint64_t)ctx->num_cus) : 1;
    const uint64_t R = R_all / g, inner = inner_out * g;
    const uint64_t tiles = (inner + per_tile - 1) / per_tile;
    // One block of four waves per CU, eight loads in flight per lane, each block streaming a long run of rows: the segments are cut so
    // that the blocks fill the CUs in whole rounds (1 GiB f32 sums over axis 0, one block per CU against two: 8192 x 32768 0.857 ->
    // 0.893 of peak, 26844 x 10000 0.66 -> 0.82, 13422 x 20000 0.74 -> 0.88; eight blocks per CU: 0.70-0.83); see rt_cols_splits_plain / _wide.
    // Outputs that already give every CU a block are not split unless their last round would be far from full.
    const uint64_t cus = (uint64_t)ctx->num_cus;
    uint32_t splits = 1;
    if (allow_split) splits = g > 1 ? rt_cols_splits_plain(outer * tiles, cus, R / 64) : rt_cols_splits_wide(outer * tiles, cus, R / 64, true);
    uint64_t seglen = (R + splits - 1) / splits;
    if (splits > 1) {
        seglen = (seglen + 8 * kWaves - 1) / (8 * kWaves) * (8 * kWaves);
        splits = (uint32_t)((R + seglen - 1) / seglen);
    }
    const uint64_t blocks = outer * splits * tiles;
    if (blocks >= (1ull << 31) || tiles >= (1ull << 31)) return rt_fail(RT_E_INVALID, "reduce: too many outputs for one launch");
    if (splits == 1 && g == 1) {
        // (eight loads in flight per lane from 256 rows on; a short axis would spend its time in the one-row-at-a-time remainder)
        if (R >= 256)
            hipLaunchKernelGGL((reduce_cols_kernel<OP, T, VW, 8>), dim3((unsigned)blocks), dim3(kBlock), 0, s, src, out, R, inner, outer,
                               (uint32_t)tiles, 1u, seglen, count, 1);
        else
            hipLaunchKernelGGL((reduce_cols_kernel<OP, T, VW>), dim3((unsigned)blocks), dim3(kBlock), 0, s, src, out, R, inner, outer,
                               (uint32_t)tiles, 1u, seglen, count, 1);
        RT_HIP(hipGetLastError());
        return RT_OK;
    }
    void* scratch = nullptr;
    RT_TRY(rt_scratch(ctx, (size_t)(splits * outer * inner) * sizeof(T), &scratch));
    T* part = (T*)scratch;
    hipLaunchKernelGGL((reduce_cols_kernel<OP, T, VW, 8>), dim3((unsigned)blocks), dim3(kBlock), 0, s, src, part, R, inner, outer,
                       (uint32_t)tiles, splits, seglen, count, 0);
    RT_HIP(hipGetLastError());
    // second stage: partials are (splits, outer * inner) -- with regrouped rows (splits * g, inner_out): a column reduce with R = splits * g
    const uint64_t inner2 = outer * inner_out, R2 = (uint64_t)splits * g;
    if constexpr (Acc<OP, T>::kTrack) {
        if (g > 1) {
            hipLaunchKernelGGL((reduce_merge_regroup_kernel<OP, T>), dim3((unsigned)((inner2 + kWaves - 1) / kWaves)), dim3(kBlock), 0, s, part, out, src, inner2,
                               (uint32_t)R2, R_all);
            RT_HIP(hipGetLastError());
            return RT_OK;
        }
    }
    if (merge_few_outputs<OP, T>(ctx, part, out, inner2, (uint32_t)R2, count)) { RT_HIP(hipGetLastError()); return RT_OK; }
    const uint64_t tiles2 = (inner2 + per_tile - 1) / per_tile;
    if (tiles2 >= (1ull << 31)) return rt_fail(RT_E_INVALID, "reduce: too many outputs for one launch");
    hipLaunchKernelGGL((reduce_cols_kernel<OP, T, VW>), dim3((unsigned)tiles2), dim3(kBlock), 0, s, part, out, R2, inner2, (uint64_t)1,
                       (uint32_t)tiles2, 1u, R2, count, 1);
    RT_HIP(hipGetLastError());
    return RT_OK;
}

template <int OP, class T>
int32_t cols_narrow(rt_ctx* ctx, const T* src, T* out, uint64_t outer, uint64_t R, uint64_t inner) {
    constexpr uint32_t N = 16 / sizeof(T);
    const uint32_t vw = N;                                     // 16-byte loads at element alignment: any phase of the slabs
    uint32_t g = (uint32_t)inner, h = vw;                      // gcd(inner, vw)
    while (h) { uint32_t t = g % h; g = h; h = t; }
    const uint32_t innerp = (uint32_t)inner / g;               // lanes per period: Tn * vw must be a multiple of inner
    ColsNarrowArgs a;
    a.R = R;
    a.outer = outer;
    a.inner = (uint32_t)inner;
    a.Tn = (uint32_t)kBlock / innerp * innerp;
    a.L = a.Tn * vw / (uint32_t)inner;
    a.inner_div = make_fastdiv((uint32_t)inner);
    a.G = 1;
    while (a.G < 64 && (uint64_t)a.G * 2 * inner <= (uint64_t)kBlock && a.G * 2 <= a.L) a.G <<= 1;
    const uint64_t ntiles = (R + a.L - 1) / a.L;
    // resident blocks per CU: 1 GiB over 3 .. 100 columns runs at 0.82 .. 0.86 of peak with six, 0.72 .. 0.76 with four, 0.55 .. 0.80 with eight
    const uint64_t want = (uint64_t)ctx->num_cus * 6;
    uint64_t splits = outer >= want ? 1 : (want + outer - 1) / outer;
    if (splits > ntiles / 8) splits = ntiles / 8;              // at least 8 tiles per block
    if (splits < 1) splits = 1;
    a.seg_tiles = (ntiles + splits - 1) / splits;
    splits = (ntiles + a.seg_tiles - 1) / a.seg_tiles;
    a.splits = (uint32_t)splits;
    const uint64_t blocks = outer * splits;
    if (blocks >= (1ull << 31)) return rt_fail(RT_E_INVALID, "reduce: too many outputs for one launch");
    T* dst1 = out;
    if (splits > 1) {
        void* scratch = nullptr;
        RT_TRY(rt_scratch(ctx, (size_t)(splits * outer * inner) * sizeof(T), &scratch));
        dst1 = (T*)scratch;
    }
    const int last = splits == 1 ? 1 : 0;
    hipLaunchKernelGGL((reduce_cols_narrow_kernel<OP, T, N>), dim3((unsigned)blocks), dim3(kBlock), 0, ctx->stream, src, dst1, a, R, last);
    RT_HIP(hipGetLastError());
    if (splits == 1) return RT_OK;
    // second stage: the partials are (splits, outer * inner); fold the segments in order (mean divides by the original count)
    const uint64_t inner2 = outer * inner;
    if (merge_few_outputs<OP, T>(ctx, dst1, out, inner2, (uint32_t)splits, R)) { RT_HIP(hipGetLastError()); return RT_OK; }
    const uint64_t tiles2 = (inner2 + RT_WAVE - 1) / RT_WAVE;
    hipLaunchKernelGGL((reduce_cols_kernel<OP, T, 1>), dim3((unsigned)tiles2), dim3(kBlock), 0, ctx->stream, dst1, out, (uint64_t)splits, inner2, (uint64_t)1,
                       (uint32_t)tiles2, 1u, (uint64_t)splits, R, 1);
    RT_HIP(hipGetLastError());
    return RT_OK;
}

template <int OP, class T>
int32_t reduce_typed(rt_ctx* ctx, const T* src, T* out, uint64_t outer, uint64_t R, uint64_t inner) {
    if (outer == 0 || inner == 0) return RT_OK;
    if (OP == RT_R_MEAN && !is_flt<T>::value && R == 0) return rt_fail(RT_E_ARITH, "reduce: integer mean over an empty axis divides by zero");
    // an axis of one element: every output is its own input, whatever the outer and inner dims -- one run of outer * inner elements
    if (R == 1 && outer > 1) { inner *= outer; outer = 1; }
    if (inner == 1) return rows_stage<OP, T>(ctx, src, out, outer, R, R, true);
    constexpr int N = 16 / sizeof(T);
    // Which kernel: measured on MI355X over 1 GiB of f32 (sum), TB/s -- rows of 8 / 32 / 100 / 256 elements 4.8 / 5.2 / 5.4 / 5.7;
    // columns with inner 3 / 17 / 100 5.0 / 5.0 / 4.8; (65536, 64, 64) 6.4; (2^20, 4, 64) 5.4.  One lane or one wave per short row
    // gave 0.3-2.3, lanes along a narrow inner 0.2-1.2.
    // short reduced axis: a lane per output vector.  Also for slabs of at most 8 KiB with up to 256 rows, which leave a block of the
    // narrow-column kernel too little to do ((262144, 64, 16) f32: 0.35 -> 0.61 of peak; from 16 KiB on the narrow kernel wins)
    // A short reduced axis goes to a lane per output vector, many small slabs with a few columns through LDS (see RowsTileArgs).  Where
    // both apply, the lane-per-vector form when the rows of a slab are whole 128-byte lines, or at most four of them of 32 elements
    // and more (f32 sum over (.., 4, 64): 0.85 of peak against 0.82; over (.., 8, 12): 0.41 against 0.79).  Slabs of more than 8 KiB are
    // streamed by a block each (sum over (67108, 2000, 2) f32: 0.82 against 0.72 through LDS).
    // An axis of up to four elements is an elementwise pass over `inner` lanes wide: any inner.
    const bool short_ok = (R <= 32 || (R <= 256 && R * inner * sizeof(T) <= 8192)) && (inner <= 1024 || R <= 4);
    const bool slab_ok = inner <= 128 && R >= 2 && R * inner * sizeof(T) <= 8192 && outer >= 1024;
    const bool prefer_short = short_ok && ((inner * sizeof(T)) % 128 == 0 || (R <= 4 && inner >= 32));
    if (slab_ok && !prefer_short) return tile_launch<OP, T>(ctx, src, out, outer, R, inner, R);
    if (short_ok) {
        const bool v = inner >= (uint64_t)N;                                    // rows may start at any element and have any length
        const uint64_t ivecs = v ? (inner + N - 1) / N : inner;
        if (ivecs < (1ull << 31) && outer * ivecs < (1ull << 31)) {
            const uint64_t nvec_out = outer * ivecs;
            const uint64_t blocks = (nvec_out + kBlock - 1) / kBlock;
            if (v) hipLaunchKernelGGL((reduce_cols_short_kernel<OP, T, N>), dim3((unsigned)blocks), dim3(kBlock), 0, ctx->stream, src, out, (uint32_t)R, inner,
                                      (uint32_t)ivecs, make_fastdiv((uint32_t)ivecs), nvec_out, R);
            else hipLaunchKernelGGL((reduce_cols_short_kernel<OP, T, 1>), dim3((unsigned)blocks), dim3(kBlock), 0, ctx->stream, src, out, (uint32_t)R, inner,
                                    (uint32_t)ivecs, make_fastdiv((uint32_t)ivecs), nvec_out, R);
            RT_HIP(hipGetLastError());
            return RT_OK;
        }
    }
    if (inner < 128 && R >= 64 && R < (1ull << 32) && outer < (1ull << 20)) return cols_narrow<OP, T>(ctx, src, out, outer, R, inner);
    // one 16-byte vector of columns per lane whatever the alignment of the rows (1 GiB f32 sum over axis 0 with 32767 columns:
    // 0.307 ms with one column per lane, 0.17 ms with unaligned vectors)
    const bool vec = inner >= (uint64_t)N;
    if (vec) return cols_launch<OP, T, N>(ctx, src, out, outer, R, inner, R, true);
    return cols_launch<OP, T, 1>(ctx, src, out, outer, R, inner, R, true);
}

// Wrapping sums and products have the same bits for a signed integer and the unsigned one of its width: one instantiation serves both.
template <class T> struct wrap_twin { typedef T type; };
template <> struct wrap_twin<int8_t> { typedef uint8_t type; };
template <> struct wrap_twin<int16_t> { typedef uint16_t type; };
template <> struct wrap_twin<int32_t> { typedef uint32_t type; };
template <> struct wrap_twin<int64_t> { typedef uint64_t type; };

template <class T>
int32_t reduce_ops(rt_ctx* ctx, int op, const void* src, void* out, uint64_t outer, uint64_t R, uint64_t inner) {
    typedef typename wrap_twin<T>::type W;
    switch (op) {
        case RT_R_SUM: return reduce_typed<RT_R_SUM, W>(ctx, (const W*)src, (W*)out, outer, R, inner);
        case RT_R_PROD: return reduce_typed<RT_R_PROD, W>(ctx, (const W*)src, (W*)out, outer, R, inner);
        case RT_R_MAX: return reduce_typed<RT_R_MAX, T>(ctx, (const T*)src, (T*)out, outer, R, inner);
        case RT_R_MIN: return reduce_typed<RT_R_MIN, T>(ctx, (const T*)src, (T*)out, outer, R, inner);
        case RT_R_MEAN: return reduce_typed<RT_R_MEAN, T>(ctx, (const T*)src, (T*)out, outer, R, inner);
    }
    return rt_fail(RT_E_INVALID, "reduce: op 0x%x is not a reduction op code with valid flags", op);
}

int32_t reduce_any(rt_ctx* ctx, int dtype, int op, const void* src, void* out, uint64_t outer, uint64_t R, uint64_t inner) {
    switch (dtype) {
        case RT_U8: return reduce_ops<uint8_t>(ctx, op, src, out, outer, R, inner);
        case RT_I8: return reduce_ops<int8_t>(ctx, op, src, out, outer, R, inner);
        case RT_U16: return reduce_ops<uint16_t>(ctx, op, src, out, outer, R, inner);
        case RT_I16: return reduce_ops<int16_t>(ctx, op, src, out, outer, R, inner);
        case RT_U32: return reduce_ops<uint32_t>(ctx, op, src, out, outer, R, inner);
        case RT_I32: return reduce_ops<int32_t>(ctx, op, src, out, outer, R, inner);
        case RT_U64: return reduce_ops<uint64_t>(ctx, op, src, out, outer, R, inner);
        case RT_I64: return reduce_ops<int64_t>(ctx, op, src, out, outer, R, inner);
        case RT_F32: return reduce_ops<float>(ctx, op, src, out, outer, R, inner);
        case RT_F64: return reduce_ops<double>(ctx, op, src, out, outer, R, inner);
    }
    return rt_fail(RT_E_DTYPE, "reduce: dtype code %d is not reducible (f32/f64 in the reference, 8..64-bit integers added here)", dtype);
}

}  // namespace

// check_reduce_flat, backend/remote/server.rs:375-380
int32_t rt_check_reduce_flat(uint64_t src_len, const void* src, const void* dst, uint64_t dst_len, uint64_t start, uint64_t len) {
    if (start > src_len || len > src_len - start)
        return rt_fail(RT_E_OUT_OF_BOUNDS, "reduction source: elements %llu..%llu of a buffer with %llu elements",
                       (unsigned long long)start, (unsigned long long)(start + len), (unsigned long long)src_len);
    if (dst_len == 0) return rt_fail(RT_E_OUT_OF_BOUNDS, "reduction output buffer is empty");
    if (!dst || (!src && len)) return rt_fail(RT_E_INVALID, "reduce: null buffer");
    return RT_OK;
}

// check_reduce_nd, backend/remote/server.rs:327-373
int32_t rt_check_reduce_nd(uint64_t src_len, const void* src, uint64_t offset, int32_t rank, const uint64_t* shape, const int64_t* strides,
                           const void* dst, uint64_t dst_len, int32_t dim, uint64_t* outer_out, uint64_t* inner_out, bool* run) {
    *run = false;
    if (rank < 1 || rank > RT_MAX_INPUT_RANK || !shape || !strides) return rt_fail(RT_E_INVALID, "reduce: bad rank %d or null shape", rank);
    if (dim < 0 || dim >= rank) return rt_fail(RT_E_INVALID, "reduction dim %d out of range for rank %d", dim, rank);
    unsigned __int128 size = 1, outer = 1, inner = 1;
    for (int i = 0; i < rank; ++i) {
        size *= shape[i];
        if (i < dim) outer *= shape[i];
        if (i > dim) inner *= shape[i];
        if (size > (unsigned __int128)INT64_MAX || outer > (unsigned __int128)INT64_MAX || inner > (unsigned __int128)INT64_MAX) {
            bool has_zero = false;
            for (int j = 0; j < rank; ++j) has_zero = has_zero || shape[j] == 0;
            if (!has_zero) return rt_fail(RT_E_INVALID, "reduction source shape has too many elements");
            size = outer = inner = 0;
            break;
        }
    }
    if (outer * inner == 0) return RT_OK;                      // no outputs: the kernel must not run
    int64_t expected = 1;
    for (int d = rank - 1; d >= 0; --d) {
        if (shape[d] > 1 && strides[d] != expected)
            return rt_fail(RT_E_WRONG_DIMS, "Reduction over non-contiguous tensors is not implemented yet.");
        expected *= (int64_t)shape[d];
    }
    if (offset > src_len || (uint64_t)size > src_len - offset)
        return rt_fail(RT_E_OUT_OF_BOUNDS, "reduction source of %llu elements at offset %llu exceeds buffer of %llu",
                       (unsigned long long)size, (unsigned long long)offset, (unsigned long long)src_len);
    if ((unsigned __int128)dst_len < outer * inner)
        return rt_fail(RT_E_OUT_OF_BOUNDS, "reduction output needs %llu elements, buffer has %llu", (unsigned long long)(outer * inner),
                       (unsigned long long)dst_len);
    if (!dst || !src) return rt_fail(RT_E_INVALID, "reduce: null buffer");
    *outer_out = (uint64_t)outer;
    *inner_out = (uint64_t)inner;
    *run = true;
    return RT_OK;
}

static int32_t reduce_dispatch(rt_ctx* ctx, int dtype, int op, const void* src, void* out, uint64_t outer, uint64_t R, uint64_t inner) {
    const int code = op & 0xff;
    if (code == RT_R_ARGMAX || code == RT_R_ARGMIN)
        return rt_fail(RT_E_INVALID, "reduce: argmax / argmin produce indices, use rt_argmax_flat / rt_argmax_nd");
    if (code == RT_R_VARIANCE || code == RT_R_LOGSUMEXP || code == RT_R_NORM) return rt_reduce_stat(ctx, dtype, op, src, out, outer, R, inner);
    return reduce_any(ctx, dtype, op, src, out, outer, R, inner);
}

// For other translation units (the fused training-step passes): fold `rows` contiguous rows of R elements, or the R rows of an
// (R, inner) matrix; caller holds ctx->mu.
int32_t rt_reduce_rows(rt_ctx* ctx, int dtype, int op, const void* src, void* out, uint64_t rows, uint64_t R) {
    return reduce_dispatch(ctx, dtype, op, src, out, rows, R, 1);
}
int32_t rt_reduce_cols(rt_ctx* ctx, int dtype, int op, const void* src, void* out, uint64_t R, uint64_t inner) {
    return reduce_dispatch(ctx, dtype, op, src, out, 1, R, inner);
}

extern "C" int32_t rt_reduce_flat(rt_ctx* ctx, int32_t dtype, int32_t op, const void* src, uint64_t src_len, void* dst, uint64_t dst_len,
                                  uint64_t start, uint64_t len) {
    RT_TRY(rt_ctx_enter(ctx));
    int es = rt_elem_size(dtype);
    if (!es) return rt_fail(RT_E_DTYPE, "reduce: unknown dtype code %d", dtype);
    RT_TRY(rt_check_reduce_flat(src_len, src, dst, dst_len, start, len));
    CtxGuard g(ctx);
    return reduce_dispatch(ctx, dtype, op, (const char*)src + start * es, dst, 1, len, 1);
}

extern "C" int32_t rt_reduce_nd(rt_ctx* ctx, int32_t dtype, int32_t op, const void* src, uint64_t src_len, uint64_t offset, int32_t rank,
                                const uint64_t* shape, const int64_t* strides, void* dst, uint64_t dst_len, int32_t dim) {
    RT_TRY(rt_ctx_enter(ctx));
    int es = rt_elem_size(dtype);
    if (!es) return rt_fail(RT_E_DTYPE, "reduce: unknown dtype code %d", dtype);
    uint64_t outer = 0, inner = 0;
    bool run = false;
    RT_TRY(rt_check_reduce_nd(src_len, src, offset, rank, shape, strides, dst, dst_len, dim, &outer, &inner, &run));
    if (!run) return RT_OK;
    CtxGuard g(ctx);
    return reduce_dispatch(ctx, dtype, op, (const char*)src + offset * es, dst, outer, shape[dim], inner);
}

// ---- the entry point that allocates nothing ------------------------------------------------------------------------------------
// rt_reduce_nd with the partial results of a split reduction in a workspace that is part of the library's device image instead of
// device memory allocated on demand, for callers that cannot allocate (HIP graph capture, serving loops, harnesses that forbid
// hipMalloc).  `scratch` below is a host-side stand-in for the device array, not a device address: the address on each device
// is fetched with hipGetSymbolAddress, with that device current, when the first context on that device is created, and only that
// pointer is ever handed to a kernel.  The entry point itself makes no runtime query.
// Nothing in the workspace has to start at zero: every partial that the second stage reads was written by the first stage of the
// same call.  All calls on one device share the workspace, so calls that overlap on one device (two contexts, two streams) race.
constexpr size_t kStaticScratchBytes = RT_STATIC_SCRATCH_BYTES;
static __device__ __align__(256) unsigned char scratch[kStaticScratchBytes];
constexpr int kMaxDevices = 64;
static std::mutex g_static_mu;
static void* g_static_ptr[kMaxDevices] = {};

int32_t rt_static_scratch_init(int device, void** out) {
    *out = nullptr;
    if (device < 0 || device >= kMaxDevices) return RT_OK;          // such a context has no workspace; the entry point refuses it
    std::lock_guard<std::mutex> lk(g_static_mu);
    if (!g_static_ptr[device]) {
        void* p = nullptr;
        RT_HIP(hipGetSymbolAddress(&p, HIP_SYMBOL(scratch)));          // this device's copy of the array (the device is current)
        g_static_ptr[device] = p;
    }
    *out = g_static_ptr[device];
    return RT_OK;
}

extern "C" int32_t rt_reduce_nd_static(rt_ctx* ctx, int32_t dtype, int32_t op, const void* src, uint64_t src_len, uint64_t offset, int32_t rank,
                                       const uint64_t* shape, const int64_t* strides, void* dst, uint64_t dst_len, int32_t dim) {
    RT_TRY(rt_ctx_enter(ctx));
    int es = rt_elem_size(dtype);
    if (!es) return rt_fail(RT_E_DTYPE, "reduce: unknown dtype code %d", dtype);
    if (!ctx->static_scratch) return rt_fail(RT_E_INVALID, "reduce: device index %d is beyond the %d this entry point keeps a workspace for", ctx->device, kMaxDevices);
    uint64_t outer = 0, inner = 0;
    bool run = false;
    RT_TRY(rt_check_reduce_nd(src_len, src, offset, rank, shape, strides, dst, dst_len, dim, &outer, &inner, &run));
    if (!run) return RT_OK;
    CtxGuard g(ctx);
    ctx->fixed_scratch = ctx->static_scratch;
    ctx->fixed_scratch_bytes = kStaticScratchBytes;
    ctx->fixed_only = true;
    const int32_t st = reduce_dispatch(ctx, dtype, op, (const char*)src + offset * es, dst, outer, shape[dim], inner);
    ctx->fixed_only = false;
    return st;
}
