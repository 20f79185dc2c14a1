// Fused passes of the broadcast / reduce training step  y = relu(x + bias), loss = mean_l1_loss(y, t), backward to d(bias)
// (ops/broadcast/l1.rs:49-84; grad/backwards.rs:148-161 backwards_l1, 229-239 backwards_relu, 516-538 inverse_broadcast_gradient).
// The reference's engine issues this as one backend call per arithmetic step with a full-size temporary between each two of
// them; the three entry points here do the same IEEE operations per element, in the same order, in three passes:
//   rt_fused_bias_relu          y = relu(x + bias)                                           reads x, writes y            (2 N s)
//   rt_fused_l1_forward         gmap = sign(y - t) / N,  loss = sum |y - t| / N              reads y, t, writes gmap      (3 N s)
//   rt_fused_l1_relu_backward   dbias[j] = sum_i [y_ij > 0] * (gmap_ij * up)                 reads gmap, y                (2 N s)
// and, without ever storing the gradient map (it is a temporary of the tape, not a result), in two:
//   rt_fused_bias_relu_l1       y = relu(x + bias),  loss = sum |y - t| / N                  reads x, t, writes y         (3 N s)
//   rt_fused_l1_relu_backward_t dbias[j] = sum_i [y_ij > 0] * ((sign(y_ij - t_ij) / N) * up) reads y, t                   (2 N s)
// Every element-wise result (y, gmap, and the products that are summed) is bit for bit what the separate ops give; the two sums are
// tree sums, held to the same tolerance as the reductions (1e-5 / 1e-12 of sum |x|).  f32 and f64 (the autograd engine is bounded on
// WeightValue, core/value.rs:61).  The ReLU gradient map is not stored: [pre > 0] == [relu(pre) > 0].
#include "rt_common.h"

namespace {

template <class T> struct alignas(16) Vec16 { T e[16 / sizeof(T)]; };
constexpr int kFBlock = 256;
constexpr int kFWaves = kFBlock / RT_WAVE;

template <class T> __device__ __forceinline__ T relu_of(T x) { return x > (T)0 ? x : (T)0; }                       // backend/cpu.rs:650-657
template <class T> __device__ __forceinline__ T sign_of(T x) { return x < (T)0 ? (T)-1 : (x > (T)0 ? (T)1 : (T)0); }  // backend/cpu.rs:548-557
__device__ __forceinline__ float abs_of(float x) { return fabsf(x); }
__device__ __forceinline__ double abs_of(double x) { return fabs(x); }

// ---- y = relu(x + bias) ------------------------------------------------------------------------------------------------------------
// One 16-byte vector of y per lane, walked in the tiled order (see TileMap); the bias row (cols / N vectors) is read through the cache.
template <class T>
__global__ __launch_bounds__(kFBlock) void fused_bias_relu_kernel(const T* __restrict__ x, const T* __restrict__ bias, T* __restrict__ y, uint32_t nvec,
                                                                  uint32_t row_vecs, FastDiv32 row_div, TileMap m) {
    constexpr int N = 16 / sizeof(T);
    size_t vi;
    if (!rt_tile_index(m, blockIdx.x, kFBlock, threadIdx.x, nvec, &vi)) return;
    const uint32_t v = (uint32_t)vi;
    Vec16<T> a = rt_ld16_nt(reinterpret_cast<const Vec16<T>*>(x) + v);
    const uint32_t c = v - fd_div(v, row_div) * row_vecs;
    const Vec16<T> b = rt_ld16(reinterpret_cast<const Vec16<T>*>(bias) + c);
#pragma unroll
    for (int j = 0; j < N; ++j) a.e[j] = relu_of<T>(a.e[j] + b.e[j]);
    rt_st16_nt(reinterpret_cast<Vec16<T>*>(y) + v, a);
}

// ---- gmap = sign(y - t) / N, partial sums of |y - t| -----------------------------------------------------------------------------------
template <class T>
__global__ __launch_bounds__(kFBlock) void fused_l1_forward_kernel(const T* __restrict__ y, const T* __restrict__ t, T* __restrict__ gmap, T* __restrict__ part,
                                                                   uint32_t nvec, T count, TileMap m) {
    constexpr int N = 16 / sizeof(T);
    __shared__ T sv[kFWaves];
    size_t vi;
    T acc = (T)0;
    if (rt_tile_index(m, blockIdx.x, kFBlock, threadIdx.x, nvec, &vi)) {
        const Vec16<T> a = rt_ld16_nt(reinterpret_cast<const Vec16<T>*>(y) + vi);
        const Vec16<T> b = rt_ld16_nt(reinterpret_cast<const Vec16<T>*>(t) + vi);
        Vec16<T> g;
#pragma unroll
        for (int j = 0; j < N; ++j) {
            const T diff = a.e[j] - b.e[j];                       // lhs - target
            g.e[j] = sign_of<T>(diff) / count;                    // sign, then / T::from_usize(N)   (l1.rs:29-36, 58-60)
            acc = acc + abs_of(diff);                             // abs_inplace, then mean
        }
        rt_st16_nt(reinterpret_cast<Vec16<T>*>(gmap) + vi, g);
    }
#pragma unroll
    for (int d = RT_WAVE / 2; d >= 1; d >>= 1) acc = acc + __shfl_down(acc, d, RT_WAVE);
    const int lane = threadIdx.x & (RT_WAVE - 1), w = threadIdx.x / RT_WAVE;
    if (lane == 0) sv[w] = acc;
    __syncthreads();
    if (threadIdx.x == 0) {
        T s = sv[0];
#pragma unroll
        for (int k = 1; k < kFWaves; ++k) s = s + sv[k];
        part[blockIdx.x] = s;
    }
}

template <class T> __global__ void fused_divide_kernel(T* p, T count) { *p = *p / count; }

// ---- y = relu(x + bias) and the partial sums of |y - t| in one pass ----------------------------------------------------------------------
template <class T>
__global__ __launch_bounds__(kFBlock) void fused_bias_relu_l1_kernel(const T* __restrict__ x, const T* __restrict__ bias, const T* __restrict__ t,
                                                                     T* __restrict__ y, T* __restrict__ part, uint32_t nvec, uint32_t row_vecs,
                                                                     FastDiv32 row_div, TileMap m) {
    constexpr int N = 16 / sizeof(T);
    __shared__ T sv[kFWaves];
    size_t vi;
    T acc = (T)0;
    if (rt_tile_index(m, blockIdx.x, kFBlock, threadIdx.x, nvec, &vi)) {
        const uint32_t v = (uint32_t)vi;
        Vec16<T> a = rt_ld16_nt(reinterpret_cast<const Vec16<T>*>(x) + v);
        const Vec16<T> tt = rt_ld16_nt(reinterpret_cast<const Vec16<T>*>(t) + v);
        const uint32_t c = v - fd_div(v, row_div) * row_vecs;
        const Vec16<T> b = rt_ld16(reinterpret_cast<const Vec16<T>*>(bias) + c);
#pragma unroll
        for (int j = 0; j < N; ++j) {
            a.e[j] = relu_of<T>(a.e[j] + b.e[j]);
            acc = acc + abs_of(a.e[j] - tt.e[j]);
        }
        rt_st16_nt(reinterpret_cast<Vec16<T>*>(y) + v, a);
    }
#pragma unroll
    for (int d = RT_WAVE / 2; d >= 1; d >>= 1) acc = acc + __shfl_down(acc, d, RT_WAVE);
    const int lane = threadIdx.x & (RT_WAVE - 1), w = threadIdx.x / RT_WAVE;
    if (lane == 0) sv[w] = acc;
    __syncthreads();
    if (threadIdx.x == 0) {
        T s = sv[0];
#pragma unroll
        for (int k = 1; k < kFWaves; ++k) s = s + sv[k];
        part[blockIdx.x] = s;
    }
}

// ---- dbias[j] = sum_i [y_ij > 0] * (gmap_ij * up) ------------------------------------------------------------------------------------
// The shape of the column reduction: lanes along the columns (one 16-byte vector each), the four waves of a block take interleaved
// rows, four rows in flight per wave, LDS combine; the rows are split over `splits` blocks per column tile and a second launch (the
// ordinary column sum) folds the partials.  out index: seg * cols + column.
// FROM_TARGET: `gmap` holds the target instead, and the gradient map's element sign(y - t) / count is formed in registers.
template <class T, bool FROM_TARGET>
__global__ __launch_bounds__(kFBlock) void fused_backward_cols_kernel(const T* __restrict__ gmap, const T* __restrict__ y, const T* __restrict__ up,
                                                                      T* __restrict__ out, uint64_t rows, uint64_t cols, uint32_t tiles, uint64_t seglen,
                                                                      T count) {
    constexpr int N = 16 / sizeof(T);
    constexpr int U = 4;
    const uint32_t tile = blockIdx.x % tiles, seg = blockIdx.x / tiles;
    const uint32_t tx = threadIdx.x & (RT_WAVE - 1), ty = threadIdx.x / RT_WAVE;
    const uint64_t col = ((uint64_t)tile * RT_WAVE + tx) * N;
    const bool active = col < cols;                                // cols is a multiple of N
    const uint64_t begin = (uint64_t)seg * seglen;
    uint64_t end = begin + seglen;
    if (end > rows) end = rows;
    const T u = up[0];
    T acc[N];
#pragma unroll
    for (int j = 0; j < N; ++j) acc[j] = (T)0;
    auto fold = [&](const Vec16<T>& g, const Vec16<T>& a) {
#pragma unroll
        for (int j = 0; j < N; ++j) {
            T gm = g.e[j];
            if constexpr (FROM_TARGET) gm = sign_of<T>(a.e[j] - g.e[j]) / count;   // l1.rs:29-36, 58-60: sign(lhs - target) / N
            const T g1 = gm * u;                                   // backwards_l1: grad_map * upstream
            const T g2 = (a.e[j] > (T)0 ? (T)1 : (T)0) * g1;       // backwards_relu: relu map * upstream
            acc[j] = acc[j] + g2;
        }
    };
    if (active) {
        const T* gp = gmap + col;
        const T* yp = y + col;
        uint64_t k = begin + ty;
        for (; k + (uint64_t)(U - 1) * kFWaves < end; k += (uint64_t)U * kFWaves) {
            Vec16<T> g[U], a[U];
#pragma unroll
            for (int q = 0; q < U; ++q) {
                g[q] = rt_ld16_nt(reinterpret_cast<const Vec16<T>*>(gp + (k + (uint64_t)q * kFWaves) * cols));
                a[q] = rt_ld16_nt(reinterpret_cast<const Vec16<T>*>(yp + (k + (uint64_t)q * kFWaves) * cols));
            }
            __builtin_amdgcn_sched_barrier(0);                    // all loads of a trip before the first use
#pragma unroll
            for (int q = 0; q < U; ++q) fold(g[q], a[q]);
        }
        for (; k < end; k += kFWaves)
            fold(rt_ld16_nt(reinterpret_cast<const Vec16<T>*>(gp + k * cols)), rt_ld16_nt(reinterpret_cast<const Vec16<T>*>(yp + k * cols)));
    }
    __shared__ T sv[kFWaves][RT_WAVE][N];
#pragma unroll
    for (int j = 0; j < N; ++j) sv[ty][tx][j] = acc[j];
    __syncthreads();
    if (ty == 0 && active) {
        T* q = out + (uint64_t)seg * cols + col;
#pragma unroll
        for (int j = 0; j < N; ++j) {
            T s = acc[j];
#pragma unroll
            for (int w = 1; w < kFWaves; ++w) s = s + sv[w][tx][j];
            q[j] = s;
        }
    }
}

int32_t check_float(const char* what, int dtype) {
    if (dtype != RT_F32 && dtype != RT_F64) return rt_fail(RT_E_DTYPE, "%s: f32 / f64 only (the autograd engine is bounded on WeightValue)", what);
    return RT_OK;
}
bool aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15) == 0; }
// An output may be the very same run as an input of its own length (every lane reads its vector before it writes it); any other
// overlap would let block order decide the result.
bool bad_overlap(const void* out, uint64_t out_n, const void* in, uint64_t in_n, int es) {
    if (out == in && out_n == in_n) return false;
    return rt_spans_meet(rt_run_span(out, es, 0, out_n), rt_run_span(in, es, 0, in_n));
}

template <class T>
int32_t bias_relu_typed(rt_ctx* ctx, const void* x, const void* bias, void* y, uint64_t rows, uint64_t cols) {
    constexpr uint64_t N = 16 / sizeof(T);
    const uint32_t nvec = (uint32_t)(rows * cols / N), row_vecs = (uint32_t)(cols / N);
    const TileMap m = rt_make_tilemap(y, nvec, kFBlock);
    hipLaunchKernelGGL((fused_bias_relu_kernel<T>), dim3((unsigned)rt_tilemap_blocks(m, nvec, kFBlock)), dim3(kFBlock), 0, ctx->stream, (const T*)x,
                       (const T*)bias, (T*)y, nvec, row_vecs, make_fastdiv(row_vecs), m);
    RT_HIP(hipGetLastError());
    return RT_OK;
}

template <class T>
int32_t l1_forward_typed(rt_ctx* ctx, int dtype, const void* y, const void* t, void* gmap, void* loss, uint64_t n) {
    constexpr uint64_t N = 16 / sizeof(T);
    const uint32_t nvec = (uint32_t)(n / N);
    const TileMap m = rt_make_tilemap(gmap, nvec, kFBlock);
    const size_t blocks = rt_tilemap_blocks(m, nvec, kFBlock);
    void* part = nullptr;                                          // one partial per block; a cached block of the allocator, returned below
    RT_TRY(rt_alloc_bytes(ctx, blocks * sizeof(T), &part));
    const T count = (T)(float)n;                                   // WeightValue::from_usize goes through f32 (core/value.rs:54-56)
    hipLaunchKernelGGL((fused_l1_forward_kernel<T>), dim3((unsigned)blocks), dim3(kFBlock), 0, ctx->stream, (const T*)y, (const T*)t, (T*)gmap, (T*)part, nvec,
                       count, m);
    hipError_t e = hipGetLastError();
    int32_t st = e == hipSuccess ? RT_OK : rt_hip_fail(e, "fused l1 forward launch");
    if (st == RT_OK) st = rt_reduce_rows(ctx, dtype, RT_R_SUM, part, loss, 1, blocks);
    if (st == RT_OK) {
        hipLaunchKernelGGL((fused_divide_kernel<T>), dim3(1), dim3(1), 0, ctx->stream, (T*)loss, count);
        e = hipGetLastError();
        if (e != hipSuccess) st = rt_hip_fail(e, "fused l1 forward launch");
    }
    (void)rt_free_locked(ctx, part);                               // stream ordered: the next user runs after the kernels above
    return st;
}

template <class T>
int32_t bias_relu_l1_typed(rt_ctx* ctx, int dtype, const void* x, const void* bias, const void* t, void* y, void* loss, uint64_t rows, uint64_t cols) {
    constexpr uint64_t N = 16 / sizeof(T);
    const uint64_t n = rows * cols;
    const uint32_t nvec = (uint32_t)(n / N), row_vecs = (uint32_t)(cols / N);
    const TileMap m = rt_make_tilemap(y, nvec, kFBlock);
    const size_t blocks = rt_tilemap_blocks(m, nvec, kFBlock);
    void* part = nullptr;
    RT_TRY(rt_alloc_bytes(ctx, blocks * sizeof(T), &part));
    const T count = (T)(float)n;
    hipLaunchKernelGGL((fused_bias_relu_l1_kernel<T>), dim3((unsigned)blocks), dim3(kFBlock), 0, ctx->stream, (const T*)x, (const T*)bias, (const T*)t, (T*)y,
                       (T*)part, nvec, row_vecs, make_fastdiv(row_vecs), m);
    hipError_t e = hipGetLastError();
    int32_t st = e == hipSuccess ? RT_OK : rt_hip_fail(e, "fused bias relu l1 launch");
    if (st == RT_OK) st = rt_reduce_rows(ctx, dtype, RT_R_SUM, part, loss, 1, blocks);
    if (st == RT_OK) {
        hipLaunchKernelGGL((fused_divide_kernel<T>), dim3(1), dim3(1), 0, ctx->stream, (T*)loss, count);
        e = hipGetLastError();
        if (e != hipSuccess) st = rt_hip_fail(e, "fused bias relu l1 launch");
    }
    (void)rt_free_locked(ctx, part);
    return st;
}

template <class T>
int32_t backward_typed(rt_ctx* ctx, int dtype, const void* gmap, const void* y, const void* up, void* dbias, uint64_t rows_all, uint64_t cols_out, bool from_target) {
    constexpr uint64_t N = 16 / sizeof(T);
    // Short rows are regrouped as in the column reduction (rt_reduce.hip, cols_launch): g consecutive rows are read as one row of
    // g * cols columns, and the g partial sums per column join the partials of the split in the column sum that follows.
    const uint64_t g = rt_cols_regroup(rows_all, cols_out * sizeof(T), (uint64_t)ctx->num_cus * 2);
    const uint64_t rows = rows_all / g, cols = cols_out * g;
    const uint64_t tiles = (cols / N + RT_WAVE - 1) / RT_WAVE;
    const uint64_t want = (uint64_t)ctx->num_cus * 2;              // two resident blocks per CU, as the column reduction
    uint64_t splits = 1;
    if (tiles < want) {
        splits = (want + tiles - 1) / tiles;
        if (splits > rows / 64) splits = rows / 64;
        if (splits < 1) splits = 1;
        if (splits > 1024) splits = 1024;
    }
    uint64_t seglen = (rows + splits - 1) / splits;
    seglen = (seglen + 4 * kFWaves - 1) / (4 * kFWaves) * (4 * kFWaves);
    splits = (rows + seglen - 1) / seglen;
    if (tiles * splits >= (1ull << 31)) return rt_fail(RT_E_INVALID, "fused backward: too many blocks for one launch");
    void* part = dbias;
    const bool staged = splits > 1 || g > 1;
    if (staged) RT_TRY(rt_alloc_bytes(ctx, (size_t)(splits * cols) * sizeof(T), &part));
    const T count = (T)(float)(rows * cols);                       // WeightValue::from_usize goes through f32 (core/value.rs:54-56)
    if (from_target)
        hipLaunchKernelGGL((fused_backward_cols_kernel<T, true>), dim3((unsigned)(tiles * splits)), dim3(kFBlock), 0, ctx->stream, (const T*)gmap, (const T*)y,
                           (const T*)up, (T*)part, rows, cols, (uint32_t)tiles, seglen, count);
    else
        hipLaunchKernelGGL((fused_backward_cols_kernel<T, false>), dim3((unsigned)(tiles * splits)), dim3(kFBlock), 0, ctx->stream, (const T*)gmap, (const T*)y,
                           (const T*)up, (T*)part, rows, cols, (uint32_t)tiles, seglen, count);
    hipError_t e = hipGetLastError();
    int32_t st = e == hipSuccess ? RT_OK : rt_hip_fail(e, "fused backward launch");
    if (staged) {
        if (st == RT_OK) st = rt_reduce_cols(ctx, dtype, RT_R_SUM, part, dbias, splits * g, cols_out);
        (void)rt_free_locked(ctx, part);
    }
    return st;
}

}  // namespace

extern "C" int32_t rt_fused_bias_relu(rt_ctx* ctx, int32_t dtype, const void* x, uint64_t x_len, const void* bias, uint64_t bias_len, void* y, uint64_t y_len,
                                      uint64_t rows, uint64_t cols) {
    RT_TRY(rt_ctx_enter(ctx));
    RT_TRY(check_float("fused bias relu", dtype));
    const uint64_t N = 16 / (uint64_t)rt_elem_size(dtype);
    if (cols == 0 || (rows && (rows > (uint64_t)INT64_MAX / cols || rows * cols / N >= (1ull << 31))))
        return rt_fail(RT_E_INVALID, "fused bias relu: %llu x %llu is empty or too long for one launch", (unsigned long long)rows, (unsigned long long)cols);
    if (rows * cols > x_len || rows * cols > y_len || cols > bias_len) return rt_fail(RT_E_OUT_OF_BOUNDS, "fused bias relu: operands shorter than rows * cols");
    if (rows == 0) return RT_OK;
    if (!x || !bias || !y) return rt_fail(RT_E_INVALID, "fused bias relu: null buffer");
    if (cols % N || !aligned16(x) || !aligned16(bias) || !aligned16(y))
        return rt_fail(RT_E_INVALID, "fused bias relu: needs 16-byte aligned operands and whole vectors per row (issue the separate ops instead)");
    {
        const int es = rt_elem_size(dtype);
        if (bad_overlap(y, rows * cols, x, rows * cols, es) || rt_spans_meet(rt_run_span(y, es, 0, rows * cols), rt_run_span(bias, es, 0, cols)))
            return rt_fail(RT_E_INVALID, "fused bias relu: the output overlaps an input");
    }
    CtxGuard g(ctx);
    return dtype == RT_F32 ? bias_relu_typed<float>(ctx, x, bias, y, rows, cols) : bias_relu_typed<double>(ctx, x, bias, y, rows, cols);
}

extern "C" int32_t rt_fused_l1_forward(rt_ctx* ctx, int32_t dtype, const void* y, uint64_t y_len, const void* target, uint64_t target_len, void* gmap,
                                       uint64_t gmap_len, void* loss, uint64_t loss_len, uint64_t n) {
    RT_TRY(rt_ctx_enter(ctx));
    RT_TRY(check_float("fused l1 forward", dtype));
    const uint64_t N = 16 / (uint64_t)rt_elem_size(dtype);
    if (n == 0 || n >= (1ull << 31) * N) return rt_fail(RT_E_INVALID, "fused l1 forward: %llu elements is empty or too long for one launch", (unsigned long long)n);
    if (n > y_len || n > target_len || n > gmap_len || loss_len < 1) return rt_fail(RT_E_OUT_OF_BOUNDS, "fused l1 forward: operands shorter than n");
    if (!y || !target || !gmap || !loss) return rt_fail(RT_E_INVALID, "fused l1 forward: null buffer");
    if (n % N || !aligned16(y) || !aligned16(target) || !aligned16(gmap))
        return rt_fail(RT_E_INVALID, "fused l1 forward: needs 16-byte aligned operands and a whole number of vectors (issue the separate ops instead)");
    {
        const int es = rt_elem_size(dtype);
        const ByteSpan ls = rt_run_span(loss, es, 0, 1);
        if (bad_overlap(gmap, n, y, n, es) || bad_overlap(gmap, n, target, n, es) || rt_spans_meet(ls, rt_run_span(y, es, 0, n)) ||
            rt_spans_meet(ls, rt_run_span(target, es, 0, n)) || rt_spans_meet(ls, rt_run_span(gmap, es, 0, n)))
            return rt_fail(RT_E_INVALID, "fused l1 forward: an output overlaps an input or the other output");
    }
    CtxGuard g(ctx);
    return dtype == RT_F32 ? l1_forward_typed<float>(ctx, dtype, y, target, gmap, loss, n) : l1_forward_typed<double>(ctx, dtype, y, target, gmap, loss, n);
}

extern "C" int32_t rt_fused_l1_relu_backward(rt_ctx* ctx, int32_t dtype, const void* gmap, uint64_t gmap_len, const void* y, uint64_t y_len, const void* upstream,
                                             uint64_t upstream_len, void* dbias, uint64_t dbias_len, uint64_t rows, uint64_t cols) {
    RT_TRY(rt_ctx_enter(ctx));
    RT_TRY(check_float("fused backward", dtype));
    const uint64_t N = 16 / (uint64_t)rt_elem_size(dtype);
    if (cols == 0 || rows == 0) return rt_fail(RT_E_INVALID, "fused backward: empty operand");
    if (rows > (uint64_t)INT64_MAX / cols || rows * cols > gmap_len || rows * cols > y_len || cols > dbias_len || upstream_len < 1)
        return rt_fail(RT_E_OUT_OF_BOUNDS, "fused backward: operands shorter than rows * cols");
    if (!gmap || !y || !upstream || !dbias) return rt_fail(RT_E_INVALID, "fused backward: null buffer");
    if (cols % N || !aligned16(gmap) || !aligned16(y) || !aligned16(dbias))
        return rt_fail(RT_E_INVALID, "fused backward: needs 16-byte aligned operands and whole vectors per row (issue the separate ops instead)");
    {
        const int es = rt_elem_size(dtype);
        const ByteSpan ds = rt_run_span(dbias, es, 0, cols);
        if (rt_spans_meet(ds, rt_run_span(gmap, es, 0, rows * cols)) || rt_spans_meet(ds, rt_run_span(y, es, 0, rows * cols)) ||
            rt_spans_meet(ds, rt_run_span(upstream, es, 0, 1)))
            return rt_fail(RT_E_INVALID, "fused backward: the output overlaps an input");
    }
    CtxGuard g(ctx);
    return dtype == RT_F32 ? backward_typed<float>(ctx, dtype, gmap, y, upstream, dbias, rows, cols, false)
                           : backward_typed<double>(ctx, dtype, gmap, y, upstream, dbias, rows, cols, false);
}

extern "C" int32_t rt_fused_bias_relu_l1(rt_ctx* ctx, int32_t dtype, const void* x, uint64_t x_len, const void* bias, uint64_t bias_len, const void* target,
                                         uint64_t target_len, void* y, uint64_t y_len, void* loss, uint64_t loss_len, uint64_t rows, uint64_t cols) {
    RT_TRY(rt_ctx_enter(ctx));
    RT_TRY(check_float("fused bias relu l1", dtype));
    const uint64_t N = 16 / (uint64_t)rt_elem_size(dtype);
    if (cols == 0 || rows == 0 || rows > (uint64_t)INT64_MAX / cols || rows * cols / N >= (1ull << 31))
        return rt_fail(RT_E_INVALID, "fused bias relu l1: %llu x %llu is empty or too long for one launch", (unsigned long long)rows, (unsigned long long)cols);
    const uint64_t n = rows * cols;
    if (n > x_len || n > y_len || n > target_len || cols > bias_len || loss_len < 1)
        return rt_fail(RT_E_OUT_OF_BOUNDS, "fused bias relu l1: operands shorter than rows * cols");
    if (!x || !bias || !target || !y || !loss) return rt_fail(RT_E_INVALID, "fused bias relu l1: null buffer");
    if (cols % N || !aligned16(x) || !aligned16(bias) || !aligned16(target) || !aligned16(y))
        return rt_fail(RT_E_INVALID, "fused bias relu l1: needs 16-byte aligned operands and whole vectors per row (issue the separate ops instead)");
    {
        const int es = rt_elem_size(dtype);
        const ByteSpan ys = rt_run_span(y, es, 0, n), ls = rt_run_span(loss, es, 0, 1);
        if (bad_overlap(y, n, x, n, es) || rt_spans_meet(ys, rt_run_span(target, es, 0, n)) || rt_spans_meet(ys, rt_run_span(bias, es, 0, cols)) ||
            rt_spans_meet(ls, ys) || rt_spans_meet(ls, rt_run_span(x, es, 0, n)) || rt_spans_meet(ls, rt_run_span(target, es, 0, n)) ||
            rt_spans_meet(ls, rt_run_span(bias, es, 0, cols)))
            return rt_fail(RT_E_INVALID, "fused bias relu l1: an output overlaps an input or the other output");
    }
    CtxGuard g(ctx);
    return dtype == RT_F32 ? bias_relu_l1_typed<float>(ctx, dtype, x, bias, target, y, loss, rows, cols)
                           : bias_relu_l1_typed<double>(ctx, dtype, x, bias, target, y, loss, rows, cols);
}

extern "C" int32_t rt_fused_l1_relu_backward_t(rt_ctx* ctx, int32_t dtype, const void* y, uint64_t y_len, const void* target, uint64_t target_len,
                                               const void* upstream, uint64_t upstream_len, void* dbias, uint64_t dbias_len, uint64_t rows, uint64_t cols) {
    RT_TRY(rt_ctx_enter(ctx));
    RT_TRY(check_float("fused backward", dtype));
    const uint64_t N = 16 / (uint64_t)rt_elem_size(dtype);
    if (cols == 0 || rows == 0) return rt_fail(RT_E_INVALID, "fused backward: empty operand");
    if (rows > (uint64_t)INT64_MAX / cols || rows * cols > target_len || rows * cols > y_len || cols > dbias_len || upstream_len < 1)
        return rt_fail(RT_E_OUT_OF_BOUNDS, "fused backward: operands shorter than rows * cols");
    if (!target || !y || !upstream || !dbias) return rt_fail(RT_E_INVALID, "fused backward: null buffer");
    if (cols % N || !aligned16(target) || !aligned16(y) || !aligned16(dbias))
        return rt_fail(RT_E_INVALID, "fused backward: needs 16-byte aligned operands and whole vectors per row (issue the separate ops instead)");
    {
        const int es = rt_elem_size(dtype);
        const ByteSpan ds = rt_run_span(dbias, es, 0, cols);
        if (rt_spans_meet(ds, rt_run_span(target, es, 0, rows * cols)) || rt_spans_meet(ds, rt_run_span(y, es, 0, rows * cols)) ||
            rt_spans_meet(ds, rt_run_span(upstream, es, 0, 1)))
            return rt_fail(RT_E_INVALID, "fused backward: the output overlaps an input");
    }
    CtxGuard g(ctx);
    return dtype == RT_F32 ? backward_typed<float>(ctx, dtype, target, y, upstream, dbias, rows, cols, true)
                           : backward_typed<double>(ctx, dtype, target, y, upstream, dbias, rows, cols, true);
}
