// Batched matrix product dst[b] = lhs[b] (m x k) * rhs[b] (k x n), dst row-major and contiguous from element 0.
// Replaces BackendMatMul::matmul (backend/mod.rs:474-485; Cpu: backend/cpu.rs:725-951 -- OpenBLAS gemm for f32/f64, a
// triple loop `sum += a * b` for every other dtype).  Operand checks are those of the reference's remote server
// (backend/remote/server.rs:299-334, 605-636).
//
//   f32 / f64 : rocBLAS gemm_strided_batched (MFMA), reached through dlopen on first use so that the library itself has no
//               link-time dependency on it; row-major operands are handed over as their column-major transposes, the same
//               trick the Cpu backend plays on OpenBLAS (cpu.rs:756-821).
//   the rest  : an LDS-tiled kernel, 64 x 64 outputs per 256-lane block, 4 x 4 per lane, k in ascending order with the
//               reference's element arithmetic (wrapping integers, OR/AND for boolean): bit-exact with the Cpu loop.  It also
//               serves f32/f64 when rocBLAS cannot be loaded or a leading dimension is one BLAS does not accept.
//
// Bounds: the float path is MFMA-bound (2*b*m*n*k flops against 157.3 / 78.6 TFLOP/s for f32 / f64); the integer path is
// bound by the vector ALU (one multiply-add per k per output).
#include "rt_broadcast_common.h"

#include <dlfcn.h>
#include <mutex>

using namespace rtb;

namespace {

// ---- generic tiled kernel ------------------------------------------------------------------------------------------------
constexpr int kMT = 64, kNT = 64, kKT = 16, kMBlock = 256;

struct MatArgs {
    uint32_t m, n, k;
    int64_t a_rs, a_cs, a_bs;      // lhs strides: row, column, batch (elements)
    int64_t b_rs, b_cs, b_bs;      // rhs
    uint32_t mtiles, ntiles;
};

template <class T> __device__ __forceinline__ T mat_zero() { return T{}; }

template <class T>
__global__ __launch_bounds__(kMBlock) void matmul_tiled_kernel(const T* __restrict__ A, const T* __restrict__ B, T* __restrict__ C, MatArgs a) {
    __shared__ T As[kKT][kMT + 1];
    __shared__ T Bs[kKT][kNT + 1];
    uint32_t blk = blockIdx.x;
    const uint32_t nt = blk % a.ntiles;
    blk /= a.ntiles;
    const uint32_t mt = blk % a.mtiles;
    const uint32_t batch = blk / a.mtiles;
    const T* Ab = A + (int64_t)batch * a.a_bs;
    const T* Bb = B + (int64_t)batch * a.b_bs;
    T* Cb = C + (uint64_t)batch * a.m * a.n;
    const uint32_t i0 = mt * kMT, j0 = nt * kNT;
    const uint32_t tx = threadIdx.x % 16, ty = threadIdx.x / 16;      // lane's outputs: rows ty*4.., columns tx*4..
    T acc[4][4];
#pragma unroll
    for (int r = 0; r < 4; ++r)
#pragma unroll
        for (int c = 0; c < 4; ++c) acc[r][c] = mat_zero<T>();

    for (uint32_t kk = 0; kk < a.k; kk += kKT) {
        // 16 x 64 elements of each operand, 4 per lane; out-of-range elements read as zero
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            const uint32_t idx = threadIdx.x + e * kMBlock;          // 0..1023
            {
                // lhs: lanes run along k when columns are unit-stride (row-major), along rows otherwise
                const bool k_fast = a.a_cs == 1;
                const uint32_t kq = k_fast ? idx % kKT : idx / kMT;
                const uint32_t iq = k_fast ? idx / kKT : idx % kMT;
                const uint32_t gi = i0 + iq, gk = kk + kq;
                T v = mat_zero<T>();
                if (gi < a.m && gk < a.k) v = Ab[(int64_t)gi * a.a_rs + (int64_t)gk * a.a_cs];
                As[kq][iq] = v;
            }
            {
                const bool j_fast = a.b_cs == 1;
                const uint32_t kq = j_fast ? idx / kNT : idx % kKT;
                const uint32_t jq = j_fast ? idx % kNT : idx / kKT;
                const uint32_t gj = j0 + jq, gk = kk + kq;
                T v = mat_zero<T>();
                if (gj < a.n && gk < a.k) v = Bb[(int64_t)gk * a.b_rs + (int64_t)gj * a.b_cs];
                Bs[kq][jq] = v;
            }
        }
        __syncthreads();
#pragma unroll
        for (int q = 0; q < kKT; ++q) {
            T av[4], bv[4];
#pragma unroll
            for (int r = 0; r < 4; ++r) av[r] = As[q][ty * 4 + r];
#pragma unroll
            for (int c = 0; c < 4; ++c) bv[c] = Bs[q][tx * 4 + c];
#pragma unroll
            for (int r = 0; r < 4; ++r)
#pragma unroll
                for (int c = 0; c < 4; ++c) acc[r][c] = bin_apply<RT_ADD, T>(acc[r][c], bin_apply<RT_MUL, T>(av[r], bv[c]));   // sum += a * b
        }
        __syncthreads();
    }
#pragma unroll
    for (int r = 0; r < 4; ++r) {
        const uint32_t gi = i0 + ty * 4 + r;
        if (gi >= a.m) continue;
#pragma unroll
        for (int c = 0; c < 4; ++c) {
            const uint32_t gj = j0 + tx * 4 + c;
            if (gj < a.n) Cb[(uint64_t)gi * a.n + gj] = acc[r][c];
        }
    }
}

struct Operand {
    int64_t rs, cs, bs;    // row, column, batch stride
    uint64_t offset;
};

template <class T>
int32_t matmul_tiled(rt_ctx* ctx, const void* lhs, const Operand& L, const void* rhs, const Operand& R, void* dst, uint64_t b, uint64_t m, uint64_t k,
                     uint64_t n) {
    if (m >= (1ull << 31) || n >= (1ull << 31) || k >= (1ull << 31)) return rt_fail(RT_E_INVALID, "matmul: a matrix dim of 2^31 or more");
    MatArgs a;
    a.m = (uint32_t)m; a.n = (uint32_t)n; a.k = (uint32_t)k;
    a.a_rs = L.rs; a.a_cs = L.cs; a.a_bs = L.bs;
    a.b_rs = R.rs; a.b_cs = R.cs; a.b_bs = R.bs;
    a.mtiles = (uint32_t)((m + kMT - 1) / kMT);
    a.ntiles = (uint32_t)((n + kNT - 1) / kNT);
    const uint64_t blocks = b * a.mtiles * a.ntiles;
    if (blocks >= (1ull << 31)) return rt_fail(RT_E_INVALID, "matmul: too many output tiles for one launch");
    hipLaunchKernelGGL((matmul_tiled_kernel<T>), dim3((unsigned)blocks), dim3(kMBlock), 0, ctx->stream, (const T*)lhs + L.offset, (const T*)rhs + R.offset,
                       (T*)dst, a);
    RT_HIP(hipGetLastError());
    return RT_OK;
}

// ---- rocBLAS through dlopen ------------------------------------------------------------------------------------------------
// Minimal declarations of the five entry points used (rocblas/rocblas-functions.h): rocblas_int is int32_t, rocblas_stride
// int64_t, rocblas_operation_none = 111, rocblas_operation_transpose = 112, status 0 = success.
typedef void* rb_handle;
typedef int (*rb_create_t)(rb_handle*);
typedef int (*rb_destroy_t)(rb_handle);
typedef int (*rb_set_stream_t)(rb_handle, hipStream_t);
typedef int (*rb_sgemm_sb_t)(rb_handle, int, int, int32_t, int32_t, int32_t, const float*, const float*, int32_t, int64_t, const float*, int32_t, int64_t,
                             const float*, float*, int32_t, int64_t, int32_t);
typedef int (*rb_dgemm_sb_t)(rb_handle, int, int, int32_t, int32_t, int32_t, const double*, const double*, int32_t, int64_t, const double*, int32_t, int64_t,
                             const double*, double*, int32_t, int64_t, int32_t);
constexpr int kRbNone = 111, kRbTrans = 112;

struct RocBlas {
    void* lib = nullptr;
    rb_create_t create = nullptr;
    rb_destroy_t destroy = nullptr;
    rb_set_stream_t set_stream = nullptr;
    rb_sgemm_sb_t sgemm = nullptr;
    rb_dgemm_sb_t dgemm = nullptr;
    bool ok = false;
};

RocBlas& rocblas() {
    static RocBlas rb;
    static std::once_flag once;
    std::call_once(once, [] {
        const char* names[] = {"librocblas.so.5", "librocblas.so", "/opt/rocm/lib/librocblas.so"};
        for (const char* nm : names) {
            rb.lib = dlopen(nm, RTLD_NOW | RTLD_LOCAL);
            if (rb.lib) break;
        }
        if (!rb.lib) return;
        rb.create = (rb_create_t)dlsym(rb.lib, "rocblas_create_handle");
        rb.destroy = (rb_destroy_t)dlsym(rb.lib, "rocblas_destroy_handle");
        rb.set_stream = (rb_set_stream_t)dlsym(rb.lib, "rocblas_set_stream");
        rb.sgemm = (rb_sgemm_sb_t)dlsym(rb.lib, "rocblas_sgemm_strided_batched");
        rb.dgemm = (rb_dgemm_sb_t)dlsym(rb.lib, "rocblas_dgemm_strided_batched");
        rb.ok = rb.create && rb.destroy && rb.set_stream && rb.sgemm && rb.dgemm;
    });
    return rb;
}

// one rocBLAS handle per context, bound to the context's stream; created under ctx->mu
int32_t blas_handle(rt_ctx* ctx, rb_handle* out) {
    RocBlas& rb = rocblas();
    if (!rb.ok) return RT_E_INVALID;
    if (!ctx->blas) {
        rb_handle h = nullptr;
        if (rb.create(&h) != 0 || !h) return RT_E_HIP;
        if (rb.set_stream(h, ctx->stream) != 0) { rb.destroy(h); return RT_E_HIP; }
        ctx->blas = h;
        ctx->blas_destroy = rb.destroy;
    }
    *out = ctx->blas;
    return RT_OK;
}

// Can BLAS take this operand?  A leading dimension must be at least the extent of the unit-stride dim (and >= 1).
bool blas_ld_ok(int64_t ld, uint64_t unit_extent) { return ld >= 1 && (uint64_t)ld >= unit_extent && ld < (1ll << 31); }

template <class T>
int32_t matmul_float(rt_ctx* ctx, const void* lhs, const Operand& L, int lc, const void* rhs, const Operand& R, int rc, void* dst, uint64_t b, uint64_t m,
                     uint64_t k, uint64_t n) {
    // row-major dst (m x n) is the column-major n x m matrix dst^T = rhs^T * lhs^T.  A row-major operand *is* its transpose in
    // column-major terms (no-trans, ld = row stride); a column-major one has to be transposed (trans, ld = column stride).
    const int64_t lda = lc == RT_ROW_MAJOR ? L.rs : L.cs;
    const int64_t ldb = rc == RT_ROW_MAJOR ? R.rs : R.cs;
    const bool fits = m < (1ull << 31) && n < (1ull << 31) && k < (1ull << 31) && b < (1ull << 31) &&
                      blas_ld_ok(lda, lc == RT_ROW_MAJOR ? k : m) && blas_ld_ok(ldb, rc == RT_ROW_MAJOR ? n : k) &&
                      (lc == RT_ROW_MAJOR ? L.cs == 1 : L.rs == 1) && (rc == RT_ROW_MAJOR ? R.cs == 1 : R.rs == 1);
    rb_handle h = nullptr;
    if (!fits || blas_handle(ctx, &h) != RT_OK) return matmul_tiled<T>(ctx, lhs, L, rhs, R, dst, b, m, k, n);
    RocBlas& rb = rocblas();
    const T one = 1, zero = 0;
    const T* A = (const T*)lhs + L.offset;
    const T* B = (const T*)rhs + R.offset;
    const int ta = rc == RT_ROW_MAJOR ? kRbNone : kRbTrans;      // first BLAS operand is rhs
    const int tb = lc == RT_ROW_MAJOR ? kRbNone : kRbTrans;
    int st;
    if constexpr (std::is_same<T, float>::value)
        st = rb.sgemm(h, ta, tb, (int32_t)n, (int32_t)m, (int32_t)k, &one, B, (int32_t)ldb, R.bs, A, (int32_t)lda, L.bs, &zero, (T*)dst, (int32_t)n,
                      (int64_t)(m * n), (int32_t)b);
    else
        st = rb.dgemm(h, ta, tb, (int32_t)n, (int32_t)m, (int32_t)k, &one, B, (int32_t)ldb, R.bs, A, (int32_t)lda, L.bs, &zero, (T*)dst, (int32_t)n,
                      (int64_t)(m * n), (int32_t)b);
    if (st != 0) return rt_fail(RT_E_HIP, "matmul: rocblas gemm_strided_batched returned status %d", st);
    return RT_OK;
}

// check_matmul_operand, backend/remote/server.rs:299-334
int32_t check_operand(const char* what, uint64_t offset, int rank, const uint64_t* shape, const int64_t* strides, int contiguity, uint64_t batches,
                      uint64_t rows, uint64_t cols, uint64_t len, Operand* out) {
    if (rank < 2 || rank > RT_MAX_INPUT_RANK || !shape || !strides) return rt_fail(RT_E_INVALID, "%s: matmul operands need rank >= 2", what);
    if (shape[rank - 2] != rows || shape[rank - 1] != cols)
        return rt_fail(RT_E_INVALID, "%s: expected a %llux%llu matrix, got %llux%llu", what, (unsigned long long)rows, (unsigned long long)cols,
                       (unsigned long long)shape[rank - 2], (unsigned long long)shape[rank - 1]);
    unsigned __int128 bp = 1;
    for (int i = 0; i < rank - 2; ++i) {
        bp *= shape[i];
        if (bp > (unsigned __int128)UINT64_MAX) break;
    }
    if (bp != (unsigned __int128)batches) return rt_fail(RT_E_INVALID, "%s: batch dims do not multiply to %llu", what, (unsigned long long)batches);
    const int64_t rs = strides[rank - 2], cs = strides[rank - 1];
    bool unit_ok = false;
    if (contiguity == RT_ROW_MAJOR) unit_ok = cs == 1 || cols <= 1;
    else if (contiguity == RT_COLUMN_MAJOR) unit_ok = rs == 1 || rows <= 1;
    if (!unit_ok || rs < 0 || cs < 0)
        return rt_fail(RT_E_INVALID, "%s: strides (%lld, %lld) do not match layout code %d", what, (long long)rs, (long long)cs, contiguity);
    const int64_t bs = rank > 2 ? strides[rank - 3] : 0;
    bool collapsible = true;
    for (int d = 0; d + 3 < rank; ++d)
        collapsible = collapsible && (shape[d] <= 1 || strides[d] == strides[d + 1] * (int64_t)shape[d + 1]);
    if (bs < 0 || !collapsible) return rt_fail(RT_E_INVALID, "%s: batch dims must be collapsible into one", what);
    const uint64_t as_shape[3] = {batches, rows, cols};
    const int64_t as_strides[3] = {bs, rs, cs};
    uint64_t count = 0;
    RT_TRY(rt_check_extent(what, offset, 3, as_shape, as_strides, len, &count));
    out->rs = rs; out->cs = cs; out->bs = bs; out->offset = offset;
    return RT_OK;
}

__global__ void matmul_zero_kernel(uint8_t* p, size_t bytes) {
    size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i < bytes) p[i] = 0;
}

}  // namespace

extern "C" int32_t rt_matmul(rt_ctx* ctx, int32_t dtype,
                             const void* lhs, uint64_t lhs_len, uint64_t lhs_offset, int32_t lhs_rank, const uint64_t* lhs_shape, const int64_t* lhs_strides,
                             int32_t lhs_contiguity,
                             const void* rhs, uint64_t rhs_len, uint64_t rhs_offset, int32_t rhs_rank, const uint64_t* rhs_shape, const int64_t* rhs_strides,
                             int32_t rhs_contiguity,
                             void* dst, uint64_t dst_len, uint64_t b, uint64_t m, uint64_t k, uint64_t n) {
    RT_TRY(rt_ctx_enter(ctx));
    const int es = rt_elem_size(dtype);
    if (!es) return rt_fail(RT_E_DTYPE, "matmul: unknown dtype code %d", dtype);
    if (lhs_rank != rhs_rank) return rt_fail(RT_E_INVALID, "matmul operands must have the same rank (%d and %d)", lhs_rank, rhs_rank);
    Operand L, R;
    RT_TRY(check_operand("matmul lhs", lhs_offset, lhs_rank, lhs_shape, lhs_strides, lhs_contiguity, b, m, k, lhs_len, &L));
    RT_TRY(check_operand("matmul rhs", rhs_offset, rhs_rank, rhs_shape, rhs_strides, rhs_contiguity, b, k, n, rhs_len, &R));
    unsigned __int128 out = (unsigned __int128)b * m;
    if (out <= (unsigned __int128)UINT64_MAX) out *= n;
    if (out > (unsigned __int128)dst_len) return rt_fail(RT_E_INVALID, "matmul dst has %llu elements, needs b*m*n", (unsigned long long)dst_len);
    if (out == 0) return RT_OK;
    if (!dst || ((!lhs || !rhs) && k)) return rt_fail(RT_E_INVALID, "matmul: null buffer");
    if (dst == lhs || dst == rhs) return rt_fail(RT_E_INVALID, "matmul destination must not alias an input");
    CtxGuard g(ctx);
    if (k == 0) {                                            // empty sums: all outputs are zero
        const size_t bytes = (size_t)out * es;
        hipLaunchKernelGGL(matmul_zero_kernel, dim3((unsigned)((bytes + 255) / 256)), dim3(256), 0, ctx->stream, (uint8_t*)dst, bytes);
        RT_HIP(hipGetLastError());
        return RT_OK;
    }
    switch (dtype) {
        case RT_F32: return matmul_float<float>(ctx, lhs, L, lhs_contiguity, rhs, R, rhs_contiguity, dst, b, m, k, n);
        case RT_F64: return matmul_float<double>(ctx, lhs, L, lhs_contiguity, rhs, R, rhs_contiguity, dst, b, m, k, n);
        // sum += a * b on two's-complement integers does not depend on signedness: one instantiation per width
        case RT_U8: case RT_I8: return matmul_tiled<uint8_t>(ctx, lhs, L, rhs, R, dst, b, m, k, n);
        case RT_U16: case RT_I16: return matmul_tiled<uint16_t>(ctx, lhs, L, rhs, R, dst, b, m, k, n);
        case RT_U32: case RT_I32: return matmul_tiled<uint32_t>(ctx, lhs, L, rhs, R, dst, b, m, k, n);
        case RT_U64: case RT_I64: return matmul_tiled<uint64_t>(ctx, lhs, L, rhs, R, dst, b, m, k, n);
        case RT_U128: case RT_I128: return matmul_tiled<u128_t>(ctx, lhs, L, rhs, R, dst, b, m, k, n);
        case RT_BOOL: return matmul_tiled<boolean_t>(ctx, lhs, L, rhs, R, dst, b, m, k, n);
    }
    return rt_fail(RT_E_DTYPE, "matmul: unknown dtype code %d", dtype);
}
