// Row-major copy of a view whose contiguous pieces are short in src, in dst or in both: N-d tiles through LDS (rt_permute.h has the
// plan and the index arithmetic).  Used by rt_gather (TensorView::owned / contiguous, core/tensor.rs:299-325).
#include "rt_broadcast_common.h"
#include "rt_permute.h"

using namespace rtb;
using namespace rtp;

namespace {

template <class T, int W, int V>
__global__ __launch_bounds__(kPBlock) void permute_tile_kernel(const T* __restrict__ src, T* __restrict__ dst, PermArgs a) {
    extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
    const PermTables tb = pm_tables(a, smem, (uint32_t)sizeof(T));
    const uint32_t block = pm_remap(a, blockIdx.x);
    const PermBlock b = pm_block(a, block);
    pm_stage0<T>(a, block, threadIdx.x, tb);
    __syncthreads();
    pm_stage1<T, V>(src, a, b, threadIdx.x, smem, tb);
    __syncthreads();
    pm_stage2<T, W>(dst, a, b, threadIdx.x, smem, tb, PmCopy{});
}

// Stage 2 of a binary op whose other input lies in memory like dst: that input's piece is loaded at the piece's own byte offset and
// combined with the piece of the tile.
template <class T, int OP> struct PmBinary {
    const unsigned char* other;              // the other input at the tile's origin
    uint32_t tile_is_left;                   // the permuted input is the op's left operand
    template <class VT> __device__ __forceinline__ VT fetch(uint32_t off) const { return __builtin_nontemporal_load(reinterpret_cast<const VT*>(other + off)); }
    template <class VT> __device__ __forceinline__ VT combine(const VT& x, const VT& o) const {
        constexpr int W = (int)(sizeof(VT) / sizeof(T));
        VT out;
#pragma unroll
        for (int i = 0; i < W; ++i) {
            const T xe = pm_lane<VT, T, W>(x, i), oe = pm_lane<VT, T, W>(o, i);
            const T r = tile_is_left ? bin_apply<OP, T>(xe, oe) : bin_apply<OP, T>(oe, xe);
            if constexpr (W == 1) out = r; else out[i] = r;
        }
        return out;
    }
};

template <class T, int OP, int W, int V>
__global__ __launch_bounds__(kPBlock) void permute_bin_kernel(const T* __restrict__ xt, const T* xo, T* dst, PermArgs a, uint32_t tile_is_left) {
    extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
    const PermTables tb = pm_tables(a, smem, (uint32_t)sizeof(T));
    const uint32_t block = pm_remap(a, blockIdx.x);
    const PermBlock b = pm_block(a, block);
    pm_stage0<T>(a, block, threadIdx.x, tb);
    __syncthreads();
    pm_stage1<T, V>(xt, a, b, threadIdx.x, smem, tb);
    __syncthreads();
    const PmBinary<T, OP> f = {reinterpret_cast<const unsigned char*>(xo + b.dbase), tile_is_left};
    pm_stage2<T, W>(dst, a, b, threadIdx.x, smem, tb, f);
}

}  // namespace

namespace rtb {

template <class T>
bool permute_try(rt_ctx* ctx, const NdDesc& dsc, uint64_t count, const T* src, T* dst, int32_t* status, bool force) {
    constexpr uint32_t N = 16 / sizeof(T);
    if (dsc.rank < 2 || count >= (1ull << 31)) return false;
    PermArgs a;
    uint64_t blocks = 0;
    // Where this kernel is the faster one, from timing permuted, reversed and stepped views of 256 MiB in every element size against
    // the row, flat and transposing kernels (fractions of the HBM peak, 2 x the view's bytes per copy):
    //   * src steps by 64 bytes or more along dst's inner dim and has a unit-stride dim somewhere else -- the permuted views proper.
    //     4- and 8-byte elements: the median goes from 0.57 to 0.71, the lowest tenth from 0.22 to 0.48 (unit-stride dims of 2 .. 7
    //     elements, dst rows of a few elements: 0.05 before).  1- and 2-byte elements only where the transposing tile kernel does
    //     not apply (it packs four or two of them per LDS word; this kernel moves them one by one);
    //   * src is unit-stride along dst's inner dim but the rows are shorter than 256 bytes (64 bytes for 1- and 2-byte elements):
    //     a slice or a reversed outer dim over short rows, where a tile gathers many rows per block.
    // A smaller step along dst's inner dim (an interleaved source, every second element) keeps whole lines in use from one dst row to
    // the next and stays with the row kernels; a view with no unit-stride dim at all gains nothing from a tile.
    const int rank = dsc.rank;
    const int64_t is1 = dsc.stride[0][rank - 1], mag1 = is1 < 0 ? -is1 : is1;
    const uint64_t row_bytes = (uint64_t)dsc.shape[rank - 1] * sizeof(T);
    bool unit_dim = false, transposable = false;
    for (int k = 0; k < rank; ++k) {
        const bool unit = dsc.stride[0][k] == 1 || dsc.stride[0][k] == -1;
        unit_dim = unit_dim || unit;
        transposable = transposable || (unit && k < rank - 1 && dsc.shape[k] >= 16);
    }
    // (the tile kernel takes 1- and 2-byte elements from dst rows of 128 elements on, a quarter of its tile's columns)
    const bool tile_kernel_fits = transposable && mag1 > 1 && dsc.shape[rank - 1] >= 128;
    bool wanted;
    if (sizeof(T) >= 4)
        wanted = (mag1 > 1 && unit_dim && (uint64_t)mag1 * sizeof(T) >= 64) || (mag1 == 1 && row_bytes < 256 && (is1 == 1 || row_bytes >= 64));
    else
        wanted = (mag1 > 1 && unit_dim && (uint64_t)mag1 * sizeof(T) >= 64 && !tile_kernel_fits) || (is1 == 1 && row_bytes < 64);
    if (!wanted && !force) return false;
    const T* sp = src + dsc.offset[0];
    T* dp = dst + dsc.offset[2];
    if (!rt_permute_plan(dsc.rank, dsc.shape, dsc.stride[0], dsc.stride[2], (uint32_t)sizeof(T), &a, &blocks, kPTileBytes, reinterpret_cast<uintptr_t>(sp) % 128 == 0)) return false;
    uint32_t w = rt_permute_store_width(a, N);
    while (w > 1 && (reinterpret_cast<uintptr_t>(dp) % (w * sizeof(T))) != 0) w >>= 1;
    constexpr uint32_t kWord = sizeof(T) < 4 ? 4 / sizeof(T) : 1;      // a 32-bit store of 1- and 2-byte elements
    const uint32_t v = rt_permute_load_width(a, N) == N ? N : 1u;
    w = w == N ? N : (kWord > 1 && w >= kWord ? kWord : 1u);
    rt_permute_set_widths(&a, v, w);
    dim3 grid((unsigned)blocks), blk(kPBlock);
    const uint32_t lds = rt_permute_lds_bytes(a, (uint32_t)sizeof(T));
    if (lds > 64u * 1024u) return false;                           // (the plan stays below 52 KiB: a 40 KiB tile and 12 KiB of tables)
    auto go = [&](auto wc) {
        constexpr int W = decltype(wc)::value;
        if (v == N) hipLaunchKernelGGL((permute_tile_kernel<T, W, (int)N>), grid, blk, lds, ctx->stream, sp, dp, a);
        else hipLaunchKernelGGL((permute_tile_kernel<T, W, 1>), grid, blk, lds, ctx->stream, sp, dp, a);
    };
    if (w == N) go(std::integral_constant<int, (int)N>{});
    else if (kWord > 1 && w >= kWord) go(std::integral_constant<int, (int)kWord>{});
    else go(std::integral_constant<int, 1>{});
    hipError_t e = hipGetLastError();
    *status = e == hipSuccess ? RT_OK : rt_hip_fail(e, "gather (permuting tile kernel) launch");
    return true;
}

template <class T, int OP>
bool permute_bin_try(rt_ctx* ctx, const NdDesc& dsc, uint64_t count, const T* xt, const T* xo, T* dst, bool tile_is_left, int32_t* status) {
    constexpr uint32_t N = 16 / sizeof(T);
    if (dsc.rank < 2 || count >= (1ull << 31)) return false;
    PermArgs a;
    uint64_t blocks = 0;
    const T* sp = xt + dsc.offset[0];
    if (!rt_permute_plan(dsc.rank, dsc.shape, dsc.stride[0], dsc.stride[2], (uint32_t)sizeof(T), &a, &blocks, kPTileBytes, reinterpret_cast<uintptr_t>(sp) % 128 == 0)) return false;
    uint32_t w = rt_permute_store_width(a, N);
    while (w > 1 && ((reinterpret_cast<uintptr_t>(dst) | reinterpret_cast<uintptr_t>(xo)) % (w * sizeof(T))) != 0) w >>= 1;
    w = w == N ? N : 1u;
    const uint32_t v = rt_permute_load_width(a, N) == N ? N : 1u;
    // With single-element accesses on both sides -- to the permuted input, and to dst and the other input -- the two-pass form is the
    // faster one (rows of 2905 f32 out of a unit-stride dim of 7: 0.32 of peak here, 0.37 there); with vectors on either side this one
    // is (rows of 299593 out of contiguous pieces of 224: 0.61 against 0.45).
    if (w != N && v != N) return false;
    rt_permute_set_widths(&a, v, w);
    const uint32_t lds = rt_permute_lds_bytes(a, (uint32_t)sizeof(T));
    if (lds > 64u * 1024u) return false;
    dim3 grid((unsigned)blocks), blk(kPBlock);
    const uint32_t left = tile_is_left ? 1u : 0u;
    if (w == N && v == N) hipLaunchKernelGGL((permute_bin_kernel<T, OP, (int)N, (int)N>), grid, blk, lds, ctx->stream, sp, xo, dst, a, left);
    else if (w == N) hipLaunchKernelGGL((permute_bin_kernel<T, OP, (int)N, 1>), grid, blk, lds, ctx->stream, sp, xo, dst, a, left);
    else hipLaunchKernelGGL((permute_bin_kernel<T, OP, 1, (int)N>), grid, blk, lds, ctx->stream, sp, xo, dst, a, left);
    hipError_t e = hipGetLastError();
    *status = e == hipSuccess ? RT_OK : rt_hip_fail(e, "broadcast (permuting tile kernel) launch");
    return true;
}

#define RT_PERM_BIN(T, OP) template bool permute_bin_try<T, OP>(rt_ctx*, const NdDesc&, uint64_t, const T*, const T*, T*, bool, int32_t*);
RT_PERM_BIN(float, RT_ADD) RT_PERM_BIN(float, RT_SUB) RT_PERM_BIN(float, RT_MUL) RT_PERM_BIN(float, RT_DIV)
RT_PERM_BIN(double, RT_ADD) RT_PERM_BIN(double, RT_SUB) RT_PERM_BIN(double, RT_MUL) RT_PERM_BIN(double, RT_DIV)
RT_PERM_BIN(uint32_t, RT_ADD) RT_PERM_BIN(uint32_t, RT_SUB) RT_PERM_BIN(uint32_t, RT_MUL)
RT_PERM_BIN(uint64_t, RT_ADD) RT_PERM_BIN(uint64_t, RT_SUB) RT_PERM_BIN(uint64_t, RT_MUL)
#undef RT_PERM_BIN

template bool permute_try<uint8_t>(rt_ctx*, const NdDesc&, uint64_t, const uint8_t*, uint8_t*, int32_t*, bool);
template bool permute_try<uint16_t>(rt_ctx*, const NdDesc&, uint64_t, const uint16_t*, uint16_t*, int32_t*, bool);
template bool permute_try<uint32_t>(rt_ctx*, const NdDesc&, uint64_t, const uint32_t*, uint32_t*, int32_t*, bool);
template bool permute_try<uint64_t>(rt_ctx*, const NdDesc&, uint64_t, const uint64_t*, uint64_t*, int32_t*, bool);

}  // namespace rtb
