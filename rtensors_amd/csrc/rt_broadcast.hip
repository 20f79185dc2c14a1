// N-d broadcast binary kernel family: dst[c] = left[c] (op) right[c] over a shared shape, operands pre-broadcast
// (expansion = stride 0), strides signed.  Replaces Backend::broadcast (backend/mod.rs:296-309; Cpu loop
// backend/cpu.rs:292-352; the reference's CUDA kernel is K/kernels/elementwise/binary/broadcast.cu:3-55).
//
// Host side: size-1 dims are dropped, dims are flipped/sorted so that dst is walked in ascending address order, and
// adjacent dims that are mergeable in all three operands are merged (rt_collapse).  The descriptor travels in the
// kernel arguments; nothing is uploaded per call.
//
// Device side, three shapes of kernel:
//   contig : all three operands are one unit-stride run -> 16-byte accesses, 2 loads + 1 store per vector
//   rows   : dst's innermost collapsed dim is unit-stride.  A block owns a column tile of a row and loops over a
//            chosen outer dim `g`; an operand whose stride along g is 0 (the broadcast one) is loaded once and kept
//            in registers for the whole loop, so it costs no traffic per output row.  (row, chunk, tile) come from
//            blockIdx by multiply-high division on the scalar unit; no per-element index arithmetic.
//   generic: anything else, one element per lane, per-element multiply-high index decomposition.
// Algorithmic traffic: (|left|_unique + |right|_unique + N) * sizeof(T).
#include "rt_broadcast_common.h"

using namespace rtb;

namespace {

// ---- contig ---------------------------------------------------------------------------------------------------------
// One vector per lane, non-temporal loads and stores: every byte is touched exactly once.
constexpr int kCBlock2 = 256;
template <class T, int OP>
__global__ __launch_bounds__(kCBlock2) void bin_contig_kernel(const Vec16<T>* l, const Vec16<T>* r, Vec16<T>* d, size_t nvec, uint32_t head,
                                                              uint32_t tail, TileMap m, int32_t* fault) {
    __shared__ int32_t div8[uses_div8<T, OP>::value ? 256 : 1];
    if constexpr (uses_div8<T, OP>::value) {
        div8_table_init<T>(div8);
        __syncthreads();
    }
    // the `head` elements before and the `tail` elements after the aligned body (fewer than a vector each; all three operands
    // share the phase) are taken by lanes of the first and the last block instead of launches of their own
    auto edge = [&](int64_t e) {
        const T x = *(reinterpret_cast<const T*>(l) + e);
        T y = x;
        if constexpr (OP != kOpCopy) y = *(reinterpret_cast<const T*>(r) + e);
        *(reinterpret_cast<T*>(d) + e) = bin_apply<OP, T>(x, y, fault);
    };
    if (blockIdx.x == 0 && threadIdx.x < head) edge((int64_t)threadIdx.x - (int64_t)head);
    if (blockIdx.x == gridDim.x - 1 && threadIdx.x < tail) edge((int64_t)(nvec * (16 / sizeof(T))) + (int64_t)threadIdx.x);
    size_t i;
    if (!rt_tile_index(m, blockIdx.x, kCBlock2, threadIdx.x, nvec, &i)) return;     // a block owns a quarter of four pages (see TileMap)
    Vec16<T> a = rt_ld16_nt(l + i);
    Vec16<T> b;
    if constexpr (OP != kOpCopy) b = rt_ld16_nt(r + i); else b = a;
    bin_apply_vec_t<OP, T>(a, b, fault, div8);
    rt_st16_nt(d + i, a);
}

// ---- rows -------------------------------------------------------------------------------------------------------------
struct RowArgs {
    uint32_t L;                     // inner length (elements)
    uint32_t G;                     // extent of the loop dim (1 when there is none)
    uint32_t gchunk;                // loop-dim iterations owned by one block
    uint32_t nchunks;               // ceil(G / gchunk)
    uint32_t tiles;                 // column tiles per row
    uint32_t tpr;                   // lanes per row inside a block (power of two <= kRBlock)
    uint32_t lead;                  // columns [0, lead) of every row do not exist: the column origin was moved back to a line boundary
    FastDiv32 tiles_div, nchunks_div;
    int nouter;                     // remaining outer dims (loop dim and inner dim excluded), outermost first
    uint32_t oshape[RT_MAX_RANK];
    FastDiv32 odiv[RT_MAX_RANK];
    int64_t ostride[3][RT_MAX_RANK];
    int64_t gstride[3];
    int64_t istride[2];             // inner strides of left, right (dst: 1)
};

template <class T, int OP, int LM, int RM, int GU>
__global__ __launch_bounds__(256) void bin_rows_kernel(const T* l, const T* r, T* d, RowArgs a, int32_t* fault) {
    constexpr int N = 16 / sizeof(T);
    // blockIdx -> (outer index, chunk of the loop dim, column tile); all uniform, computed on the scalar unit
    uint32_t b = blockIdx.x;
    uint32_t q = fd_div(b, a.tiles_div);
    const uint32_t tile = b - q * a.tiles;
    b = q;
    q = fd_div(b, a.nchunks_div);
    const uint32_t chunk = b - q * a.nchunks;
    int64_t off3[3];
    rt_outer_offsets<3>(q, a.nouter, a.oshape, a.odiv, a.ostride, off3);
    const int64_t ol = off3[0], orr = off3[1], od = off3[2];
    const uint32_t tx = threadIdx.x & (a.tpr - 1);
    const uint32_t ty = threadIdx.x / a.tpr;
    const uint32_t gy = blockDim.x / a.tpr;
    const uint32_t c = (tile * a.tpr + tx) * N;                 // first column of this lane's vector
    if (c >= a.L) return;
    const uint32_t g_begin = chunk * a.gchunk;
    const uint32_t g_end = min(a.G, g_begin + a.gchunk);

    if (c >= a.lead && c + N <= a.L) {
        const bool l_fixed = (a.gstride[0] == 0), r_fixed = (a.gstride[1] == 0);
        // Vectors cross the control flow below as four 32-bit words: held as arrays of 1-byte elements they would be split into
        // sixteen separate registers at every select and re-packed before the store.
        typedef rt_u32x4 Raw;
        auto ldl = [&](int64_t off) { return load_raw<T, LM>(l + off, c, a.istride[0]); };
        auto ldr = [&](int64_t off) { return load_raw<T, RM>(r + off, c, a.istride[1]); };
        auto combine_store = [&](Raw x, Raw y, uint32_t g) {
            Vec16<T> xv = __builtin_bit_cast(Vec16<T>, x);
            bin_apply_vec<OP, T>(xv, __builtin_bit_cast(Vec16<T>, y), fault);
            rt_st16u_nt<T>(d + od + (int64_t)g * a.gstride[2] + c, __builtin_bit_cast(rt_u32x4, xv));
        };
        Raw lh = {}, rh = {};                                   // operands that do not move along the loop dim
        if (l_fixed) lh = ldl(ol);
        if (r_fixed) rh = ldr(orr);
        if constexpr (GU == 1) {
            // short loop (two steps per lane by default): load, combine, store
            for (uint32_t g = g_begin + ty; g < g_end; g += gy) {
                Raw x = l_fixed ? lh : ldl(ol + (int64_t)g * a.gstride[0]);
                Raw y;
                if constexpr (OP == kOpCopy) y = x;
                else y = r_fixed ? rh : ldr(orr + (int64_t)g * a.gstride[1]);
                combine_store(x, y, g);
            }
        } else {
            // long loop (an expensive operand is held in registers while the block walks the loop dim): GU steps per
            // batch, the next batch's loads issued before this batch's stores.  Loads and stores retire in issue order,
            // so a load issued after a store would wait for that store's acknowledgement.
            Raw xn[GU], yn[GU];
            auto load_batch = [&](uint32_t g0) {
#pragma unroll
                for (int u = 0; u < GU; ++u) {
                    const uint32_t g = min(g0 + u * gy, g_end - 1);
                    if (!l_fixed) xn[u] = ldl(ol + (int64_t)g * a.gstride[0]);
                    if constexpr (OP != kOpCopy) { if (!r_fixed) yn[u] = ldr(orr + (int64_t)g * a.gstride[1]); }
                }
            };
            uint32_t g0 = g_begin + ty;
            if (g0 < g_end) load_batch(g0);
            for (; g0 < g_end; g0 += gy * GU) {
                Raw x[GU], y[GU];
#pragma unroll
                for (int u = 0; u < GU; ++u) {
                    x[u] = l_fixed ? lh : xn[u];
                    if constexpr (OP == kOpCopy) y[u] = x[u]; else y[u] = r_fixed ? rh : yn[u];
                }
                if (g0 + gy * GU < g_end) load_batch(g0 + gy * GU);
#pragma unroll
                for (int u = 0; u < GU; ++u) {
                    const uint32_t g = g0 + u * gy;
                    if (g < g_end) combine_store(x[u], y[u], g);
                }
            }
        }
    } else {
        // ragged start (columns before `lead` do not exist) or end of a row: element accesses
        for (uint32_t g = g_begin + ty; g < g_end; g += gy) {
            const T* lp = l + ol + (int64_t)g * a.gstride[0];
            const T* rp = r + orr + (int64_t)g * a.gstride[1];
            T* dp = d + od + (int64_t)g * a.gstride[2];
            for (uint32_t k = max(c, a.lead); k < min(c + (uint32_t)N, a.L); ++k)
                dp[k] = bin_apply<OP, T>(lp[(int64_t)k * a.istride[0]], rp[(int64_t)k * a.istride[1]], fault);
        }
    }
}

// ---- rows, lean form ------------------------------------------------------------------------------------------------------
// The common case of the row kernel -- rows of at least 1 KiB, no gathered input, at most two outer dims besides the loop dim,
// rows not shifted to a line boundary -- with as little work per wave as possible: a 256-lane block owns the same 1 KiB piece of
// four consecutive rows, one wave per row, one vector per lane, and the next block owns the next piece of the same rows (the tiled
// order described at TileMap).  All kernel arguments are fetched in one batch, the row index is wave-uniform and every offset is
// computed on the scalar unit.  Config 3 (x (16,1,512,1024) + y (1,64,1,1024), 2 GiB out): 0.90 of peak in this shape when a
// wave's life is one load-add-store; the general kernel above spends longer decoding its descriptor than a wave may live.
struct Rows4Args {
    uint32_t L, G, tiles;
    FastDiv32 tiles_div;
    int32_t gs[3], o0s[3], o1s[3], o2s[3];   // strides of left, right, dst along the loop dim and the three outer dims (inner one first)
    FastDiv32 n1_div;                    // grid z = index along the second outer dim + its extent n1 * index along the third
    uint32_t n1;
    // block order for a long repeated row (see the kernel): 0, or tiles per group (a power of two) * chunks of four rows per band
    uint32_t group, tg_shift, band_blocks, band_chunks;
    FastDiv32 group_div, band_div;
};

// grid: x = column tile + tiles * (chunk of four rows), y = index along the inner outer dim, z = the indices along the next two outer
// dims folded into one.  Every offset inside an operand fits 32 bits (checked on the host).
// NTM: bit 0 / 1 = the left / right input is a row-wise operand that is read exactly once (no stride-0 dim): non-temporal loads.  A
// compile-time choice: two loads that differ only in the hint are merged by the compiler, and the hint is lost.
template <class T, int OP, int LM, int RM, int NTM>
__global__ __launch_bounds__(256) void bin_rows4_kernel(const T* l, const T* r, T* d, Rows4Args a, int32_t* fault) {
    constexpr int N = 16 / sizeof(T);
    __shared__ int32_t div8[uses_div8<T, OP>::value ? 256 : 1];
    if constexpr (uses_div8<T, OP>::value) {                       // before any lane leaves: every lane fills one entry
        div8_table_init<T>(div8);
        __syncthreads();
    }
    uint32_t L = a.L, G = a.G, tiles = a.tiles, tm = a.tiles_div.mul, ts = a.tiles_div.shift, group = a.group, gm = a.group_div.mul, gsh = a.group_div.shift;
    int32_t g0 = a.gs[0], g1 = a.gs[1], g2 = a.gs[2], p0 = a.o0s[0], p1 = a.o0s[1], p2 = a.o0s[2], q0 = a.o1s[0], q1 = a.o1s[1], q2 = a.o1s[2];
    int32_t r0 = a.o2s[0], r1 = a.o2s[1], r2 = a.o2s[2];
    uint32_t n1 = a.n1, nm = a.n1_div.mul, nsh = a.n1_div.shift;
    RT_PIN(r0); RT_PIN(r1); RT_PIN(r2); RT_PIN(n1); RT_PIN(nm); RT_PIN(nsh);
    RT_PIN(L); RT_PIN(G); RT_PIN(tiles); RT_PIN(tm); RT_PIN(ts); RT_PIN(group); RT_PIN(gm); RT_PIN(gsh);
    RT_PIN(g0); RT_PIN(g1); RT_PIN(g2); RT_PIN(p0); RT_PIN(p1); RT_PIN(p2); RT_PIN(q0); RT_PIN(q1); RT_PIN(q2);
    RT_TOUCH(l); RT_TOUCH(r); RT_TOUCH(d);
    uint32_t chunk, tile;
    if (group == 0) {
        chunk = (uint32_t)(((uint64_t)__umulhi(blockIdx.x, tm) + blockIdx.x) >> ts);
        tile = blockIdx.x - chunk * tiles;
    } else {
        // A row of several MiB that repeats along the loop dim.  The rows are taken in bands of `band_chunks` chunks of four rows;
        // inside a band, a group of tiles of every chunk before the next group of tiles, so that a piece of the repeated row is used
        // by all rows of the band while it is in cache.  In plain order the row is streamed from memory once per chunk of four rows.
        const uint32_t bm = a.band_div.mul, bsh = a.band_div.shift, bb = a.band_blocks, bc = a.band_chunks, tgs = a.tg_shift;
        const uint32_t band = (uint32_t)(((uint64_t)__umulhi(blockIdx.x, bm) + blockIdx.x) >> bsh);
        const uint32_t inb = blockIdx.x - band * bb;
        const uint32_t th = (uint32_t)(((uint64_t)__umulhi(inb, gm) + inb) >> gsh);
        const uint32_t rem = inb - th * group;
        chunk = band * bc + (rem >> tgs);
        tile = (th << tgs) + (rem & ((1u << tgs) - 1));
        if (tile >= tiles) return;
    }
    const uint32_t zi2 = (uint32_t)(((uint64_t)__umulhi(blockIdx.z, nm) + blockIdx.z) >> nsh);
    const int32_t i0 = (int32_t)blockIdx.y, i1 = (int32_t)(blockIdx.z - zi2 * n1), i2 = (int32_t)zi2;
    const uint32_t g = chunk * 4 + (uint32_t)__builtin_amdgcn_readfirstlane((int)(threadIdx.x >> 6));
    if (g >= G) return;
    const T* lp = l + (i2 * r0 + i1 * q0 + i0 * p0 + (int32_t)g * g0);
    const T* rp = r + (i2 * r1 + i1 * q1 + i0 * p1 + (int32_t)g * g1);
    T* dp = d + (i2 * r2 + i1 * q2 + i0 * p2 + (int32_t)g * g2);
    // a wave's vectors sit on the 128-byte line grid of dst's memory whatever the start of the row (see rt_row_tiling); the inputs
    // follow at element alignment
    const uint32_t phase = (uint32_t)((reinterpret_cast<uintptr_t>(dp) / sizeof(T)) & (uintptr_t)(128 / sizeof(T) - 1));
    const int32_t c = (int32_t)((tile * 64 + (threadIdx.x & 63)) * N) - (int32_t)phase;
    if (c >= (int32_t)L || c + (int32_t)N <= 0) return;
    if (c >= 0 && (uint32_t)c + N <= L) {
        rt_u32x4 x, y;
        if constexpr (LM == M_VEC && (NTM & 1)) x = rt_ld16u<T, true>(lp + c); else x = load_raw<T, LM>(lp, (uint32_t)c, 1);
        if constexpr (OP == kOpCopy) y = x;
        else if constexpr (RM == M_VEC && (NTM & 2)) y = rt_ld16u<T, true>(rp + c);
        else y = load_raw<T, RM>(rp, (uint32_t)c, 1);
        Vec16<T> xv = __builtin_bit_cast(Vec16<T>, x);
        bin_apply_vec_t<OP, T>(xv, __builtin_bit_cast(Vec16<T>, y), fault, div8);
        rt_st16_nt(reinterpret_cast<Vec16<T>*>(dp + c), xv);
    } else {
        // the ragged ends of a row: all loads, then all stores
        const uint32_t k0 = c < 0 ? 0u : (uint32_t)c, k1 = min((uint32_t)(c + N), L);
        T xs[N], ys[N];
#pragma unroll
        for (int j = 0; j < N; ++j) {
            const uint32_t k = min(k0 + j, k1 - 1);
            xs[j] = lp[LM == M_VEC ? k : 0];
            if constexpr (OP != kOpCopy) ys[j] = rp[RM == M_VEC ? k : 0]; else ys[j] = xs[j];
        }
#pragma unroll
        for (int j = 0; j < N; ++j)
            if (k0 + j < k1) dp[k0 + j] = bin_apply<OP, T>(xs[j], ys[j], fault);
    }
}

template <class T, int OP>
void launch_rows4(int lm, int rm, int ntm, dim3 grid, hipStream_t s, const T* l, const T* r, T* d, const Rows4Args& a, int32_t* fault) {
    const bool nl = lm == M_VEC && (ntm & 1), nr = rm == M_VEC && (ntm & 2);
#define RT_R4(LMV, RMV, NT) hipLaunchKernelGGL((bin_rows4_kernel<T, OP, LMV, RMV, NT>), grid, dim3(256), 0, s, l, r, d, a, fault)
    if (lm == M_VEC && rm == M_VEC) {
        if (nl && nr) RT_R4(M_VEC, M_VEC, 3); else if (nl) RT_R4(M_VEC, M_VEC, 1); else if (nr) RT_R4(M_VEC, M_VEC, 2); else RT_R4(M_VEC, M_VEC, 0);
    } else if (lm == M_VEC) {
        if (nl) RT_R4(M_VEC, M_BCAST, 1); else RT_R4(M_VEC, M_BCAST, 0);
    } else if (rm == M_VEC) {
        if (nr) RT_R4(M_BCAST, M_VEC, 2); else RT_R4(M_BCAST, M_VEC, 0);
    } else {
        RT_R4(M_BCAST, M_BCAST, 0);
    }
#undef RT_R4
}

// ---- generic ------------------------------------------------------------------------------------------------------------
struct GenArgs {
    int rank;
    uint32_t shape[RT_MAX_RANK];
    FastDiv32 div[RT_MAX_RANK];
    int64_t stride[3][RT_MAX_RANK];
};

constexpr int kGU = 4;          // elements in flight per lane in the generic kernel

template <class T, int OP>
__global__ __launch_bounds__(kBlock) void bin_generic_kernel(const T* l, const T* r, T* d, GenArgs a, uint32_t first, uint32_t n, int32_t* fault) {
    // a block owns kGU * kBlock consecutive elements per trip, lane t the elements t, t + kBlock, ...; all loads are issued
    // before the first store
    constexpr uint32_t span = kGU * kBlock, step = kBlock;
    for (uint64_t base = first + (uint64_t)blockIdx.x * span; base < n; base += (uint64_t)gridDim.x * span) {
        const uint32_t i = (uint32_t)base + threadIdx.x;
        int64_t od[kGU];
        T x[kGU], y[kGU];
#pragma unroll
        for (int u = 0; u < kGU; ++u) {
            uint32_t rem = min(i + u * step, n - 1);     // lanes past the end recompute the last element and do not store it
            int64_t ol = 0, orr = 0;
            od[u] = 0;
#pragma unroll
            for (int k = RT_MAX_RANK - 1; k >= 0; --k) {
                if (k < a.rank) {
                    uint32_t q = fd_div(rem, a.div[k]);
                    uint32_t c = rem - q * a.shape[k];
                    ol += (int64_t)c * a.stride[0][k];
                    orr += (int64_t)c * a.stride[1][k];
                    od[u] += (int64_t)c * a.stride[2][k];
                    rem = q;
                }
            }
            x[u] = l[ol];
            if constexpr (OP != kOpCopy) y[u] = r[orr]; else y[u] = x[u];
        }
#pragma unroll
        for (int u = 0; u < kGU; ++u)
            if (i + u * step < n) d[od[u]] = bin_apply<OP, T>(x[u], y[u], fault);
    }
}

// dst is one forward contiguous run but its rows are too short (or not 16-byte aligned) for the row kernel, e.g. (2^26, 4) + (4,)
// or rows of 1001 elements: a lane owns one 16-byte vector of dst, an input laid out like dst (LV / RV) is read with one vector
// load, any other input element by element through the index decomposition (it is a broadcast operand: its lines stay in cache).
// Operand modes of the flat kernel: F_VEC laid out like dst (one vector load), F_ROW one row of `a.shape[rank - 1]` elements
// repeated for every row (stride 1 along the last dim, 0 along the others), F_ELEM anything else.
enum FlatMode : int { F_ELEM = 0, F_VEC = 1, F_ROW = 2 };

// 16 bytes of a repeated row starting at column c0 = (first element of the vector) mod L.  Inside the row that is one 16-byte
// load from an address that is only element-aligned (the hardware runs in unaligned-access mode); a vector that wraps around the
// end of the row is put together element by element.  Without this a 1-byte row needed sixteen index decompositions per lane
// (u8 (N, 1000) + (1000,): 2.3 TB/s).
template <class T>
__device__ __forceinline__ Vec16<T> load_row_vec(const T* __restrict__ row, uint32_t first, uint32_t L, const FastDiv32& l_div) {
    constexpr uint32_t N = 16 / sizeof(T);
    uint32_t c = first - fd_div(first, l_div) * L;
    Vec16<T> y;
    if (c + N <= L) {
        __builtin_memcpy(&y, row + c, 16);
    } else if (L >= N) {
        // the vector holds the last k elements of the row and then its first N - k: two loads that stay inside the row, joined
        // by a 128-bit funnel shift (nearly every wave of a 1000-byte row has one such lane; sixteen dependent byte loads there
        // held the whole wave back)
        const uint32_t k = L - c;                                 // 1 .. N - 1
        unsigned __int128 tail, head;
        __builtin_memcpy(&tail, row + (L - N), 16);
        __builtin_memcpy(&head, row, 16);
        const unsigned __int128 both = (tail >> ((N - k) * sizeof(T) * 8)) | (head << (k * sizeof(T) * 8));
        __builtin_memcpy(&y, &both, 16);
    } else {
#pragma unroll
        for (uint32_t j = 0; j < N; ++j) {
            y.e[j] = row[c];
            c = (c + 1 == L) ? 0u : c + 1;
        }
    }
    return y;
}

template <class T, int OP, int LMODE, int RMODE>
__global__ __launch_bounds__(kRBlock) void bin_flat_kernel(const T* l, const T* r, T* d, GenArgs a, uint32_t nvec, int32_t* fault) {
    constexpr int N = 16 / sizeof(T);
    constexpr bool LE = LMODE == F_ELEM, RE = RMODE == F_ELEM && OP != kOpCopy;
    const uint32_t v = blockIdx.x * kRBlock + threadIdx.x;
    if (v >= nvec) return;
    Vec16<T> x, y;
    const uint32_t L = a.shape[a.rank - 1];
    if constexpr (LMODE == F_VEC) x = __builtin_bit_cast(Vec16<T>, rt_ld16u<T, true>(l + (size_t)v * N));     // a run like dst, from any element
    if constexpr (LMODE == F_ROW) x = load_row_vec<T>(l, v * N, L, a.div[a.rank - 1]);
    if constexpr (OP != kOpCopy) {
        if constexpr (RMODE == F_VEC) y = __builtin_bit_cast(Vec16<T>, rt_ld16u<T, true>(r + (size_t)v * N));
        if constexpr (RMODE == F_ROW) y = load_row_vec<T>(r, v * N, L, a.div[a.rank - 1]);
    }
    if constexpr (LE || RE) {
#pragma unroll
        for (int j = 0; j < N; ++j) {
            uint32_t rem = v * N + j;
            int64_t ol = 0, orr = 0;
#pragma unroll
            for (int k = RT_MAX_RANK - 1; k >= 0; --k) {
                if (k < a.rank) {
                    uint32_t q = fd_div(rem, a.div[k]);
                    uint32_t c = rem - q * a.shape[k];
                    if constexpr (LE) ol += (int64_t)c * a.stride[0][k];
                    if constexpr (RE) orr += (int64_t)c * a.stride[1][k];
                    rem = q;
                }
            }
            if constexpr (LE) x.e[j] = l[ol];
            if constexpr (RE) y.e[j] = r[orr];
        }
    }
    if constexpr (OP == kOpCopy) y = x;
    bin_apply_vec<OP, T>(x, y, fault);
    rt_st16_nt(reinterpret_cast<Vec16<T>*>(d) + v, x);
}

// dst and one input are the same forward contiguous run, the other input is one row of L elements repeated for every row
// (bias add): a lane owns one 16-byte vector of dst, reads the streamed input at the same position and the row at position
// v mod (L / N) -- the shape of the plain copy kernel plus one cached load.
template <class T, int OP, bool ROW_IS_LEFT>
__global__ __launch_bounds__(kCBlock2) void bin_flat_row_kernel(const T* flat, const T* __restrict__ row, T* d, uint32_t nvec, uint32_t row_vecs,
                                                                FastDiv32 row_div, TileMap m, int32_t* fault) {
    // `flat` and `d` may be the same buffer (in-place form): every lane reads its vector before it writes it
    size_t vi;
    if (!rt_tile_index(m, blockIdx.x, kCBlock2, threadIdx.x, nvec, &vi)) return;
    const uint32_t v = (uint32_t)vi;
    Vec16<T> x = rt_ld16_nt(reinterpret_cast<const Vec16<T>*>(flat) + v);
    Vec16<T> y;
    if (row_vecs == 0) {                                          // the "row" is a single element (tensor op one-element tensor)
        const T e = row[0];
#pragma unroll
        for (int j = 0; j < (int)(16 / sizeof(T)); ++j) y.e[j] = e;
    } else {
        const uint32_t c = v - fd_div(v, row_div) * row_vecs;
        y = rt_ld16(reinterpret_cast<const Vec16<T>*>(row) + c);
    }
    if constexpr (ROW_IS_LEFT) { bin_apply_vec<OP, T>(y, x, fault); rt_st16_nt(reinterpret_cast<Vec16<T>*>(d) + v, y); }
    else { bin_apply_vec<OP, T>(x, y, fault); rt_st16_nt(reinterpret_cast<Vec16<T>*>(d) + v, x); }
}

template <class T, int OP>
__global__ __launch_bounds__(kBlock) void bin_generic64_kernel(const T* l, const T* r, T* d, NdDesc a, uint64_t n, int32_t* fault) {
    uint64_t i = (uint64_t)blockIdx.x * kBlock + threadIdx.x;
    const uint64_t step = (uint64_t)gridDim.x * kBlock;
    for (; i < n; i += step) {
        uint64_t rem = i;
        int64_t ol = 0, orr = 0, od = 0;
        for (int k = a.rank - 1; k >= 0; --k) {
            uint64_t q = rem / (uint64_t)a.shape[k];
            int64_t c = (int64_t)(rem - q * (uint64_t)a.shape[k]);
            ol += c * a.stride[0][k];
            orr += c * a.stride[1][k];
            od += c * a.stride[2][k];
            rem = q;
        }
        d[od] = bin_apply<OP, T>(l[ol], r[orr], fault);
    }
}

// Layouts that keep more than RT_MAX_RANK dims after collapsing (the reference accepts rank <= 128): the descriptor is read from
// device memory, one element per lane, 64-bit index arithmetic.  Correct for every layout; nothing here is tuned.
template <class T, int OP>
__global__ __launch_bounds__(kBlock) void bin_big_kernel(const T* l, const T* r, T* d, const int64_t* __restrict__ w, int rank, uint64_t n, int32_t* fault) {
    uint64_t i = (uint64_t)blockIdx.x * kBlock + threadIdx.x;
    const uint64_t step = (uint64_t)gridDim.x * kBlock;
    for (; i < n; i += step) {
        uint64_t rem = i;
        int64_t ol = 0, orr = 0, od = 0;
        for (int k = rank - 1; k >= 0; --k) {
            const uint64_t sh = (uint64_t)w[k];
            const uint64_t q = rem / sh;
            const int64_t c = (int64_t)(rem - q * sh);
            ol += c * w[rank + k];
            orr += c * w[2 * rank + k];
            od += c * w[3 * rank + k];
            rem = q;
        }
        d[od] = bin_apply<OP, T>(l[ol], r[orr], fault);
    }
}

template <class T, int OP>
int32_t broadcast_big(rt_ctx* ctx, const BigDesc& b, uint64_t count, const void* lv, const void* rv, void* dv) {
    const size_t blocks = (size_t)((count + kBlock - 1) / kBlock);
    const size_t cap = (size_t)ctx->num_cus * 64;
    hipLaunchKernelGGL((bin_big_kernel<T, OP>), dim3((unsigned)(blocks < cap ? blocks : cap)), dim3(kBlock), 0, ctx->stream,
                       (const T*)lv + b.offset[0], (const T*)rv + b.offset[1], (T*)dv + b.offset[2], b.words, b.rank, count, fault_of<T, OP>(ctx));
    RT_HIP(hipGetLastError());
    return RT_OK;
}

// ---- host: kernel choice ----------------------------------------------------------------------------------------------
template <class T, int OP, int LM, int RM>
void launch_rows_g(bool batched, dim3 grid, unsigned bs, hipStream_t s, const T* l, const T* r, T* d, const RowArgs& a, int32_t* fault) {
    // the batched long-loop form is only ever chosen when one input is gathered element-wise
    if constexpr (LM == M_ELEM || RM == M_ELEM) {
        if (batched) { hipLaunchKernelGGL((bin_rows_kernel<T, OP, LM, RM, 4>), grid, dim3(bs), 0, s, l, r, d, a, fault); return; }
    }
    hipLaunchKernelGGL((bin_rows_kernel<T, OP, LM, RM, 1>), grid, dim3(bs), 0, s, l, r, d, a, fault);
}
template <class T, int OP, int LM>
void launch_rows_r(int rm, bool batched, dim3 grid, unsigned bs, hipStream_t s, const T* l, const T* r, T* d, const RowArgs& a, int32_t* fault) {
    switch (rm) {
        case M_VEC: launch_rows_g<T, OP, LM, M_VEC>(batched, grid, bs, s, l, r, d, a, fault); break;
        case M_BCAST: launch_rows_g<T, OP, LM, M_BCAST>(batched, grid, bs, s, l, r, d, a, fault); break;
        default: launch_rows_g<T, OP, LM, M_ELEM>(batched, grid, bs, s, l, r, d, a, fault); break;
    }
}
template <class T, int OP>
void launch_rows(int lm, int rm, bool batched, dim3 grid, unsigned bs, hipStream_t s, const T* l, const T* r, T* d, const RowArgs& a, int32_t* fault) {
    switch (lm) {
        case M_VEC: launch_rows_r<T, OP, M_VEC>(rm, batched, grid, bs, s, l, r, d, a, fault); break;
        case M_BCAST: launch_rows_r<T, OP, M_BCAST>(rm, batched, grid, bs, s, l, r, d, a, fault); break;
        default: launch_rows_r<T, OP, M_ELEM>(rm, batched, grid, bs, s, l, r, d, a, fault); break;
    }
}

template <class T, int OP>
int32_t broadcast_typed(rt_ctx* ctx, const NdDesc& dsc, uint64_t count, const void* lv, const void* rv, void* dv) {
    const T* l = (const T*)lv;
    const T* r = (const T*)rv;
    T* d = (T*)dv;
    constexpr int64_t N = 16 / sizeof(T);
    hipStream_t s = ctx->stream;
    const int rank = dsc.rank;

    // 2^31 elements or more in an N-d layout (a 2 GiB u8 broadcast): slices along the outermost dim, each through the kernels below
    // (the element-per-lane 64-bit kernel that would otherwise take it runs at 3 % of their speed)
    if (count >= (1ull << 31) && rank >= 2)
        return rt_for_slices_below_2g(dsc, count, [&](const NdDesc& sub, uint64_t n) { return broadcast_typed<T, OP>(ctx, sub, n, lv, rv, dv); });

    // (1) one unit-stride run in all three operands
    // (for the gather op the right operand is a placeholder that is never read: treat it as a twin of the left one)
    const bool r_unit = (OP == kOpCopy) || rank == 0 || dsc.stride[1][0] == 1;
    if (rank <= 1 && (rank == 0 || (dsc.stride[0][0] == 1 && r_unit && dsc.stride[2][0] == 1))) {
        const T* lp = l + dsc.offset[0];
        const T* rp = (OP == kOpCopy) ? lp : r + dsc.offset[1];
        T* dp = d + dsc.offset[2];
        uintptr_t al = reinterpret_cast<uintptr_t>(lp) & 15, ar = reinterpret_cast<uintptr_t>(rp) & 15, ad = reinterpret_cast<uintptr_t>(dp) & 15;
        if (al == ar && ar == ad) {
            size_t n = (size_t)count;
            // the body starts where dst reaches a 128-byte line (the inputs, in phase with dst modulo 16, are then 16-byte aligned):
            // a wave's 1 KiB of stores covers eight whole lines instead of sharing its first and last line with a neighbour
            size_t head = ((128 - (reinterpret_cast<uintptr_t>(dp) & 127)) & 127) / sizeof(T);
            if (head > n) head = n;
            size_t nvec = (n - head) / N, tail = n - head - nvec * N;
            const TileMap m = rt_make_tilemap(dp + head, nvec, kCBlock2);
            size_t blocks = rt_tilemap_blocks(m, nvec, kCBlock2);
            if (blocks < 1) blocks = 1;                            // fewer elements than a vector: edges only
            if (blocks > 0x7fffffffull) return rt_fail(RT_E_INVALID, "broadcast: %zu elements is too long for one launch", n);
            RT_TRY(rt_check_edges("broadcast", head, nvec, (size_t)N, tail, n, kCBlock2));
            hipLaunchKernelGGL((bin_contig_kernel<T, OP>), dim3((unsigned)blocks), dim3(kCBlock2), 0, s,
                               reinterpret_cast<const Vec16<T>*>(lp + head), reinterpret_cast<const Vec16<T>*>(rp + head),
                               reinterpret_cast<Vec16<T>*>(dp + head), nvec, (uint32_t)head, (uint32_t)tail, m, fault_of<T, OP>(ctx));
            RT_HIP(hipGetLastError());
            return RT_OK;
        }
    }

    // (1b) an input that is a permuted view with short contiguous pieces -- it steps by 64 bytes or more along dst's inner dim, is
    // unit-stride along some other dim, and the transposing kernels below do not fit it (dst rows or that unit-stride dim too
    // short); or its unit-stride rows are short and lie scattered.  Read along dst's rows it costs a cache line per element or per
    // few elements (f32 `a + b.permute(..)` over 256 MiB operands: median 0.27 of peak over 54 such views, the lowest tenth 0.08).
    // Where dst and the other input are row-major runs and the type allows, the op rides on the second stage of the N-d tile copy
    // of that input (rt_permute.hip: one pass over each tensor, 0.45 - 0.75 of peak on those views); otherwise the input is copied
    // into a row-major temporary by the tile copy and the op runs on the temporary (two more passes over that operand, 0.37 - 0.48).
    // The temporary comes from the context's block cache and goes back to it; all work is on the context's stream.
    if constexpr (OP != kOpCopy && sizeof(T) <= 8) {
        auto short_pieces = [&](int o) {
            const int64_t is1 = dsc.stride[o][rank - 1], mag1 = is1 < 0 ? -is1 : is1;
            if (is1 == 1) {
                // unit-stride rows of less than 256 bytes (64 for 1- and 2-byte elements): rows of 2 out of strides (2, 32, 1) ran at
                // 0.16 of peak ...
                const uint64_t row_bytes = (uint64_t)dsc.shape[rank - 1] * sizeof(T);
                if (row_bytes >= (sizeof(T) >= 4 ? 256u : 64u)) return false;
                // ... and whose rows lie scattered: the 4096 elements that dst's order visits next span more than four times their
                // own size in the input.  Rows that are merely reversed or stepped stay compact, the row kernels find them in cache
                // (rows of 7 under a reversed dim of 64: 0.79 there, 0.43 through a temporary).
                uint64_t visited = 1, span = 1;
                for (int k = rank - 1; k >= 0; --k) {
                    if (dsc.stride[o][k] == 0) return false;
                    if (visited >= 4096) continue;
                    const uint64_t want = (4096 + visited - 1) / visited;
                    const uint64_t take = (uint64_t)dsc.shape[k] < want ? (uint64_t)dsc.shape[k] : want;
                    const int64_t st = dsc.stride[o][k];
                    span += (take - 1) * (uint64_t)(st < 0 ? -st : st);
                    visited *= take;
                }
                return span > 4 * visited;
            }
            if (mag1 <= 1 || (uint64_t)mag1 * sizeof(T) < 64) return false;
            bool unit_dim = false, transposable = false;
            uint64_t inside = 1;                                       // dst elements per index of the innermost unit-stride dim
            for (int k = 0; k < rank; ++k) {
                if (dsc.stride[o][k] == 0) return false;               // a repeated dim: the temporary would hold every repeat
                const bool unit = dsc.stride[o][k] == 1 || dsc.stride[o][k] == -1;
                unit_dim = unit_dim || unit;
                transposable = transposable || (unit && k < rank - 1 && dsc.shape[k] >= 16);
                inside = unit ? 1 : inside * (uint64_t)dsc.shape[k];
            }
            // With fewer than 32 dst elements inside the unit-stride dim (dst rows of 16 down a column of 4096), the rows that use one
            // cache line of the input follow each other closely and the row kernel's gathers hit in cache: 0.65 - 0.86 of peak there
            // against 0.48 - 0.50 in two passes; from 33 on the two passes win (0.38 against 0.46 and further apart).
            if (!unit_dim || inside < 32) return false;
            // (the transposing kernels take dst rows from a quarter of their tile's columns on)
            const int64_t tile_rows_from = sizeof(T) == 1 ? 128 : 256 / (int64_t)sizeof(T);
            return !(transposable && dsc.shape[rank - 1] >= tile_rows_from);
        };
        if (rank >= 2 && count < (1ull << 31) && count * sizeof(T) >= (256u << 10) && dsc.stride[2][rank - 1] == 1) {
            const bool p0 = short_pieces(0), p1 = short_pieces(1);
            if (p0 != p1) {
                const int o = p0 ? 0 : 1;
                typedef typename std::conditional<sizeof(T) == 1, uint8_t, typename std::conditional<sizeof(T) == 2, uint16_t,
                        typename std::conditional<sizeof(T) == 4, uint32_t, uint64_t>::type>::type>::type Word;
                void* tmp = nullptr;
                bool runs = true;                                       // dst and the other input are row-major runs over the dims
                {
                    int64_t acc = 1;
                    for (int k = rank - 1; k >= 0; --k) {
                        runs = runs && dsc.stride[2][k] == acc && dsc.stride[1 - o][k] == acc;
                        acc *= dsc.shape[k];
                    }
                }
                if constexpr (PermBinFused<T, OP>::value) {
                    // float, double and the 32- / 64-bit carriers: the op rides on the tile copy's second stage, which loads the other
                    // input's piece next to the tile's and stores the result -- one pass over each tensor
                    if (runs) {
                        NdDesc gd = dsc;
                        int64_t acc = 1;
                        for (int k = rank - 1; k >= 0; --k) {
                            gd.stride[0][k] = dsc.stride[o][k];
                            gd.stride[2][k] = acc;
                            acc *= dsc.shape[k];
                        }
                        gd.offset[0] = dsc.offset[o];
                        int32_t status = RT_OK;
                        if (permute_bin_try<T, OP>(ctx, gd, count, o == 0 ? l : r, (o == 0 ? r : l) + dsc.offset[1 - o], d + dsc.offset[2], o == 0, &status))
                            return status;
                    }
                }
                if (rt_alloc_bytes(ctx, (size_t)count * sizeof(T), &tmp) == RT_OK) {
                    NdDesc gd = dsc, d2 = dsc;
                    int64_t acc = 1;
                    for (int k = rank - 1; k >= 0; --k) {
                        gd.stride[0][k] = dsc.stride[o][k];
                        gd.stride[1][k] = 0;
                        gd.stride[2][k] = acc;
                        d2.stride[o][k] = acc;
                        acc *= dsc.shape[k];
                    }
                    gd.offset[0] = dsc.offset[o];
                    gd.offset[1] = dsc.offset[o];
                    gd.offset[2] = 0;
                    d2.offset[o] = 0;
                    if (runs) {                                         // three row-major runs: one dim
                        d2.rank = 1;
                        d2.shape[0] = (int64_t)count;
                        for (int q = 0; q < 3; ++q) d2.stride[q][0] = 1;
                    }
                    int32_t status = RT_OK;
                    const bool copied = permute_try<Word>(ctx, gd, count, (const Word*)(o == 0 ? lv : rv), (Word*)tmp, &status, /*force=*/true);
                    if (copied && status == RT_OK) status = broadcast_typed<T, OP>(ctx, d2, count, o == 0 ? tmp : lv, o == 1 ? tmp : rv, dv);
                    const int32_t freed = rt_free_locked(ctx, tmp);
                    if (copied) return status != RT_OK ? status : freed;
                }
            }
        }
    }

    // (2a) copies only: interleaved -> planar, and views whose contiguous pieces are short on one side or both (rt_permute.hip);
    // then the tile kernel for one "transposed" input (rt_broadcast_tile.hip)
    if constexpr (OP == kOpCopy && std::is_integral<T>::value && sizeof(T) <= 8) {
        int32_t status = RT_OK;
        if (planar_copy_try<T>(ctx, dsc, count, l, d, &status)) return status;
        if (permute_try<T>(ctx, dsc, count, l, d, &status)) return status;
    }
    {
        int32_t status = RT_OK;
        if (tile_try<T, OP>(ctx, dsc, count, l, r, d, &status)) return status;
    }

    // (2) rows: dst inner dim unit-stride (rows may start at any element: 16-byte accesses at element alignment), everything
    // indexable in 32 bits
    // Rows whose pitch is not a whole number of 128-byte lines make every block of the row kernel start and end inside a line it
    // shares with its neighbours; when dst is one contiguous run and every input is either laid out like dst or constant along
    // the row (a per-row scalar), the flat kernel below writes whole aligned spans instead: (2^18, 1000) + (2^18, 1) f32 takes
    // 0.338 ms there against 0.393 ms here.  An input that is a row vector stays here (it is loaded with vector loads).
    auto row_major_run = [&](int o) {
        int64_t acc = 1;
        for (int k = rank - 1; k >= 0; --k) {
            if (dsc.stride[o][k] != acc) return false;
            acc *= dsc.shape[k];
        }
        return true;
    };
    bool prefer_flat = rank >= 2 && ((uint64_t)dsc.shape[rank - 1] * sizeof(T)) % 128 != 0 && row_major_run(2);
    for (int o = 0; o < (OP == kOpCopy ? 1 : 2) && prefer_flat; ++o)
        prefer_flat = row_major_run(o) || dsc.stride[o][rank - 1] == 0;
    // (2b) bias add / tensor op one-element tensor: dst and one input are one aligned run, the other input is a single row (or a
    // single element) repeated.  Measured against the row
    // kernel on 1 GiB f32: rows of 256 B 0.347 -> 0.338 ms, 16 KiB 0.355 -> 0.335, 128 KiB 0.340 -> 0.328, in place 0.368 -> 0.333;
    // level at 4 MiB rows, slower (0.384 -> 0.455 ms) at 64 MiB, where the row no longer stays in cache between its uses.
    if constexpr (OP != kOpCopy) {
        if (rank >= 1 && count < (1ull << 31) && row_major_run(2) && count % N == 0 && (reinterpret_cast<uintptr_t>(d + dsc.offset[2]) & 15) == 0) {
            for (int o = 0; o < 2; ++o) {
                const int p = 1 - o;                                   // o: the streamed input, p: the row (or the single element)
                bool is_row = rank >= 2 && dsc.stride[p][rank - 1] == 1 && dsc.shape[rank - 1] % N == 0 &&
                              (uint64_t)dsc.shape[rank - 1] * sizeof(T) <= (1u << 20);
                bool is_scalar = true;
                for (int k = 0; k < rank - 1; ++k) is_row = is_row && dsc.stride[p][k] == 0;
                for (int k = 0; k < rank; ++k) is_scalar = is_scalar && dsc.stride[p][k] == 0;
                const T* fo = (o == 0 ? l : r) + dsc.offset[o];
                const T* ro = (p == 0 ? l : r) + dsc.offset[p];
                if (!(is_row || is_scalar) || !row_major_run(o) || (reinterpret_cast<uintptr_t>(fo) & 15)) continue;
                if (!is_scalar && (reinterpret_cast<uintptr_t>(ro) & 15)) continue;
                const uint32_t nvec = (uint32_t)(count / N), row_vecs = is_scalar ? 0u : (uint32_t)(dsc.shape[rank - 1] / N);
                const TileMap m = rt_make_tilemap(d + dsc.offset[2], nvec, kCBlock2);
                dim3 grid((unsigned)rt_tilemap_blocks(m, nvec, kCBlock2)), blk(kCBlock2);
                if (p == 0) hipLaunchKernelGGL((bin_flat_row_kernel<T, OP, true>), grid, blk, 0, s, fo, ro, d + dsc.offset[2], nvec, row_vecs, make_fastdiv(row_vecs ? row_vecs : 1u), m, fault_of<T, OP>(ctx));
                else hipLaunchKernelGGL((bin_flat_row_kernel<T, OP, false>), grid, blk, 0, s, fo, ro, d + dsc.offset[2], nvec, row_vecs, make_fastdiv(row_vecs ? row_vecs : 1u), m, fault_of<T, OP>(ctx));
                RT_HIP(hipGetLastError());
                return RT_OK;
            }
        }
    }
    // dst rows that do not start on 16-byte boundaries (an odd row length, a column slice): when dst is one aligned contiguous run
    // and every input is a run like dst, a repeated row or a single element, the flat kernel below keeps all of dst's stores
    // aligned and is faster (65536 rows of 4095 f32 plus a row: 0.34 ms there, 0.46 ms here); with any other input the row kernel's
    // unaligned vectors beat the flat kernel's element gathers (8192 x 32767 out of `m[:, 1:]` plus a row: 0.41 against 0.54 ms).
    auto rows_aligned = [&](int o, const T* base) {
        if ((reinterpret_cast<uintptr_t>(base + dsc.offset[o]) & 15) != 0) return false;
        for (int k = 0; k < rank - 1; ++k)
            if (!mult_of(dsc.stride[o][k], N)) return false;
        return true;
    };
    auto repeated_row_or_element = [&](int o) {
        for (int k = 0; k < rank - 1; ++k)
            if (dsc.stride[o][k] != 0) return false;
        return rank >= 1 && (dsc.stride[o][rank - 1] == 1 || dsc.stride[o][rank - 1] == 0);
    };
    bool flat_good = count >= (uint64_t)N && row_major_run(2) && (reinterpret_cast<uintptr_t>(d + dsc.offset[2]) & 15) == 0;
    for (int o = 0; o < (OP == kOpCopy ? 1 : 2) && flat_good; ++o) flat_good = row_major_run(o) || repeated_row_or_element(o);
    // Short rows under a short loop dim leave a block of the row kernel next to nothing (out (19737, 100, 2, 17) = (19737, 1, 2, 17) +
    // (1, 100, 1, 17): two rows of 17 per block, 0.04 of peak): when dst is one aligned run, the flat kernel, one dst vector per lane
    // with the inputs gathered by index, does far better whatever the inputs look like.  The same for rows of less than 128 bytes under
    // any loop dim, of which a lane of the row kernel gets a ragged piece ((963, 4097, 1, 17) + (963, 1, 1, 17) f32: 0.25 -> 0.70 of peak;
    // from 128 bytes on the row kernel wins: rows of 100 f32 0.64 against 0.27).
    const bool tiny_blocks = rank >= 2 && row_major_run(2) && (reinterpret_cast<uintptr_t>(d + dsc.offset[2]) & 15) == 0 && count >= (uint64_t)N &&
                             ((uint64_t)dsc.shape[rank - 1] * (uint64_t)dsc.shape[rank - 2] * sizeof(T) < 2048 || (uint64_t)dsc.shape[rank - 1] * sizeof(T) < 128);
    if (rank >= 1 && !prefer_flat && !tiny_blocks && count < (1ull << 31) && dsc.stride[2][rank - 1] == 1 && dsc.shape[rank - 1] >= 2 * N &&
        (rows_aligned(2, d) || !flat_good)) {
        RowArgs a;
        memset(&a, 0, sizeof(a));
        a.L = (uint32_t)dsc.shape[rank - 1];
        a.istride[0] = dsc.stride[0][rank - 1];
        a.istride[1] = dsc.stride[1][rank - 1];
        auto mode = [&](int o) -> int {
            int64_t is = dsc.stride[o][rank - 1];
            if (is == 0) return (int)M_BCAST;
            if (is == 1) return (int)M_VEC;
            return (int)M_ELEM;
        };
        const int lm = mode(0), rm = (OP == kOpCopy) ? (int)M_BCAST : mode(1);
        // Loop dim.  Default: the innermost outer dim, two steps per lane (measured best on MI355X: enough work to
        // amortise the per-block index arithmetic, short enough that the chip is covered by ~10^5..10^6 small blocks;
        // a broadcast operand is re-read from L2, which its reuse distance fits).  Exception: an operand that needs
        // element-wise gathers (inner stride not 0/1) and does not move along some outer dim is fetched once and kept
        // in registers while the block walks that dim.
        // When all dst rows sit in the same phase of the 128-byte lines (or at least of the 16-byte vectors) but not at phase 0 --
        // `m[:, 1:]`, a run that starts inside a line -- the column origin moves back to the boundary: columns [0, lead) do not
        // exist, the lanes that meet them work by element, and every other lane stores an aligned vector, every wave whole lines.
        // With the origin at the row start each wave would write parts of two lines that its neighbours complete: config-3 add
        // into rows one element off a boundary 0.53 ms, 0.47 ms with cached stores.
        uint32_t lead = 0;
        {
            constexpr int64_t LN = sizeof(T) <= 8 ? 128 / (int64_t)sizeof(T) : N;
            bool same_vec = true, same_line = true;
            for (int k = 0; k < rank - 1; ++k) {
                same_vec = same_vec && mult_of(dsc.stride[2][k], N);
                same_line = same_line && mult_of(dsc.stride[2][k], LN);
            }
            const uint64_t first = reinterpret_cast<uintptr_t>(d + dsc.offset[2]) / sizeof(T);
            if (same_line) lead = (uint32_t)(first % (uint64_t)LN);
            else if (same_vec) lead = (uint32_t)(first % (uint64_t)N);
        }
        a.lead = lead;
        a.L += lead;
        int gdim = rank >= 2 ? rank - 2 : -1;
        uint32_t steps = 2;     // measured: 1 step 0.62 ms, 2 steps 0.33 ms, 4 steps 0.43 ms on the 2 GiB broadcast add
        for (int o = 0; o < 2; ++o) {
            if ((o == 0 ? lm : rm) != M_ELEM) continue;
            int best = -1;
            for (int k = 0; k < rank - 1; ++k)
                if (dsc.stride[o][k] == 0 && (best < 0 || dsc.shape[k] > dsc.shape[best])) best = k;
            if (best >= 0) { gdim = best; steps = 16; }
        }
        a.G = gdim >= 0 ? (uint32_t)dsc.shape[gdim] : 1;
        for (int o = 0; o < 3; ++o) a.gstride[o] = gdim >= 0 ? dsc.stride[o][gdim] : 0;
        a.nouter = 0;
        uint64_t outer = 1;
        for (int k = 0; k < rank - 1; ++k) {
            if (k == gdim) continue;
            a.oshape[a.nouter] = (uint32_t)dsc.shape[k];
            a.odiv[a.nouter] = make_fastdiv((uint32_t)dsc.shape[k]);
            for (int o = 0; o < 3; ++o) a.ostride[o][a.nouter] = dsc.stride[o][k];
            outer *= (uint64_t)dsc.shape[k];
            a.nouter++;
        }
        for (int k = a.nouter; k < RT_MAX_RANK; ++k) { a.oshape[k] = 1; a.odiv[k] = make_fastdiv(1); }
        // lanes per row: enough for one vector per lane, at most a block
        uint32_t vecs = (uint32_t)((a.L + N - 1) / N);
        uint32_t tpr = 1;
        while (tpr < vecs && tpr < (uint32_t)kRBlock) tpr <<= 1;
        // the lean form: rows of 1 KiB and more, no gathered input, at most two outer dims (of at most 65535 each), rows not shifted,
        // every offset inside an operand below 2^31
        const uint32_t true_vecs = (uint32_t)(((uint64_t)dsc.shape[rank - 1] + N - 1) / N);
        // rows of 64 vectors and more; shorter ones, down to 32 vectors, when they are whole vectors and fill their tiles to 85 %
        // (m[:, 16:C-16] += row on 2^20 x 256 f32: 0.61 -> 0.73 of peak; rows of one half-filled or ragged tile are faster below)
        const RowTiling rt = rt_row_tiling(reinterpret_cast<uintptr_t>(d + dsc.offset[2]) / sizeof(T), dsc.stride[2], rank - 1, (uint32_t)dsc.shape[rank - 1], (uint32_t)sizeof(T));
        const bool lean = true_vecs >= 64 || (true_vecs >= 32 && !rt.ragged && (uint64_t)true_vecs * 100 >= (uint64_t)rt.tiles * 64 * 85);
        if (steps == 2 && lean && a.G >= 4 && rank <= 5 && lm != M_ELEM && rm != M_ELEM) {
            bool fits = true;
            for (int o = 0; o < 3; ++o) {
                uint64_t reach = 0;
                for (int k = 0; k < rank; ++k) reach += (uint64_t)(dsc.shape[k] - 1) * (uint64_t)(dsc.stride[o][k] < 0 ? -dsc.stride[o][k] : dsc.stride[o][k]);
                fits = fits && reach < (1ull << 31);
            }
            const uint64_t n0 = rank >= 3 ? (uint64_t)dsc.shape[rank - 3] : 1ull, n1 = rank >= 4 ? (uint64_t)dsc.shape[rank - 4] : 1ull;
            const uint64_t n2 = rank >= 5 ? (uint64_t)dsc.shape[rank - 5] : 1ull;
            Rows4Args q;
            memset(&q, 0, sizeof(q));
            q.L = (uint32_t)dsc.shape[rank - 1];
            q.G = a.G;
            q.tiles = rt.tiles;
            // rows with ragged ends: an odd number of tiles, so that the long-lived waves at the ends of the rows do not keep landing
            // on the same XCDs (see the in-place row kernel): m[:, 1:] += row on 65536 x 4096 f32 0.58 -> 0.8 of peak
            if (rt.ragged && q.tiles >= 2 && q.tiles % 2 == 0) q.tiles += 1;
            q.tiles_div = make_fastdiv(q.tiles);
            const uint32_t chunks = (a.G + 3) / 4;
            uint64_t gx = (uint64_t)q.tiles * chunks;
            // A row-wise input of more than 4 MiB per row that does not move along the loop dim: bands of 32 rows, groups of 32 tiles
            // (f32 (64, 2^21) + (1, 2^21): 0.73 -> 0.80 of peak, (16, 2^24) + (1, 2^24): 0.72 -> 0.74).  Shorter rows stay in cache from
            // one chunk of rows to the next in plain order and lose with any banding: 1.5 MiB rows 0.81 -> 0.76, 4 MiB rows level.
            bool long_repeated_row = false;
            for (int o = 0; o < 2; ++o)
                if ((o == 0 ? lm : rm) == M_VEC && dsc.stride[o][rank - 2] == 0 && (uint64_t)q.L * sizeof(T) > (4u << 20)) long_repeated_row = true;
            q.group = 0;
            q.group_div = make_fastdiv(1);
            q.band_div = make_fastdiv(1);
            if (long_repeated_row && chunks >= 2) {
                q.band_chunks = chunks < 8u ? chunks : 8u;
                q.tg_shift = 5;
                q.group = q.band_chunks << q.tg_shift;
                q.group_div = make_fastdiv(q.group);
                const uint64_t per_band = (uint64_t)((q.tiles + (1u << q.tg_shift) - 1) >> q.tg_shift) * q.group;
                const uint64_t bands = (chunks + q.band_chunks - 1) / q.band_chunks;
                if (per_band < (1ull << 31)) {
                    q.band_blocks = (uint32_t)per_band;
                    q.band_div = make_fastdiv(q.band_blocks);
                    gx = per_band * bands;
                } else {
                    q.group = 0;
                }
            }
            if (fits && n0 <= 65535 && n1 * n2 <= 65535 && gx < (1ull << 31)) {
                q.n1 = (uint32_t)n1;
                q.n1_div = make_fastdiv(q.n1);
                for (int o = 0; o < 3; ++o) {
                    q.o2s[o] = rank >= 5 ? (int32_t)dsc.stride[o][rank - 5] : 0;
                    q.gs[o] = (int32_t)dsc.stride[o][rank - 2];
                    q.o0s[o] = rank >= 3 ? (int32_t)dsc.stride[o][rank - 3] : 0;
                    q.o1s[o] = rank >= 4 ? (int32_t)dsc.stride[o][rank - 4] : 0;
                }
                // inputs that are read exactly once (no stride-0 dim) are loaded with the non-temporal hint: a left half += (R, 1) on
                // 65536 x 8192 f32 0.78 -> 0.82 of peak, w = a + b on half-width views 0.78 -> 0.85, z += x over 2 GiB 0.74 -> 0.79
                int ntm = 0;
                for (int o = 0; o < 2; ++o) {
                    bool once = true;
                    for (int k = 0; k < rank; ++k) once = once && dsc.stride[o][k] != 0;
                    if (once) ntm |= 1 << o;
                }
                launch_rows4<T, OP>(lm, rm, ntm, dim3((unsigned)gx, (unsigned)n0, (unsigned)(n1 * n2)), s, l + dsc.offset[0], r + dsc.offset[1], d + dsc.offset[2], q, fault_of<T, OP>(ctx));
                RT_HIP(hipGetLastError());
                return RT_OK;
            }
        }
        a.tpr = tpr;
        a.tiles = (vecs + tpr - 1) / tpr;
        const uint32_t gy = kRBlock / tpr;
        uint32_t gchunk = gy * steps;
        if (gchunk > a.G) gchunk = a.G;
        if (gchunk < 1) gchunk = 1;
        a.gchunk = gchunk;
        a.nchunks = (a.G + gchunk - 1) / gchunk;
        a.tiles_div = make_fastdiv(a.tiles);
        a.nchunks_div = make_fastdiv(a.nchunks);
        const uint64_t blocks = outer * a.nchunks * a.tiles;
        if (blocks < (1ull << 31)) {
            // the operand pointers address column 0 of the moved origin (never dereferenced below column `lead`)
            launch_rows<T, OP>(lm, rm, steps > 2, dim3((unsigned)blocks), kRBlock, s, l + dsc.offset[0] - (int64_t)lead * a.istride[0],
                               r + dsc.offset[1] - (int64_t)lead * a.istride[1], d + dsc.offset[2] - (int64_t)lead, a, fault_of<T, OP>(ctx));
            RT_HIP(hipGetLastError());
            return RT_OK;
        }
    }

    // (3) flat / generic
    if (count < (1ull << 31)) {
        GenArgs g;
        g.rank = rank;
        for (int k = 0; k < RT_MAX_RANK; ++k) {
            g.shape[k] = k < rank ? (uint32_t)dsc.shape[k] : 1;
            g.div[k] = make_fastdiv(g.shape[k]);
            for (int o = 0; o < 3; ++o) g.stride[o][k] = k < rank ? dsc.stride[o][k] : 0;
        }
        const T* lp = l + dsc.offset[0];
        const T* rp = r + dsc.offset[1];
        T* dp = d + dsc.offset[2];
        // dst must walk memory exactly like a row-major run over the collapsed shape from a 16-byte aligned address; an input that
        // walks the same way (from any element) is read with one vector load per lane
        uint32_t first = 0;
        if (row_major_run(2) && (reinterpret_cast<uintptr_t>(dp) & 15) == 0 && count >= (uint64_t)N) {
            const uint32_t nvec = (uint32_t)(count / N);
            const bool lv = row_major_run(0), rv = OP != kOpCopy && row_major_run(1);
            // a repeated row: stride 1 along the last dim, 0 along every other one
            auto row_like = [&](int o) {
                if (rank < 2 || dsc.stride[o][rank - 1] != 1) return false;
                for (int k = 0; k < rank - 1; ++k)
                    if (dsc.stride[o][k] != 0) return false;
                return true;
            };
            const bool lrow = !lv && rv && row_like(0), rrow = lv && !rv && OP != kOpCopy && row_like(1);
            dim3 grid((nvec + kRBlock - 1) / kRBlock), blk(kRBlock);
            if (lrow) hipLaunchKernelGGL((bin_flat_kernel<T, OP, F_ROW, F_VEC>), grid, blk, 0, s, lp, rp, dp, g, nvec, fault_of<T, OP>(ctx));
            else if (rrow) hipLaunchKernelGGL((bin_flat_kernel<T, OP, F_VEC, F_ROW>), grid, blk, 0, s, lp, rp, dp, g, nvec, fault_of<T, OP>(ctx));
            else if (lv && rv) hipLaunchKernelGGL((bin_flat_kernel<T, OP, F_VEC, F_VEC>), grid, blk, 0, s, lp, rp, dp, g, nvec, fault_of<T, OP>(ctx));
            else if (lv) hipLaunchKernelGGL((bin_flat_kernel<T, OP, F_VEC, F_ELEM>), grid, blk, 0, s, lp, rp, dp, g, nvec, fault_of<T, OP>(ctx));
            else if (rv) hipLaunchKernelGGL((bin_flat_kernel<T, OP, F_ELEM, F_VEC>), grid, blk, 0, s, lp, rp, dp, g, nvec, fault_of<T, OP>(ctx));
            else hipLaunchKernelGGL((bin_flat_kernel<T, OP, F_ELEM, F_ELEM>), grid, blk, 0, s, lp, rp, dp, g, nvec, fault_of<T, OP>(ctx));
            first = nvec * (uint32_t)N;                          // the last count % N elements go to the element kernel
        }
        if (first < count) {
            size_t blocks = ((size_t)(count - first) + kGU * kBlock - 1) / (kGU * kBlock);
            hipLaunchKernelGGL((bin_generic_kernel<T, OP>), dim3((unsigned)blocks), dim3(kBlock), 0, s, lp, rp, dp, g, first, (uint32_t)count, fault_of<T, OP>(ctx));
        }
    } else {
        size_t cap = (size_t)ctx->num_cus * 64;
        hipLaunchKernelGGL((bin_generic64_kernel<T, OP>), dim3((unsigned)cap), dim3(kBlock), 0, s,
                           l + dsc.offset[0], r + dsc.offset[1], d + dsc.offset[2], dsc, count, fault_of<T, OP>(ctx));
    }
    RT_HIP(hipGetLastError());
    return RT_OK;
}

template <class T> struct type_tag { typedef T type; };

// Calls fn(type_tag<T>, integral_constant<OP>) for the element carrier and op of a broadcast; + - * on two's-complement integers
// do not depend on signedness, so they run on the unsigned type of the same width (one instantiation per width).
template <class Fn>
int32_t with_type_op(int dtype, int op, Fn&& fn) {
    if (op == RT_DIV) {
        typedef std::integral_constant<int, RT_DIV> D;
        switch (dtype) {
            case RT_U8: return fn(type_tag<uint8_t>{}, D{});
            case RT_I8: return fn(type_tag<int8_t>{}, D{});
            case RT_U16: return fn(type_tag<uint16_t>{}, D{});
            case RT_I16: return fn(type_tag<int16_t>{}, D{});
            case RT_U32: return fn(type_tag<uint32_t>{}, D{});
            case RT_I32: return fn(type_tag<int32_t>{}, D{});
            case RT_U64: return fn(type_tag<uint64_t>{}, D{});
            case RT_I64: return fn(type_tag<int64_t>{}, D{});
            case RT_F32: return fn(type_tag<float>{}, D{});
            case RT_F64: return fn(type_tag<double>{}, D{});
            case RT_U128: return fn(type_tag<u128_t>{}, D{});
            case RT_I128: return fn(type_tag<i128_t>{}, D{});
            case RT_BOOL: return rt_fail(RT_E_ARITH, "broadcast: division is not implemented for boolean in the reference (todo!())");
        }
        return rt_fail(RT_E_DTYPE, "broadcast: unknown dtype code %d", dtype);
    }
    auto ops = [&](auto t) -> int32_t {
        switch (op) {
            case RT_ADD: return fn(t, std::integral_constant<int, RT_ADD>{});
            case RT_SUB: return fn(t, std::integral_constant<int, RT_SUB>{});
            case RT_MUL: return fn(t, std::integral_constant<int, RT_MUL>{});
        }
        return rt_fail(RT_E_INVALID, "broadcast: unknown op code %d", op);
    };
    switch (dtype) {
        case RT_U8: case RT_I8: return ops(type_tag<uint8_t>{});
        case RT_U16: case RT_I16: return ops(type_tag<uint16_t>{});
        case RT_U32: case RT_I32: return ops(type_tag<uint32_t>{});
        case RT_U64: case RT_I64: return ops(type_tag<uint64_t>{});
        case RT_F32: return ops(type_tag<float>{});
        case RT_F64: return ops(type_tag<double>{});
        case RT_BOOL: return ops(type_tag<boolean_t>{});
        case RT_U128: case RT_I128: return ops(type_tag<u128_t>{});
    }
    return rt_fail(RT_E_DTYPE, "broadcast: unknown dtype code %d", dtype);
}

}  // namespace

// Row-major copy of the elements a view addresses (TensorView::owned / contiguous, core/tensor.rs:299-325).
extern "C" int32_t rt_gather(rt_ctx* ctx, int32_t dtype, const void* src, uint64_t src_len, uint64_t offset, int32_t rank,
                             const uint64_t* shape, const int64_t* strides, void* dst, uint64_t dst_len) {
    RT_TRY(rt_ctx_enter(ctx));
    const int es = rt_elem_size(dtype);
    if (!es) return rt_fail(RT_E_DTYPE, "gather: unknown dtype code %d", dtype);
    uint64_t count = 0;
    RT_TRY(rt_check_extent("gather source", offset, rank, shape, strides, src_len, &count));
    if (count > dst_len) return rt_fail(RT_E_OUT_OF_BOUNDS, "gather: %llu elements into a buffer of %llu", (unsigned long long)count, (unsigned long long)dst_len);
    if (count == 0) return RT_OK;
    if (!src || !dst) return rt_fail(RT_E_INVALID, "gather: null buffer");
    if (rt_spans_meet(rt_view_span(src, es, offset, rank, shape, strides), rt_run_span(dst, es, 0, count)))
        return rt_fail(RT_E_INVALID, "gather: the destination overlaps the source view");
    // 128-bit elements move as pairs of 64-bit words: one more unit-stride dim of size 2
    const int words = es == 16 ? 2 : 1;
    uint64_t shp[RT_MAX_INPUT_RANK + 1];
    int64_t sst[RT_MAX_INPUT_RANK + 1], dstr[RT_MAX_INPUT_RANK + 1];
    int r2 = rank;
    for (int i = 0; i < rank; ++i) { shp[i] = shape[i]; sst[i] = strides[i] * words; }
    if (words == 2) { shp[rank] = 2; sst[rank] = 1; r2 = rank + 1; }
    int64_t acc = 1;
    for (int i = r2 - 1; i >= 0; --i) { dstr[i] = acc; acc *= (int64_t)shp[i]; }
    NdDesc d;
    const int64_t* sp[3] = {sst, sst, dstr};
    const uint64_t offs[3] = {offset * words, offset * words, 0};
    const uint64_t n = count * words;
    const int32_t cst = rt_collapse(3, r2, shp, sp, offs, /*reorder=*/true, /*key=*/2, &d);
    CtxGuard g(ctx);
    if (cst == RT_E_RANK) {
        BigDesc b;
        RT_TRY(rt_collapse_big(ctx, 3, r2, shp, sp, offs, /*reorder=*/true, /*key=*/2, &b));
        switch (es) {
            case 1: return broadcast_big<uint8_t, kOpCopy>(ctx, b, n, src, src, dst);
            case 2: return broadcast_big<uint16_t, kOpCopy>(ctx, b, n, src, src, dst);
            case 4: return broadcast_big<uint32_t, kOpCopy>(ctx, b, n, src, src, dst);
            default: return broadcast_big<uint64_t, kOpCopy>(ctx, b, n, src, src, dst);
        }
    }
    RT_TRY(cst);
    for (int k = 0; k < RT_MAX_RANK; ++k) d.stride[1][k] = 0;           // right operand: one element, never advanced
    switch (es) {
        case 1: return broadcast_typed<uint8_t, kOpCopy>(ctx, d, n, src, src, dst);
        case 2: return broadcast_typed<uint16_t, kOpCopy>(ctx, d, n, src, src, dst);
        case 4: return broadcast_typed<uint32_t, kOpCopy>(ctx, d, n, src, src, dst);
        default: return broadcast_typed<uint64_t, kOpCopy>(ctx, d, n, src, src, dst);
    }
}

extern "C" int32_t rt_broadcast(rt_ctx* ctx, int32_t dtype, int32_t op, int32_t rank, const uint64_t* shape,
                                const void* left, uint64_t left_len, uint64_t left_offset, const int64_t* left_strides,
                                const void* right, uint64_t right_len, uint64_t right_offset, const int64_t* right_strides,
                                void* dst, uint64_t dst_len, uint64_t dst_offset, const int64_t* dst_strides) {
    RT_TRY(rt_ctx_enter(ctx));
    if (op < RT_ADD || op > RT_DIV) return rt_fail(RT_E_INVALID, "broadcast: unknown op code %d", op);
    if (!rt_elem_size(dtype)) return rt_fail(RT_E_DTYPE, "broadcast: unknown dtype code %d", dtype);
    uint64_t count = 0, c2 = 0, c3 = 0;
    RT_TRY(rt_check_extent("broadcast left", left_offset, rank, shape, left_strides, left_len, &count));
    RT_TRY(rt_check_extent("broadcast right", right_offset, rank, shape, right_strides, right_len, &c2));
    RT_TRY(rt_check_extent("broadcast dst", dst_offset, rank, shape, dst_strides, dst_len, &c3));
    if (count == 0) return RT_OK;
    if (!left || !right || !dst) return rt_fail(RT_E_INVALID, "broadcast: null buffer");
    for (int i = 0; i < rank; ++i)
        if (shape[i] > 1 && dst_strides[i] == 0)
            return rt_fail(RT_E_INVALID, "broadcast: destination has stride 0 along dim %d of size %llu (it would be written more than once)",
                           i, (unsigned long long)shape[i]);
    {
        const int es = rt_elem_size(dtype);
        const ByteSpan ds = rt_view_span(dst, es, dst_offset, rank, shape, dst_strides);
        if (rt_spans_meet(ds, rt_view_span(left, es, left_offset, rank, shape, left_strides)) &&
            !rt_same_view(left, left_offset, left_strides, dst, dst_offset, dst_strides, rank, shape))
            return rt_fail(RT_E_INVALID, "broadcast: the destination overlaps the left operand without being the same view");
        if (rt_spans_meet(ds, rt_view_span(right, es, right_offset, rank, shape, right_strides)) &&
            !rt_same_view(right, right_offset, right_strides, dst, dst_offset, dst_strides, rank, shape))
            return rt_fail(RT_E_INVALID, "broadcast: the destination overlaps the right operand without being the same view");
    }
    NdDesc d;
    const int64_t* sp[3] = {left_strides, right_strides, dst_strides};
    const uint64_t offs[3] = {left_offset, right_offset, dst_offset};
    const int32_t cst = rt_collapse(3, rank, shape, sp, offs, /*reorder=*/true, /*key=*/2, &d);
    CtxGuard g(ctx);
    if (cst == RT_E_RANK) {
        BigDesc b;
        RT_TRY(rt_collapse_big(ctx, 3, rank, shape, sp, offs, /*reorder=*/true, /*key=*/2, &b));
        return with_type_op(dtype, op, [&](auto t, auto opc) -> int32_t {
            return broadcast_big<typename decltype(t)::type, decltype(opc)::value>(ctx, b, count, left, right, dst);
        });
    }
    RT_TRY(cst);
    return with_type_op(dtype, op, [&](auto t, auto opc) -> int32_t {
        return broadcast_typed<typename decltype(t)::type, decltype(opc)::value>(ctx, d, count, left, right, dst);
    });
}
