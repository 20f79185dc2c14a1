// Row-major copy of a permuted view through an N-d tile in LDS: the plan (host) and the index arithmetic of the three stages of a
// block (host and device, so that a host build can walk every lane of every block and check the map).
//
// The copy `dst[row-major] = src[view]` (TensorView::owned / contiguous of a permuted or sliced view, core/tensor.rs:299-325) is
// fast when src is unit-stride along dst's inner dim (the row kernels) or along one other long dim while dst's inner dim is long
// too (the transposing tile kernels).  What is left are views whose contiguous pieces are short on one side or on both:
// (64, 3, 2, 4096, 42) with strides (1, 262144, 786432, 64, 1572864) has dst rows of 42 elements, (7, 100, 33, 2905) with strides
// (1, 231, 7, 23100) has a unit-stride dim of 7.  Reading such a view in dst order touches a cache line per element.
//
// A tile here is a box of the N-d index space: extent t[k] along dim k, chosen so that the box holds a long piece of dst's memory
// order (the innermost dst dims in full, one more in part: the "dst run") *and* a long piece of src's memory order (the dims with
// the smallest |stride| in full, one more in part: the "src run").  A block
//   stage 0: tabulates byte offsets: for every position of the src run its offset in src and its place in the LDS tile, and for
//            every "row" of the two stages below (one index combination of the dims outside a run) its offset in src or dst, its
//            place in LDS and whether it exists in a tile that the view's edge cuts.  Every index decomposition of the block
//            happens here, once per position and once per row;
//   stage 1: walks the box in src order, lanes along the src run (several rows per wave instruction when the run is short), each
//            lane with loads for 8 or 16 rows in flight, and scatters the elements into LDS, which is laid out in dst order;
//   stage 2: walks the box in dst order, lanes along the dst run, reading LDS linearly (16-byte vectors where the run allows) and
//            storing whole pieces of dst rows with non-temporal stores.
// The tile and the tables live in dynamic LDS sized by the plan (up to 36 KiB + tables; three to eight blocks per CU).
#pragma once
#include <stdint.h>
#include <string.h>

#include "rt_common.h"

namespace rtp {

constexpr int kPBlock = 256;
constexpr uint32_t kPTileBytes = 32768;      // payload of a tile
constexpr uint32_t kPTabMax = 1024;          // positions of a src run
constexpr uint32_t kPRowMax = 512;           // rows of a stage

// A dim as a block needs it: the tile's extent, the whole extent, how to find the block's tile index along it, the strides.
struct PermDim {
    uint32_t t, shape, ntile, lstride;       // lstride: stride in the LDS tile, in elements
    FastDiv32 t_div, ntile_div, pre_div;     // pre_div: by the number of tiles of all dims after this one (they vary faster with blockIdx)
    int64_t sstride, dstride;
};

struct PermArgs {
    int32_t rank;
    PermDim dim[RT_MAX_RANK];                // dim rank-1 innermost in dst
    // stage 0 / 1: the src run (dims in src order, fastest first; only its last dim is ever cut by an edge tile) and the dims
    // enumerated by rows
    int32_t run1_n, row1_n;
    PermDim run1[RT_MAX_RANK], row1[RT_MAX_RANK], run1_last;
    uint32_t run1_len, run1_inner, rows1;    // positions of the run, positions per index of its last dim, rows
    // stage 2: the dst run is dims kd .. rank-1 (contiguous in dst and in LDS), rows enumerate the dims before kd
    int32_t row2_n;
    PermDim row2[RT_MAX_RANK], dkd;
    uint32_t run2_unit, rows2;               // elements per index of dim kd (the product of the shapes after it), rows
    uint32_t lds_elems;                      // elements of LDS the tile occupies, padding included
    uint32_t nblocks, neighbours;            // grid; tiles along the src run's cut dim share cache lines (see pm_remap)
    uint32_t lpr1, lpr2, per_iter1, per_iter2;   // lanes per row and rows per pass of the block in stages 1 and 2 (rt_permute_set_widths)
    FastDiv32 lpr1_div, lpr2_div;
    int64_t smin_run, smin_rows;             // lowest src offset (in elements, <= 0) that a position / a row of stage 1 reaches in a tile
};

__host__ __device__ __forceinline__ uint32_t pm_div(uint32_t n, const FastDiv32& f) {
    const uint32_t hi = (uint32_t)(((uint64_t)n * f.mul) >> 32);
    return (uint32_t)(((uint64_t)hi + n) >> f.shift);
}

// Index of the block's tile along a dim, and how much of the box exists there.
// (Rotating the tile index along the src run's dim by the one along the dst run's dim, so that blocks that run together form a
// diagonal of tiles instead of a line, measured level: 16384 x 16384 f32 transpose 0.635 -> 0.645 of peak, everything else unchanged.)
__host__ __device__ __forceinline__ uint32_t pm_tile_index(const PermDim& d, uint32_t block) {
    const uint32_t q = pm_div(block, d.pre_div);
    return q - pm_div(q, d.ntile_div) * d.ntile;
}
__host__ __device__ __forceinline__ uint32_t pm_extent(const PermDim& d, uint32_t block) {
    const uint32_t left = d.shape - pm_tile_index(d, block) * d.t;
    return left < d.t ? left : d.t;
}

// Blocks are dealt to the eight XCDs in turn.  When the pieces of src that a tile reads are not whole cache lines, tiles that are
// neighbours along the src run's cut dim read parts of the same lines: the plan then makes that dim the fastest in tile order, and
// this remap gives neighbours in tile order to the same XCD, one after the other, so that the second finds the line in that XCD's
// L2 (a unit-stride dim of 7 f32: 0.45 -> 0.49 of peak; 300 permuted 256 MiB views: median 0.69 -> 0.71, lowest quarter 0.53 ->
// 0.59).  With whole aligned lines nothing is shared, and the order that keeps the blocks in flight on neighbouring pieces of the
// same dst rows is the better one (16384 x 16384 transpose: 0.73 against 0.62).
__host__ __device__ __forceinline__ uint32_t pm_remap(const PermArgs& a, uint32_t block) {
    if (!a.neighbours) return block;
    const uint32_t per = a.nblocks / 8, full = per * 8;
    return block < full ? (block % 8) * per + block / 8 : block;
}

// What a block knows about its tile: where it starts in src and dst, and how much of the two runs exists.
struct PermBlock {
    int64_t sbase, dbase;
    uint32_t valid1, valid2;                 // positions of the src run / elements of the dst run that exist in this tile
};

__host__ __device__ __forceinline__ PermBlock pm_block(const PermArgs& a, uint32_t block) {
    PermBlock b;
    b.sbase = 0;
    b.dbase = 0;
#pragma unroll
    for (int k = 0; k < RT_MAX_RANK; ++k) {
        if (k < a.rank) {
            const uint32_t first = pm_tile_index(a.dim[k], block) * a.dim[k].t;
            b.sbase += (int64_t)first * a.dim[k].sstride;
            b.dbase += (int64_t)first * a.dim[k].dstride;
        }
    }
    b.valid1 = pm_extent(a.run1_last, block) * a.run1_inner;
    b.valid2 = pm_extent(a.dkd, block) * a.run2_unit;
    return b;
}

// Stage 0, position p of the src run: offset in src relative to the tile, place in LDS.  (Real loops over the dims that exist:
// unrolled over RT_MAX_RANK with a test per dim, the compiler computes all eight and selects.  Offsets inside a tile fit 32 bits.)
__host__ __device__ __forceinline__ void pm_position(const PermArgs& a, uint32_t p, int32_t* soff, uint32_t* loff) {
    int32_t s = 0;
    uint32_t l = 0, rem = p;
#pragma unroll 1
    for (int j = 0; j < a.run1_n; ++j) {
        const uint32_t q = pm_div(rem, a.run1[j].t_div);
        const uint32_t c = rem - q * a.run1[j].t;
        rem = q;
        s += (int32_t)c * (int32_t)a.run1[j].sstride;
        l += c * a.run1[j].lstride;
    }
    *soff = s;
    *loff = l;
}

// A row (index combination of the dims in `list`): offset by the chosen stride, place in LDS, and whether it exists in this tile.
template <bool DST>
__host__ __device__ __forceinline__ bool pm_row(const PermDim (&list)[RT_MAX_RANK], int n, uint32_t rows, uint32_t block, uint32_t row, int32_t* off, uint32_t* loff) {
    int32_t s = 0;
    uint32_t l = 0, rem = row;
    bool ok = row < rows;
#pragma unroll 1
    for (int j = 0; j < n; ++j) {
        const uint32_t q = pm_div(rem, list[j].t_div);
        const uint32_t c = rem - q * list[j].t;
        rem = q;
        s += (int32_t)c * (int32_t)(DST ? list[j].dstride : list[j].sstride);
        l += c * list[j].lstride;
        ok = ok && c < pm_extent(list[j], block);
    }
    *off = s;
    *loff = l;
    return ok;
}

// ---- the three stages of a block ------------------------------------------------------------------------------------------
// `tid` is the lane's index in the block.  A row is walked by `lpr` lanes -- as many as the run has loads or stores, up to the whole
// block -- so the block covers kPBlock / lpr rows per pass and a wave instruction several rows when the runs are short.
//
// All tables hold byte offsets, so that an access costs one addition per operand: positions and rows of stage 1 hold src offsets
// above the lowest one of the tile (unsigned 32-bit, added to a base pointer the block computes once; the plan keeps a tile's reach
// below 4 GiB), rows of stage 2 hold dst offsets, and the LDS places are bytes too.
constexpr int kPRows2 = 4;                   // rows a lane has in flight in stage 2

// Where a byte of the tile really lives: the 16-byte group's index within its 256-byte block is XORed with the block's index
// (bits 4..7 with bits 8..11).  Lanes of stage 1 that step through the tile by a multiple of 256 bytes -- a src-fastest dim that
// lies inside the dst run, e.g. dst rows of 16 floats written down a column -- would otherwise all write to the same banks
// ((1024, 4096, 16) out of strides (65536, 1, 4096): 0.43 of peak without).  16-byte groups stay whole, so stage 2 still reads
// vectors; the tile's allocation is a whole number of 4 KiB blocks so that the map stays inside it.
__host__ __device__ __forceinline__ uint32_t pm_swizzle(uint32_t byte) { return byte ^ ((byte >> 4) & 0xf0u); }
constexpr uint32_t kPNoRow = 0xffff;         // LDS place of a row that does not exist in a cut tile

// The block's tables in LDS: by position of the src run, by row of stage 1, by row of stage 2.
struct PermTables {
    uint32_t* pos_src;
    uint16_t* pos_lds;
    uint32_t* row1_src;
    uint16_t* row1_lds;
    uint32_t* row2_dst;
    uint16_t* row2_lds;
};

// Stage 0: every index decomposition of the block happens here, once per position and once per row; the two stages that move the
// data only add table entries.  (With the rows decomposed where they are used, a wave spent some 2000 vector and 1200 scalar
// instructions on 32 loads and 18 stores.)
template <class T>
__host__ __device__ __forceinline__ void pm_stage0(const PermArgs& a, uint32_t block, uint32_t tid, const PermTables& tb) {
    constexpr uint32_t ES = (uint32_t)sizeof(T);
    for (uint32_t p = tid; p < a.run1_len; p += kPBlock) {
        int32_t so;
        uint32_t lo;
        pm_position(a, p, &so, &lo);
        tb.pos_src[p] = (uint32_t)(so - (int32_t)a.smin_run) * ES;
        tb.pos_lds[p] = (uint16_t)(lo * ES);
    }
    for (uint32_t r = tid; r < a.rows1; r += kPBlock) {
        int32_t so;
        uint32_t lo;
        const bool ok = pm_row<false>(a.row1, a.row1_n, a.rows1, block, r, &so, &lo);
        tb.row1_src[r] = (uint32_t)(so - (int32_t)a.smin_rows) * ES;
        tb.row1_lds[r] = (uint16_t)(ok ? lo * ES : kPNoRow);
    }
    for (uint32_t r = tid; r < a.rows2; r += kPBlock) {
        int32_t dof;
        uint32_t lo;
        const bool ok = pm_row<true>(a.row2, a.row2_n, a.rows2, block, r, &dof, &lo);
        tb.row2_dst[r] = (uint32_t)dof * ES;
        tb.row2_lds[r] = (uint16_t)(ok ? lo * ES : kPNoRow);
    }
}

// W elements at element alignment
template <class T, int W> struct PmVecU { typedef T type __attribute__((ext_vector_type(W), aligned(sizeof(T)))); };
template <class T> struct PmVecU<T, 1> { typedef T type; };
template <class T, int W> struct PmVec { typedef T type __attribute__((ext_vector_type(W))); };
template <class T> struct PmVec<T, 1> { typedef T type; };
template <class V, class T, int W> __host__ __device__ __forceinline__ T pm_lane(const V& v, int i) {
    if constexpr (W == 1) return v; else return v[i];
}

// V: positions of the src run per load; V consecutive positions from a multiple of V are V consecutive elements of src (the plan
// checks that on the position table).  What keeps the memory system busy here is bytes in flight, and what costs time is every
// round trip to memory that a block makes one after another: a lane holds one load for each of 8 rows (16 rows when it loads single
// elements) before it turns to LDS, which for 4-byte elements and more is the lane's whole share of a 32 KiB tile at once.
template <class T, int V>
__host__ __device__ __forceinline__ void pm_stage1(const T* src, const PermArgs& a, const PermBlock& b, uint32_t tid, unsigned char* tile, const PermTables& tb) {
    constexpr int U = V > 1 ? 8 : 16;
    typedef typename PmVecU<T, V>::type VT;
    const uint32_t lpr = a.lpr1, sub = pm_div(tid, a.lpr1_div), pos = tid - sub * lpr;
    const uint32_t per_iter = a.per_iter1;
    if (sub >= per_iter) return;                                   // kPBlock is not a multiple of lpr: the last lanes have no row
    const unsigned char* sp = reinterpret_cast<const unsigned char*>(src + (b.sbase + a.smin_run + a.smin_rows));
    for (uint32_t r0 = sub; r0 < a.rows1; r0 += per_iter * U) {
        uint32_t so[U], lo[U];
#pragma unroll
        for (int u = 0; u < U; ++u) {
            const uint32_t r = r0 + u * per_iter;
            lo[u] = r < a.rows1 ? (uint32_t)tb.row1_lds[r] : kPNoRow;
            so[u] = r < a.rows1 ? tb.row1_src[r] : 0u;
        }
        for (uint32_t p = pos * V; p < b.valid1; p += lpr * V) {
            if (V == 1 || p + V <= b.valid1) {
                const uint32_t ts = tb.pos_src[p];
                VT v[U];
#pragma unroll
                for (int u = 0; u < U; ++u)
                    if (lo[u] != kPNoRow) v[u] = *reinterpret_cast<const VT*>(sp + (so[u] + ts));
                uint32_t tl[V];
#pragma unroll
                for (int i = 0; i < V; ++i) tl[i] = tb.pos_lds[p + i];
#pragma unroll
                for (int u = 0; u < U; ++u) {
                    if (lo[u] != kPNoRow) {
#pragma unroll
                        for (int i = 0; i < V; ++i) *reinterpret_cast<T*>(tile + pm_swizzle(lo[u] + tl[i])) = pm_lane<VT, T, V>(v[u], i);
                    }
                }
            } else {
                // the run ends inside this vector (a cut tile): by element
                for (uint32_t i = 0; p + i < b.valid1; ++i) {
                    const uint32_t ts = tb.pos_src[p + i];
                    const uint32_t tl = tb.pos_lds[p + i];
#pragma unroll
                    for (int u = 0; u < U; ++u)
                        if (lo[u] != kPNoRow) *reinterpret_cast<T*>(tile + pm_swizzle(lo[u] + tl)) = *reinterpret_cast<const T*>(sp + (so[u] + ts));
                }
            }
        }
    }
}

// What stage 2 does with a piece of the tile before it stores it.  The plain copy stores it as it is; a binary op whose other input
// is laid out like dst loads that input's piece at the same byte offset -- before the LDS reads, so that the loads of all rows a lane
// handles are in flight together: behind the stores they could not move up, because dst may be that very input (`c += v`) -- and
// combines the two.
struct PmCopy {
    template <class VT> __host__ __device__ __forceinline__ VT fetch(uint32_t) const { return VT{}; }
    template <class VT> __host__ __device__ __forceinline__ VT combine(const VT& tile_piece, const VT&) const { return tile_piece; }
};

// W: elements per store (rt_permute_store_width)
template <class T, int W, class F>
__host__ __device__ __forceinline__ void pm_stage2(T* dst, const PermArgs& a, const PermBlock& b, uint32_t tid, const unsigned char* tile, const PermTables& tb,
                                                    const F& f) {
    constexpr int U = kPRows2;
    constexpr uint32_t ES = (uint32_t)sizeof(T);
    typedef typename PmVec<T, W>::type VT;
    const uint32_t lpr = a.lpr2, sub = pm_div(tid, a.lpr2_div), pos = tid - sub * lpr;
    const uint32_t per_iter = a.per_iter2;
    if (sub >= per_iter) return;
    unsigned char* dp = reinterpret_cast<unsigned char*>(dst + b.dbase);
    const uint32_t valid = b.valid2 * ES;
    for (uint32_t r0 = sub; r0 < a.rows2; r0 += per_iter * U) {
        uint32_t dof[U], lo[U];
#pragma unroll
        for (int u = 0; u < U; ++u) {
            const uint32_t r = r0 + u * per_iter;
            lo[u] = r < a.rows2 ? (uint32_t)tb.row2_lds[r] : kPNoRow;
            dof[u] = r < a.rows2 ? tb.row2_dst[r] : 0u;
        }
        for (uint32_t p = pos * W * ES; p < valid; p += lpr * W * ES) {
            VT v[U], o[U];
#pragma unroll
            for (int u = 0; u < U; ++u)
                if (lo[u] != kPNoRow) o[u] = f.template fetch<VT>(dof[u] + p);
#pragma unroll
            for (int u = 0; u < U; ++u)
                if (lo[u] != kPNoRow) v[u] = *reinterpret_cast<const VT*>(tile + pm_swizzle(lo[u] + p));
#pragma unroll
            for (int u = 0; u < U; ++u)
                if (lo[u] != kPNoRow) __builtin_nontemporal_store(f.template combine<VT>(v[u], o[u]), reinterpret_cast<VT*>(dp + (dof[u] + p)));
        }
    }
}

// ---- the plan ---------------------------------------------------------------------------------------------------------------
// shape / sstride / dstride: the collapsed dims, dim rank-1 innermost in dst; dst is one row-major run over them (dstride[k] is
// the product of the shapes after k).  es: element size in bytes (1, 2, 4, 8).  Returns false when the copy is not for this
// kernel (an element count or a tile reach beyond 32 bits); *blocks is the grid.
static inline bool rt_permute_plan(int rank, const int64_t* shape, const int64_t* sstride, const int64_t* dstride, uint32_t es, PermArgs* out, uint64_t* blocks,
                                   uint32_t tile_bytes = kPTileBytes, bool src_base_on_line = true) {
    if (rank < 1 || rank > RT_MAX_RANK) return false;
    PermArgs a;
    memset(&a, 0, sizeof(a));
    a.rank = rank;
    uint64_t shp[RT_MAX_RANK], t[RT_MAX_RANK];
    for (int k = 0; k < rank; ++k) {
        if (shape[k] < 1 || shape[k] > 0x7fffffffll) return false;
        shp[k] = (uint64_t)shape[k];
        t[k] = 1;
    }
    {
        int64_t acc = 1;
        for (int k = rank - 1; k >= 0; --k) {
            if (dstride[k] != acc) return false;
            acc *= shape[k];
            if (acc > 0x7fffffffll) return false;
        }
    }
    // src order: ascending |stride|, repeated dims (stride 0) last
    int sord[RT_MAX_RANK];
    for (int k = 0; k < rank; ++k) sord[k] = rank - 1 - k;
    auto mag = [&](int k) -> uint64_t {
        const int64_t s = sstride[k];
        return s == 0 ? ~0ull : (uint64_t)(s < 0 ? -s : s);
    };
    for (int i = 1; i < rank; ++i)
        for (int j = i; j > 0 && mag(sord[j]) < mag(sord[j - 1]); --j) { const int x = sord[j]; sord[j] = sord[j - 1]; sord[j - 1] = x; }
    // run targets in elements: together the payload when the two runs share no dim, the dst run eight times the src run (f32: 256 and
    // 32, 1 KiB written per row piece and a 128-byte line read).  Measured on permuted 256 MiB f32 views, median fraction of peak:
    // 2:1 0.66, 8:1 0.68, 32:1 0.57; dst rows of 42 elements out of a unit-stride dim elsewhere 0.55 / 0.72 / 0.48.
    uint64_t want_d = 1, want_s = 1;
    while (want_d * want_s * 2 * es <= tile_bytes) { if (want_d <= want_s * 4) want_d *= 2; else want_s *= 2; }
    auto ceil_div = [](uint64_t x, uint64_t y) { return (x + y - 1) / y; };
    {
        uint64_t run = 1;
        for (int k = rank - 1; k >= 0; --k) {
            const uint64_t need = ceil_div(want_d, run);
            t[k] = shp[k] < need ? shp[k] : need;
            run *= t[k];
            if (t[k] < shp[k] || run >= want_d) break;
        }
    }
    {
        uint64_t run = 1;
        for (int j = 0; j < rank; ++j) {
            const int k = sord[j];
            const uint64_t need = ceil_div(want_s, run);
            const uint64_t grown = shp[k] < need ? shp[k] : need;
            if (grown > t[k]) t[k] = grown;
            run *= t[k];
            if (t[k] < shp[k] || run >= want_s) break;
        }
    }
    // the two runs as the extents now define them; a src run longer than the position table gives its outer dims to the rows
    int kd = 0, run1_n = 0;
    auto run_s = [&]() { uint64_t r = 1; for (int j = 0; j < run1_n; ++j) r *= t[sord[j]]; return r; };
    auto find_runs = [&]() {
        kd = rank - 1;
        while (kd > 0 && t[kd] == shp[kd]) --kd;
        run1_n = 0;
        for (int j = 0; j < rank; ++j) {
            run1_n = j + 1;
            if (t[sord[j]] < shp[sord[j]]) break;
        }
        while (run1_n > 1 && run_s() > kPTabMax) --run1_n;
    };
    auto volume = [&]() { uint64_t e = 1; for (int k = 0; k < rank; ++k) e *= t[k]; return e; };
    auto run_d = [&]() { uint64_t r = 1; for (int k = kd; k < rank; ++k) r *= t[k]; return r; };
    // LDS layout: the dst run as it lies in dst, then the dims before kd from the inside out, every level padded away from a
    // multiple of 128 bytes (lanes of stage 1 that step along such a dim would otherwise all hit the same banks)
    const uint64_t N = 16 / es;
    uint64_t lstride[RT_MAX_RANK];
    auto layout = [&]() -> uint64_t {
        uint64_t acc = 1;
        for (int k = rank - 1; k >= kd; --k) { lstride[k] = acc; acc *= (k == kd ? t[k] : shp[k]); }
        uint64_t cur = ceil_div(acc, N) * N + N;
        for (int k = kd - 1; k >= 0; --k) {
            lstride[k] = cur;
            if (t[k] > 1) {
                cur *= t[k];
                if ((cur / N) % 8 == 0) cur += N;
            }
        }
        return kd == 0 ? acc : cur;
    };
    // 0: fits; 1: too much payload or LDS; 2: too many rows in stage 1; 3: in stage 2; 4: a one-dim src run beyond the table
    auto misfit = [&]() -> int {
        find_runs();
        const uint64_t e = volume(), lds = layout();
        if (e * es > tile_bytes || lds * es > tile_bytes + tile_bytes / 8 || lds * es >= kPNoRow) return 1;
        if (run_s() > kPTabMax) return 4;
        if (e / run_s() > kPRowMax) return 2;
        if (e / run_d() > kPRowMax) return 3;
        return 0;
    };
    for (int guard = 0; guard < 96; ++guard) {
        const int why = misfit();
        if (why == 0) break;
        const int ks = sord[run1_n - 1];
        int k = -1;
        if (why == 1 || why == 4) {
            // shrink the partial dim of the run that exceeds its target by more
            const bool can_d = t[kd] > 1, can_s = t[ks] > 1;
            if (why == 4) k = ks;
            else if (can_d && can_s) k = (run_d() * want_s >= run_s() * want_d) ? kd : ks;
            else if (can_d) k = kd;
            else if (can_s) k = ks;
        } else {
            // too many rows: shrink the largest dim outside the run in question
            bool in_run[RT_MAX_RANK] = {};
            if (why == 2) for (int j = 0; j < run1_n; ++j) in_run[sord[j]] = true;
            else for (int q = kd; q < rank; ++q) in_run[q] = true;
            for (int q = 0; q < rank; ++q) if (!in_run[q] && t[q] > 1 && (k < 0 || t[q] > t[k])) k = q;
        }
        if (k < 0) for (int q = 0; q < rank; ++q) if (t[q] > 1 && (k < 0 || t[q] > t[k])) k = q;
        if (k < 0) return false;
        t[k] = (t[k] + 1) / 2;
    }
    if (misfit() != 0) return false;
    // a small box grows along the dst run's partial dim, else the src run's, else any dim that has room, innermost first
    for (int guard = 0; guard < 64; ++guard) {
        find_runs();
        const uint64_t e = volume();
        if (e * es * 2 >= tile_bytes) break;
        int cand[RT_MAX_RANK + 2], nc = 0;
        cand[nc++] = kd;
        cand[nc++] = sord[run1_n - 1];
        for (int q = rank - 1; q >= 0; --q) cand[nc++] = q;
        bool grew = false;
        for (int c = 0; c < nc && !grew; ++c) {
            const int k = cand[c];
            if (t[k] >= shp[k]) continue;
            const uint64_t before = t[k];
            for (uint64_t f = ceil_div(tile_bytes / 2, e * es); f >= 2 && !grew; f = (f + 1) / 2) {
                t[k] = before * f < shp[k] ? before * f : shp[k];
                if (misfit() == 0) grew = true;
                if (f == 2) break;
            }
            if (!grew) t[k] = before;
        }
        if (!grew) break;
    }
    if (misfit() != 0) return false;
    const uint64_t lds = layout();
    // fill in
    uint64_t nblocks = 1, reach_s = 0, reach_d = 0;
    // does a tile read whole aligned cache lines of src?  The contiguous piece at the start of the src run is a whole number of
    // lines, and every other dim steps by whole lines from a base on a line
    bool whole_lines = src_base_on_line;
    {
        uint64_t piece = 1;
        int64_t expect = 1;
        int j = 0;
        for (; j < run1_n; ++j) {
            const int k = sord[j];
            if (sstride[k] != expect) break;
            piece *= t[k];
            if (t[k] < shp[k]) { ++j; break; }
            expect *= shape[k];
        }
        whole_lines = whole_lines && (piece * es) % 128 == 0;
        for (; j < rank; ++j)
            if (shp[sord[j]] > 1 && sstride[sord[j]] != 0 && (mag(sord[j]) * es) % 128 != 0) whole_lines = false;
    }
    a.neighbours = whole_lines ? 0u : 1u;
    // tile order: the src run's cut dim first when its tiles share lines, then the dims from dst's innermost outward
    int order[RT_MAX_RANK], no = 0;
    const int ks_first = a.neighbours ? sord[run1_n - 1] : -1;
    if (ks_first >= 0) order[no++] = ks_first;
    for (int k = rank - 1; k >= 0; --k) if (k != ks_first) order[no++] = k;
    for (int oi = 0; oi < rank; ++oi) {
        const int k = order[oi];
        PermDim& d = a.dim[k];
        d.t = (uint32_t)t[k];
        d.shape = (uint32_t)shp[k];
        d.ntile = (uint32_t)ceil_div(shp[k], t[k]);
        d.lstride = (uint32_t)lstride[k];
        d.t_div = make_fastdiv(d.t);
        d.ntile_div = make_fastdiv(d.ntile);
        d.pre_div = make_fastdiv((uint32_t)nblocks);
        d.sstride = sstride[k];
        d.dstride = dstride[k];
        nblocks *= d.ntile;
        if (nblocks >= (1ull << 31)) return false;
        reach_s += sstride[k] != 0 ? (t[k] - 1) * mag(k) : 0;
        reach_d += (t[k] - 1) * (uint64_t)dstride[k];
    }
    if (reach_s * es >= (1ull << 31) || reach_d * es >= (1ull << 31)) return false;      // byte offsets inside a tile fit 32 bits
    bool in_run1[RT_MAX_RANK] = {};
    a.run1_n = run1_n;
    a.run1_len = 1;
    a.run1_inner = 1;
    for (int j = 0; j < run1_n; ++j) {
        const int k = sord[j];
        in_run1[k] = true;
        a.run1[j] = a.dim[k];
        if (j + 1 < run1_n) a.run1_inner *= a.dim[k].t;
        a.run1_len *= a.dim[k].t;
    }
    a.run1_last = a.dim[sord[run1_n - 1]];
    for (int k = 0; k < rank; ++k) {
        if (sstride[k] >= 0) continue;
        if (in_run1[k]) a.smin_run += (int64_t)(t[k] - 1) * sstride[k]; else a.smin_rows += (int64_t)(t[k] - 1) * sstride[k];
    }
    a.rows1 = 1;
    for (int k = rank - 1; k >= 0; --k) {
        if (in_run1[k] || a.dim[k].t == 1) continue;
        a.row1[a.row1_n++] = a.dim[k];
        a.rows1 *= a.dim[k].t;
    }
    a.dkd = a.dim[kd];
    a.run2_unit = (uint32_t)dstride[kd];
    a.rows2 = 1;
    for (int k = kd - 1; k >= 0; --k) {
        if (a.dim[k].t == 1) continue;
        a.row2[a.row2_n++] = a.dim[k];
        a.rows2 *= a.dim[k].t;
    }
    a.lds_elems = (uint32_t)lds;
    if (a.rows1 > kPRowMax || a.rows2 > kPRowMax || a.run1_len > kPTabMax) return false;
    a.nblocks = (uint32_t)nblocks;
    *out = a;
    *blocks = nblocks;
    return true;
}

// Elements that stage 2 may move per store (a power of two, at most `cap`): every piece of a dst run then starts at a multiple of
// it in dst and in LDS, and holds a whole number of them, in every tile including the cut ones.
static inline uint32_t rt_permute_store_width(const PermArgs& a, uint32_t cap) {
    uint32_t w = cap;
    while (w > 1) {
        const uint64_t step = (uint64_t)a.dkd.t * a.run2_unit;                        // between tiles along kd
        const uint64_t outer = (uint64_t)a.dkd.shape * a.run2_unit;                   // between rows (the whole of dst when kd is dim 0)
        if (step % w == 0 && outer % w == 0) break;
        w >>= 1;
    }
    return w;
}

// Positions of the src run that stage 1 may load at once (a power of two, at most `cap`): every group of that many positions
// from a multiple of it lies in src as consecutive ascending elements.  Decided on the position table itself.
static inline uint32_t rt_permute_load_width(const PermArgs& a, uint32_t cap) {
    uint32_t v = cap;
    while (v > 1) {
        bool ok = a.run1_len % v == 0;
        for (uint32_t p = 0; p + v <= a.run1_len && ok; p += v) {
            int32_t s0;
            uint32_t l0;
            pm_position(a, p, &s0, &l0);
            for (uint32_t i = 1; i < v && ok; ++i) {
                int32_t si;
                uint32_t li;
                pm_position(a, p + i, &si, &li);
                ok = si == s0 + (int32_t)i;
            }
        }
        if (ok) break;
        v >>= 1;
    }
    return v;
}

// Dynamic LDS of a launch: the tile, then the 32-bit tables, then the 16-bit ones.
static inline uint32_t rt_permute_lds_bytes(const PermArgs& a, uint32_t es) {
    const uint32_t tile = (a.lds_elems * es + 4095u) & ~4095u, entries = a.run1_len + a.rows1 + a.rows2;
    return tile + entries * 4u + ((entries * 2u + 15u) & ~15u);
}
__host__ __device__ __forceinline__ PermTables pm_tables(const PermArgs& a, unsigned char* smem, uint32_t es) {
    const uint32_t tile = (a.lds_elems * es + 4095u) & ~4095u;
    PermTables tb;
    tb.pos_src = reinterpret_cast<uint32_t*>(smem + tile);
    tb.row1_src = tb.pos_src + a.run1_len;
    tb.row2_dst = tb.row1_src + a.rows1;
    tb.pos_lds = reinterpret_cast<uint16_t*>(tb.row2_dst + a.rows2);
    tb.row1_lds = tb.pos_lds + a.run1_len;
    tb.row2_lds = tb.row1_lds + a.rows1;
    return tb;
}

// Lanes per row for load width v and store width w: one lane per load or store of a run, at most the block.
static inline void rt_permute_set_widths(PermArgs* a, uint32_t v, uint32_t w) {
    auto lanes = [](uint64_t items) { return (uint32_t)(items < 1 ? 1 : items > (uint64_t)kPBlock ? (uint64_t)kPBlock : items); };
    a->lpr1 = lanes((a->run1_len + v - 1) / v);
    a->lpr2 = lanes(((uint64_t)a->dkd.t * a->run2_unit + w - 1) / w);
    a->per_iter1 = kPBlock / a->lpr1;
    a->per_iter2 = kPBlock / a->lpr2;
    a->lpr1_div = make_fastdiv(a->lpr1);
    a->lpr2_div = make_fastdiv(a->lpr2);
}

}  // namespace rtp
