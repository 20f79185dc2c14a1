// LDS-transpose kernel of the broadcast family (see rt_broadcast.hip for the family and rt_broadcast_common.h for the
// shared definitions).  One input has its unit-|stride| dim `t` somewhere other than dst's inner dim (a permuted, possibly
// reversed view, e.g. `a + b.transpose()` or the row-major copy of a permuted tensor): reading it along dst's inner dim would
// touch one cache line per element.  A block instead gathers a (TK x TL) tile of it along *its* unit-stride dim with
// 16-byte loads (full 128-byte lines), scatters the elements into LDS transposed, and then writes full rows of dst with
// 16-byte non-temporal stores, combining with the other input on the way.
//
// Measured on MI355X, 16384 x 16384 f32: transposing copy 6.0 TB/s in a standalone kernel of this shape (tile 32 x 256,
// tile index along dst's inner dim fastest); square 64 x 64 tiles reach 5.1 TB/s and 32 x 32 tiles 3.9 TB/s.  What matters
// is 1 KiB contiguous per written row, whole lines per gathered row, no register array indexed at run time (that puts it in
// scratch memory) and three to four resident blocks per CU (100-170 VGPRs, 33 KiB of LDS).
#include "rt_broadcast_common.h"

using namespace rtb;

namespace {

constexpr int kTBlock = 256;
constexpr int kTWaves = kTBlock / RT_WAVE;
constexpr int kTSteps = 8;                   // 16-byte vectors of dst written by each lane per tile

// Tile geometry by element size.  4 bytes and more: 32 elements along the transposed operand's unit-stride dim (a 128-byte line
// of f32) by 64 vectors along dst's inner dim, so a wave writes 1 KiB of one dst row per instruction.  1-byte elements: 64 by 32
// vectors (512 bytes of two dst rows per wave instruction), because 32 elements along t would gather only a quarter of a line
// per inner-dim position (32768^2 u8 add with a transposed operand: 5.5 TB/s against 4.8 with the 32 x 64 shape).  2-byte
// elements keep 32 x 64: the 64 x 32 shape measured +1 % on that add and -7 % on the transposing copy.
template <class T> struct TileGeom {
    static constexpr int LPR = sizeof(T) == 1 ? 32 : 64;           // lanes (vectors) per tile row
    static constexpr int RPI = RT_WAVE / LPR;                       // dst rows per wave instruction
    static constexpr int TK = kTSteps * kTWaves * RPI;              // tile extent along dim t
    static constexpr int TL = LPR * (16 / (int)sizeof(T));          // tile extent along dst's inner dim
};

struct TileArgs {
    uint32_t L, K, G;               // inner length, extent of dim t, extent of the loop dim (1 if none)
    uint32_t gchunk, nchunks, ktiles, ltiles;
    FastDiv32 ltiles_div, ktiles_div, nchunks_div;
    int nouter;
    uint32_t oshape[RT_MAX_RANK];
    FastDiv32 odiv[RT_MAX_RANK];
    int64_t ostride[3][RT_MAX_RANK];              // by role, see below
    // strides by role: 0 = the transposed input, 1 = the other input, 2 = dst
    int64_t gstride[3], tstride[3], istride[3];   // loop dim, dim t, inner dim
    uint32_t x_is_left;             // the transposed input is the left operand of the op
    uint32_t nt_xt;                 // every element of the transposed input is used once -> non-temporal gather (tr_add 0.536 -> 0.509 ms)
};

// xt / xo: the transposed and the other input.  OM = access mode of the other input along the inner dim; VG = the transposed
// input can be read with aligned 16-byte loads along dim t (else element loads).
template <class T, int OP, int OM, bool VG>
__global__ __launch_bounds__(kTBlock) void bin_tile_kernel(const T* xt, const T* xo, T* d, TileArgs a) {
    constexpr int N = 16 / sizeof(T);
    constexpr int LPR = TileGeom<T>::LPR, RPI = TileGeom<T>::RPI, TK = TileGeom<T>::TK, TL = TileGeom<T>::TL;
    __shared__ alignas(16) T tile[TK][TL + N];
    // blockIdx -> (outer index, chunk of the loop dim, tile along t, tile along the inner dim); the last is the fastest so
    // that blocks running together write neighbouring 1 KiB pieces of the same dst rows
    uint32_t b = blockIdx.x;
    uint32_t q = fd_div(b, a.ltiles_div);
    const uint32_t ltile = b - q * a.ltiles;
    b = q;
    q = fd_div(b, a.ktiles_div);
    const uint32_t ktile = b - q * a.ktiles;
    b = q;
    q = fd_div(b, a.nchunks_div);
    const uint32_t chunk = b - q * a.nchunks;
    uint32_t rem = q;
    int64_t offx = 0, offo = 0, offd = 0;
#pragma unroll
    for (int k = RT_MAX_RANK - 1; k >= 0; --k) {
        if (k < a.nouter) {
            uint32_t qq = fd_div(rem, a.odiv[k]);
            uint32_t c = rem - qq * a.oshape[k];
            offx += (int64_t)c * a.ostride[0][k];
            offo += (int64_t)c * a.ostride[1][k];
            offd += (int64_t)c * a.ostride[2][k];
            rem = qq;
        }
    }
    xt += offx;
    xo += offo;
    T* dp = d + offd;
    const uint32_t k0 = ktile * TK, l0 = ltile * TL;
    const uint32_t g_begin = chunk * a.gchunk;
    const uint32_t g_end = min(a.G, g_begin + a.gchunk);
    const bool xt_fixed = a.gstride[0] == 0;
    const bool o_fixed = a.tstride[1] == 0;
    const bool x_left = a.x_is_left != 0;

    const uint32_t lane = threadIdx.x & (RT_WAVE - 1), wv = threadIdx.x / RT_WAVE;
    const uint32_t c = l0 + (lane % LPR) * N;                // first inner column of this lane's vectors
    const uint32_t krow = wv * RPI + lane / LPR;             // this lane's tile row in step 0; step i adds i * kTWaves * RPI
    const bool full_vec = c + N <= a.L;

    for (uint32_t g = g_begin; g < g_end; ++g) {
        // rows of the other operand for this step: issued before the gather so that both are in flight together (issuing them
        // after the gather's LDS writes saves 40 VGPRs and reaches four waves per SIMD instead of three, but measured 3 % slower)
        Vec16<T> ov[kTSteps] = {};
        if constexpr (OP != kOpCopy) {
            if (full_vec) {
                const T* orow = xo + (int64_t)g * a.gstride[1];
#pragma unroll
                for (int i = 0; i < kTSteps; ++i) {
                    const uint32_t k = min(k0 + krow + i * kTWaves * RPI, a.K - 1);
                    if (i == 0 || !o_fixed) ov[i] = load_vec<T, OM>(orow + (int64_t)k * a.tstride[1], c, a.istride[1]);
                    else ov[i] = ov[0];
                }
            }
        }
        if (g == g_begin || !xt_fixed) {
            if (g != g_begin) __syncthreads();
            const T* xg = xt + (int64_t)g * a.gstride[0];
            if constexpr (VG && sizeof(T) < 4) {
                // 1- and 2-byte elements: a lane loads the vectors of P = 4 / sizeof(T) neighbouring inner-dim positions and
                // transposes P x P blocks in registers (byte permutes), so that every LDS write carries a full 32-bit word of P
                // neighbouring columns of one tile row.  One LDS write per element, as the 4-byte path does, costs 2x / 4x the
                // LDS instructions per byte moved and held a 16384^2 add with a transposed operand at 4.5 (i16) / 2.5 (u8) TB/s
                // (now 5.7 / 5.5).
                constexpr int P = 4 / sizeof(T);
                constexpr int VT = TK / N;                     // vectors per tile row along t
                constexpr int GPI = kTBlock / VT;              // groups of P inner-dim positions covered per iteration
                constexpr int IT = TL / (GPI * P);
                const uint32_t tq = threadIdx.x % VT, lg = threadIdx.x / VT;
                const uint32_t t0 = k0 + tq * N;
                const bool fwd = a.tstride[0] > 0;
                const T* src = xg + (fwd ? (int64_t)t0 : -(int64_t)(t0 + N - 1));
                rt_u32x4 grp[IT][P];
#pragma unroll
                for (int i = 0; i < IT; ++i) {
#pragma unroll
                    for (int p = 0; p < P; ++p) {
                        const uint32_t col = min(l0 + (lg + i * GPI) * P + p, a.L - 1);
                        if (t0 < a.K) {                        // K is a multiple of N on this path
                            const rt_u32x4* q4 = reinterpret_cast<const rt_u32x4*>(src + (int64_t)col * a.istride[0]);
                            grp[i][p] = rt_ld16_dyn(q4, a.nt_xt != 0);
                        } else {
                            grp[i][p] = rt_u32x4{0, 0, 0, 0};
                        }
                    }
                }
#pragma unroll
                for (int i = 0; i < IT; ++i) {
                    const uint32_t colw = (lg + i * GPI) * P;
                    auto put = [&](int j, uint32_t w) {       // word of the P columns at element j of the loaded vectors
                        *reinterpret_cast<uint32_t*>(&tile[tq * N + (fwd ? j : N - 1 - j)][colw]) = w;
                    };
#pragma unroll
                    for (int k = 0; k < 4; ++k) {
                        if constexpr (P == 2) {
                            put(2 * k, __builtin_amdgcn_perm(grp[i][1][k], grp[i][0][k], 0x05040100u));
                            put(2 * k + 1, __builtin_amdgcn_perm(grp[i][1][k], grp[i][0][k], 0x07060302u));
                        } else {
                            const uint32_t p0 = __builtin_amdgcn_perm(grp[i][1][k], grp[i][0][k], 0x05010400u);   // a0 b0 a1 b1
                            const uint32_t p1 = __builtin_amdgcn_perm(grp[i][1][k], grp[i][0][k], 0x07030602u);   // a2 b2 a3 b3
                            const uint32_t q0 = __builtin_amdgcn_perm(grp[i][3][k], grp[i][2][k], 0x05010400u);   // c0 d0 c1 d1
                            const uint32_t q1 = __builtin_amdgcn_perm(grp[i][3][k], grp[i][2][k], 0x07030602u);   // c2 d2 c3 d3
                            put(4 * k, __builtin_amdgcn_perm(q0, p0, 0x05040100u));
                            put(4 * k + 1, __builtin_amdgcn_perm(q0, p0, 0x07060302u));
                            put(4 * k + 2, __builtin_amdgcn_perm(q1, p1, 0x05040100u));
                            put(4 * k + 3, __builtin_amdgcn_perm(q1, p1, 0x07060302u));
                        }
                    }
                }
            } else if constexpr (VG) {
                // 16-byte loads along dim t: 8 lanes cover one 128-byte line of 4-byte elements, a wave instruction covers 8
                // tile rows; the N elements of a vector go to N different tile rows, one LDS write each
                constexpr int VT = TK / N;                     // vectors per tile row along t
                constexpr int LPI = kTBlock / VT;              // inner-dim positions covered per iteration
                constexpr int IT = TL / LPI;
                const uint32_t tq = threadIdx.x % VT, ls = threadIdx.x / VT;
                const uint32_t t0 = k0 + tq * N;
                const bool fwd = a.tstride[0] > 0;
                // lowest address of the vector: element t0 when dim t ascends in memory, element t0+N-1 when it descends
                const T* src = xg + (fwd ? (int64_t)t0 : -(int64_t)(t0 + N - 1));
                Vec16<T> grp[IT];
#pragma unroll
                for (int i = 0; i < IT; ++i) {
                    const uint32_t col = min(l0 + ls + i * LPI, a.L - 1);
                    if (t0 < a.K) {                            // K is a multiple of N on this path
                        const Vec16<T>* p = reinterpret_cast<const Vec16<T>*>(src + (int64_t)col * a.istride[0]);
                        grp[i] = rt_ld16_dyn(p, a.nt_xt != 0);
                    } else {
                        grp[i] = Vec16<T>{};
                    }
                }
#pragma unroll
                for (int i = 0; i < IT; ++i) {
#pragma unroll
                    for (int j = 0; j < N; ++j) tile[tq * N + (fwd ? j : N - 1 - j)][ls + i * LPI] = grp[i].e[j];
                }
            } else {
                // element loads with lanes along dim t (32 consecutive lanes read one 128-byte line of 4-byte elements); each
                // lane collects the N elements of one 16-byte group of a tile row and writes the group with one LDS store
                const uint32_t tk = threadIdx.x % TK, grp0 = threadIdx.x / TK;
                constexpr int kGroups = LPR / (kTBlock / TK);                      // groups per tile row / rows of lanes = 8
                constexpr int kBatch = sizeof(T) >= 4 ? 4 : 1;                     // groups in flight per lane
                const T* src = xg + (int64_t)min(k0 + tk, a.K - 1) * a.tstride[0];
#pragma unroll 1
                for (int i0 = 0; i0 < kGroups; i0 += kBatch) {
                    Vec16<T> grp[kBatch];
#pragma unroll
                    for (int i = 0; i < kBatch; ++i) {
                        const uint32_t col = l0 + (grp0 + (i0 + i) * (kTBlock / TK)) * N;
#pragma unroll
                        for (int j = 0; j < N; ++j) grp[i].e[j] = src[(int64_t)min(col + j, a.L - 1) * a.istride[0]];
                    }
#pragma unroll
                    for (int i = 0; i < kBatch; ++i)
                        *reinterpret_cast<Vec16<T>*>(&tile[tk][(grp0 + (i0 + i) * (kTBlock / TK)) * N]) = grp[i];
                }
            }
            __syncthreads();
        }
        if (c >= a.L) continue;
        T* drow = dp + (int64_t)g * a.gstride[2];
        if (full_vec) {
#pragma unroll
            for (int i = 0; i < kTSteps; ++i) {
                const uint32_t kk = krow + i * kTWaves * RPI;
                if (k0 + kk < a.K) {
                    const Vec16<T> xv = *reinterpret_cast<const Vec16<T>*>(&tile[kk][(lane % LPR) * N]);
                    Vec16<T> out;
                    if (x_left) { out = xv; bin_apply_vec<OP, T>(out, ov[i]); }
                    else { out = ov[i]; bin_apply_vec<OP, T>(out, xv); }
                    rt_st16u_nt<T>(drow + (int64_t)(k0 + kk) * a.tstride[2] + c, __builtin_bit_cast(rt_u32x4, out));
                }
            }
        } else {
            // ragged end of a row: element accesses
            const T* orow = xo + (int64_t)g * a.gstride[1];
            for (int i = 0; i < kTSteps; ++i) {
                const uint32_t kk = krow + i * kTWaves * RPI;
                if (k0 + kk < a.K) {
                    for (uint32_t cc = c; cc < a.L; ++cc) {
                        T xe = tile[kk][cc - l0];
                        T oe = xe;
                        if constexpr (OP != kOpCopy) oe = (orow + (int64_t)(k0 + kk) * a.tstride[1])[(int64_t)cc * a.istride[1]];
                        drow[(int64_t)(k0 + kk) * a.tstride[2] + cc] = x_left ? bin_apply<OP, T>(xe, oe) : bin_apply<OP, T>(oe, xe);
                    }
                }
            }
        }
    }
}

}  // namespace

namespace rtb {

template <class T, int OP>
bool tile_try(rt_ctx* ctx, const NdDesc& dsc, uint64_t count, const T* l, const T* r, T* d, int32_t* status) {
    constexpr int64_t N = 16 / sizeof(T);
    const int rank = dsc.rank;
    // rows shorter than a quarter of the tile's columns would leave most lanes of every wave idle
    if (!(rank >= 2 && count < (1ull << 31) && dsc.stride[2][rank - 1] == 1 && dsc.shape[rank - 1] >= TileGeom<T>::TL / 4)) return false;
    auto transposed_dim = [&](int o) -> int {
        int64_t is = dsc.stride[o][rank - 1];
        if (is == 0 || is == 1) return -1;
        for (int k = rank - 2; k >= 0; --k)
            if ((dsc.stride[o][k] == 1 || dsc.stride[o][k] == -1) && dsc.shape[k] >= 16) return k;
        return -1;
    };
    const int tl = transposed_dim(0), tr = (OP == kOpCopy) ? -1 : transposed_dim(1);
    // When the transposed input does not move along some long outer dim, the row kernel gathers it once per block and
    // reuses it from registers for 16 output rows, which measured faster than this kernel looping over that dim (2 GiB add
    // with a 32 MiB permuted operand: 0.37 ms against 0.45 ms).  Copying
    // such an input into a compact temporary first and then running the plain stride-0 broadcast was also measured (2 GiB
    // add, 32 MiB permuted operand): 0.024 ms copy + 0.347 ms add against 0.368 ms for the hoisted gather.
    auto hoistable = [&](int o) {
        for (int k = 0; k < rank - 1; ++k)
            if (dsc.stride[o][k] == 0 && dsc.shape[k] >= 8) return true;
        return false;
    };
    if ((tl >= 0) == (tr >= 0) || hoistable(tl >= 0 ? 0 : 1)) return false;
    const int xt = tl >= 0 ? 0 : 1, o = 1 - xt, tdim = tl >= 0 ? tl : tr;
    int om;
    {
        int64_t is = dsc.stride[o][rank - 1];
        om = is == 0 ? (int)M_BCAST : (is == 1 ? (int)M_VEC : (int)M_ELEM);
    }
    TileArgs a;
    memset(&a, 0, sizeof(a));
    a.L = (uint32_t)dsc.shape[rank - 1];
    a.K = (uint32_t)dsc.shape[tdim];
    int gdim = -1;
    for (int k = 0; k < rank - 1; ++k)
        if (k != tdim && dsc.stride[xt][k] == 0 && (gdim < 0 || dsc.shape[k] > dsc.shape[gdim])) gdim = k;
    a.G = gdim >= 0 ? (uint32_t)dsc.shape[gdim] : 1;
    const int role[3] = {xt, o, 2};               // operand index of each role
    a.x_is_left = xt == 0 ? 1u : 0u;
    for (int q = 0; q < 3; ++q) {
        a.gstride[q] = gdim >= 0 ? dsc.stride[role[q]][gdim] : 0;
        a.tstride[q] = dsc.stride[role[q]][tdim];
        a.istride[q] = dsc.stride[role[q]][rank - 1];
    }
    uint64_t outer = 1;
    for (int k = 0; k < rank - 1; ++k) {
        if (k == gdim || k == tdim) continue;
        a.oshape[a.nouter] = (uint32_t)dsc.shape[k];
        a.odiv[a.nouter] = make_fastdiv((uint32_t)dsc.shape[k]);
        for (int q = 0; q < 3; ++q) a.ostride[q][a.nouter] = dsc.stride[role[q]][k];
        outer *= (uint64_t)dsc.shape[k];
        a.nouter++;
    }
    for (int k = a.nouter; k < RT_MAX_RANK; ++k) { a.oshape[k] = 1; a.odiv[k] = make_fastdiv(1); }
    const uint32_t TL = TileGeom<T>::TL, TK = TileGeom<T>::TK;
    a.ktiles = (a.K + TK - 1) / TK;
    a.ltiles = (a.L + TL - 1) / TL;
    // loop-dim steps per block: the gathered tile is reused for all of them; keep enough blocks to fill the chip
    uint32_t gchunk = a.G;
    const uint64_t want_blocks = (uint64_t)ctx->num_cus * 16;
    while (gchunk > 8 && outer * a.ktiles * a.ltiles * ((a.G + gchunk - 1) / gchunk) < want_blocks) gchunk = (gchunk + 1) / 2;
    a.gchunk = gchunk;
    a.nchunks = (a.G + gchunk - 1) / gchunk;
    a.ltiles_div = make_fastdiv(a.ltiles);
    a.ktiles_div = make_fastdiv(a.ktiles);
    a.nchunks_div = make_fastdiv(a.nchunks);
    bool vec_gather = false;
    {
        const T* xbase = (xt == 0 ? l : r) + dsc.offset[xt];
        const int64_t ts = dsc.stride[xt][tdim];
        // every vector starts at (base + multiples of N) for an ascending dim t, and ends there for a descending one
        const T* first = ts > 0 ? xbase : xbase - (N - 1);
        bool ok = (reinterpret_cast<uintptr_t>(first) & 15) == 0 && (a.K % (uint32_t)N) == 0 && TK % (uint32_t)N == 0;
        bool xstream = true;
        for (int k = 0; k < rank; ++k) {
            if (k != tdim) ok = ok && mult_of(dsc.stride[xt][k], N);
            xstream = xstream && dsc.stride[xt][k] != 0;
        }
        vec_gather = ok;
        a.nt_xt = xstream ? 1u : 0u;
    }
    const uint64_t blocks = outer * a.nchunks * a.ktiles * a.ltiles;
    if (blocks >= (1ull << 31)) return false;
    const T* xp = (xt == 0 ? l : r) + dsc.offset[xt];
    const T* op = (xt == 0 ? r : l) + dsc.offset[o];
    T* dp = d + dsc.offset[2];
    hipStream_t s = ctx->stream;
    dim3 grid((unsigned)blocks), blk(kTBlock);
#define RT_TILE(OM) do { if (vec_gather) hipLaunchKernelGGL((bin_tile_kernel<T, OP, OM, true>), grid, blk, 0, s, xp, op, dp, a); \
                         else hipLaunchKernelGGL((bin_tile_kernel<T, OP, OM, false>), grid, blk, 0, s, xp, op, dp, a); } while (0)
    if constexpr (OP == kOpCopy) {
        RT_TILE(M_BCAST);                        // the copy op has no second input
    } else {
        if (om == M_VEC) RT_TILE(M_VEC); else if (om == M_BCAST) RT_TILE(M_BCAST); else RT_TILE(M_ELEM);
    }
#undef RT_TILE
    hipError_t e = hipGetLastError();
    *status = e == hipSuccess ? RT_OK : rt_hip_fail(e, "broadcast (tile kernel) launch");
    return true;
}

}  // namespace rtb

// ---- interleaved -> planar copy ---------------------------------------------------------------------------------------------
// dst (.., C, M) row-major, src strides (.., 1, C): the C planes of dst are C interleaved channels of src.  Reading src along
// dst's inner dim (what the row kernel does) steps C elements per lane and fetches every line C times, once per plane, far
// enough apart to miss every cache: (3, 2^28/3) f32 measured 0.86 ms.  Here a block reads the contiguous run of B * C source
// elements once with 16-byte loads, scatters it into LDS as C rows of B, and writes the C row pieces with 16-byte stores: 0.41 ms.
namespace {

constexpr uint32_t kPlanarBytes = 32768;

struct PlanarArgs {
    uint32_t C, M, B, pitch, ntiles;    // channels, plane length, positions per block, LDS row pitch, tiles per plane
    FastDiv32 c_div, ntiles_div;
    int64_t d_cstride;                  // dst stride between planes
    uint32_t vec_store;                 // plane pieces start 16-byte aligned
    int nouter;
    uint32_t oshape[RT_MAX_RANK];
    FastDiv32 odiv[RT_MAX_RANK];
    int64_t ostride[2][RT_MAX_RANK];    // 0 = src, 1 = dst
};

template <class T>
__global__ __launch_bounds__(kTBlock) void planar_copy_kernel(const T* __restrict__ src, T* __restrict__ dst, PlanarArgs a) {
    constexpr uint32_t N = 16 / sizeof(T);
    __shared__ alignas(16) T tile[kPlanarBytes / sizeof(T)];
    uint32_t b = blockIdx.x;
    uint32_t q = fd_div(b, a.ntiles_div);
    const uint32_t tl = b - q * a.ntiles;
    uint32_t rem = q;
    int64_t offs = 0, offd = 0;
#pragma unroll
    for (int k = RT_MAX_RANK - 1; k >= 0; --k) {
        if (k < a.nouter) {
            uint32_t qq = fd_div(rem, a.odiv[k]);
            uint32_t c = rem - qq * a.oshape[k];
            offs += (int64_t)c * a.ostride[0][k];
            offd += (int64_t)c * a.ostride[1][k];
            rem = qq;
        }
    }
    const uint32_t n0 = tl * a.B;
    const uint32_t nb = min(a.B, a.M - n0);
    const uint32_t ne = nb * a.C;
    const T* p = src + offs + (int64_t)n0 * a.C;
    auto put = [&](uint32_t e, T v) {
        const uint32_t n = fd_div(e, a.c_div);
        tile[(e - n * a.C) * a.pitch + n] = v;
    };
    uint32_t head = (uint32_t)(((16 - (reinterpret_cast<uintptr_t>(p) & 15)) & 15) / sizeof(T));
    if (head > ne) head = ne;
    if (threadIdx.x < head) put(threadIdx.x, p[threadIdx.x]);
    const uint32_t nvec = (ne - head) / N;
    const Vec16<T>* pv = reinterpret_cast<const Vec16<T>*>(p + head);
    constexpr int U = 4;
    for (uint32_t v0 = threadIdx.x; v0 < nvec; v0 += U * kTBlock) {
        Vec16<T> x[U];
#pragma unroll
        for (int u = 0; u < U; ++u)
            if (v0 + u * kTBlock < nvec) x[u] = rt_ld16_nt(pv + v0 + u * kTBlock);
#pragma unroll
        for (int u = 0; u < U; ++u) {
            if (v0 + u * kTBlock < nvec) {
#pragma unroll
                for (uint32_t j = 0; j < N; ++j) put(head + (v0 + u * kTBlock) * N + j, x[u].e[j]);
            }
        }
    }
    const uint32_t tb = head + nvec * N;
    if (tb + threadIdx.x < ne) put(tb + threadIdx.x, p[tb + threadIdx.x]);
    __syncthreads();
    T* dp = dst + offd + n0;
    const uint32_t nbv = a.vec_store ? nb / N : 0;             // whole vectors of a plane piece
    for (uint32_t ch = 0; ch < a.C; ++ch) {
        const T* row = tile + ch * a.pitch;
        T* drow = dp + (int64_t)ch * a.d_cstride;
        for (uint32_t v = threadIdx.x; v < nbv; v += kTBlock)
            rt_st16_nt(reinterpret_cast<Vec16<T>*>(drow) + v, *reinterpret_cast<const Vec16<T>*>(row + v * N));
        for (uint32_t n = nbv * N + threadIdx.x; n < nb; n += kTBlock) drow[n] = row[n];
    }
}

}  // namespace

namespace rtb {

template <class T>
bool planar_copy_try(rt_ctx* ctx, const NdDesc& dsc, uint64_t count, const T* src, T* dst, int32_t* status) {
    constexpr uint32_t N = 16 / sizeof(T);
    const int rank = dsc.rank;
    if (rank < 2 || count >= (1ull << 31)) return false;
    const int64_t C = dsc.shape[rank - 2], M = dsc.shape[rank - 1];
    if (C < 2 || C >= 16 || M < 256) return false;             // from 16 channels on the transposing tile kernel does better
    if (dsc.stride[2][rank - 1] != 1 || dsc.stride[0][rank - 2] != 1 || dsc.stride[0][rank - 1] != C) return false;
    PlanarArgs a;
    memset(&a, 0, sizeof(a));
    a.C = (uint32_t)C;
    a.M = (uint32_t)M;
    // LDS rows of B + N elements (16 bytes of padding keep the 16-byte LDS reads aligned and spread the rows over the banks),
    // B a multiple of 32
    uint32_t B = ((uint32_t)(kPlanarBytes / sizeof(T)) / a.C - N) / 32 * 32;
    if (B > (uint32_t)M) B = ((uint32_t)M + 31) / 32 * 32;
    if (B < 32) return false;
    a.B = B;
    a.pitch = B + N;
    a.ntiles = (a.M + B - 1) / B;
    a.c_div = make_fastdiv(a.C);
    a.ntiles_div = make_fastdiv(a.ntiles);
    a.d_cstride = dsc.stride[2][rank - 2];
    uint64_t outer = 1;
    bool vec = (reinterpret_cast<uintptr_t>(dst + dsc.offset[2]) & 15) == 0 && a.d_cstride % N == 0;
    for (int k = 0; k < rank - 2; ++k) {
        a.oshape[a.nouter] = (uint32_t)dsc.shape[k];
        a.odiv[a.nouter] = make_fastdiv((uint32_t)dsc.shape[k]);
        a.ostride[0][a.nouter] = dsc.stride[0][k];
        a.ostride[1][a.nouter] = dsc.stride[2][k];
        vec = vec && dsc.stride[2][k] % N == 0;
        outer *= (uint64_t)dsc.shape[k];
        a.nouter++;
    }
    for (int k = a.nouter; k < RT_MAX_RANK; ++k) { a.oshape[k] = 1; a.odiv[k] = make_fastdiv(1); }
    a.vec_store = vec ? 1u : 0u;
    const uint64_t blocks = outer * a.ntiles;
    if (blocks >= (1ull << 31)) return false;
    hipLaunchKernelGGL((planar_copy_kernel<T>), dim3((unsigned)blocks), dim3(kTBlock), 0, ctx->stream, src + dsc.offset[0], dst + dsc.offset[2], a);
    hipError_t e = hipGetLastError();
    *status = e == hipSuccess ? RT_OK : rt_hip_fail(e, "planar copy launch");
    return true;
}

template bool planar_copy_try<uint8_t>(rt_ctx*, const NdDesc&, uint64_t, const uint8_t*, uint8_t*, int32_t*);
template bool planar_copy_try<uint16_t>(rt_ctx*, const NdDesc&, uint64_t, const uint16_t*, uint16_t*, int32_t*);
template bool planar_copy_try<uint32_t>(rt_ctx*, const NdDesc&, uint64_t, const uint32_t*, uint32_t*, int32_t*);
template bool planar_copy_try<uint64_t>(rt_ctx*, const NdDesc&, uint64_t, const uint64_t*, uint64_t*, int32_t*);

}  // namespace rtb

namespace rtb {

// every (element type, op) that rt_broadcast.hip instantiates
#define RT_TILE_INST(T, OP) template bool tile_try<T, OP>(rt_ctx*, const NdDesc&, uint64_t, const T*, const T*, T*, int32_t*);
#define RT_TILE_INST_ASM(T) RT_TILE_INST(T, RT_ADD) RT_TILE_INST(T, RT_SUB) RT_TILE_INST(T, RT_MUL)
RT_TILE_INST_ASM(uint8_t) RT_TILE_INST_ASM(uint16_t) RT_TILE_INST_ASM(uint32_t) RT_TILE_INST_ASM(uint64_t)
RT_TILE_INST_ASM(float) RT_TILE_INST_ASM(double) RT_TILE_INST_ASM(boolean_t) RT_TILE_INST_ASM(u128_t)
RT_TILE_INST(uint8_t, RT_DIV) RT_TILE_INST(int8_t, RT_DIV) RT_TILE_INST(uint16_t, RT_DIV) RT_TILE_INST(int16_t, RT_DIV)
RT_TILE_INST(uint32_t, RT_DIV) RT_TILE_INST(int32_t, RT_DIV) RT_TILE_INST(uint64_t, RT_DIV) RT_TILE_INST(int64_t, RT_DIV)
RT_TILE_INST(float, RT_DIV) RT_TILE_INST(double, RT_DIV)
RT_TILE_INST(uint8_t, kOpCopy) RT_TILE_INST(uint16_t, kOpCopy) RT_TILE_INST(uint32_t, kOpCopy) RT_TILE_INST(uint64_t, kOpCopy)

}  // namespace rtb
