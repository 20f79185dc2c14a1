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
__global__ __launch_bounds__(kTBlock) void bin_tile_kernel(const T* xt, const T* xo, T* d, TileArgs a, int32_t* fault) {
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
    int64_t off3[3];
    rt_outer_offsets<3>(q, a.nouter, a.oshape, a.odiv, a.ostride, off3);
    const int64_t offx = off3[0], offo = off3[1], offd = off3[2];
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
                // K is a multiple of N on this path; tile rows past the end of dim t hold a repeat of its last vector and are never stored
                const uint32_t t0 = min(k0 + tq * N, a.K - N);
                const bool fwd = a.tstride[0] > 0;
                const T* src = xg + (fwd ? (int64_t)t0 : -(int64_t)(t0 + N - 1));
                rt_u32x4 grp[IT][P];
                // one branch on the launch-wide non-temporal hint around all loads, so that they are in flight together
                auto load_all = [&](auto nt_c) {
#pragma unroll
                    for (int i = 0; i < IT; ++i) {
#pragma unroll
                        for (int p = 0; p < P; ++p) {
                            const uint32_t col = min(l0 + (lg + i * GPI) * P + p, a.L - 1);
                            const rt_u32x4* q4 = reinterpret_cast<const rt_u32x4*>(src + (int64_t)col * a.istride[0]);
                            if constexpr (decltype(nt_c)::value) grp[i][p] = rt_ld16_nt(q4); else grp[i][p] = rt_ld16(q4);
                        }
                    }
                };
                if (a.nt_xt) load_all(std::true_type{}); else load_all(std::false_type{});
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
                // K is a multiple of N on this path; tile rows past the end of dim t hold a repeat of its last vector and are never stored
                const uint32_t t0 = min(k0 + tq * N, a.K - N);
                const bool fwd = a.tstride[0] > 0;
                // lowest address of the vector: element t0 when dim t ascends in memory, element t0+N-1 when it descends
                const T* src = xg + (fwd ? (int64_t)t0 : -(int64_t)(t0 + N - 1));
                Vec16<T> grp[IT];
                auto load_all = [&](auto nt_c) {
#pragma unroll
                    for (int i = 0; i < IT; ++i) {
                        const uint32_t col = min(l0 + ls + i * LPI, a.L - 1);
                        const Vec16<T>* p = reinterpret_cast<const Vec16<T>*>(src + (int64_t)col * a.istride[0]);
                        if constexpr (decltype(nt_c)::value) grp[i] = rt_ld16_nt(p); else grp[i] = rt_ld16(p);
                    }
                };
                if (a.nt_xt) load_all(std::true_type{}); else load_all(std::false_type{});
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
                    if (x_left) { out = xv; bin_apply_vec<OP, T>(out, ov[i], fault); }
                    else { out = ov[i]; bin_apply_vec<OP, T>(out, xv, fault); }
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
                        drow[(int64_t)(k0 + kk) * a.tstride[2] + cc] = x_left ? bin_apply<OP, T>(xe, oe, fault) : bin_apply<OP, T>(oe, xe, fault);
                    }
                }
            }
        }
    }
}


// ---- staged kernel: 4- and 8-byte elements, vector gather -------------------------------------------------------------------------
// The same job as bin_tile_kernel in the shape that measured fastest for 4-byte elements on MI355X: 512 lanes, a tile of 16 rows
// (along dim t) by 64 vectors (1 KiB) of dst's inner dim, two stores per lane and no loop over other dims -- a dim along which the
// transposed input does not move is just one more outer dim, so blocks that run together write one compact window of dst and the
// transposed input's tile is re-read from cache for every index of that dim.  (Keeping the tile for several indices of such a dim
// makes every lane store to places megabytes apart: config 3b, x (16,1,512,1024) permuted + reversed plus y (1,64,1,1024): 0.90 of
// peak with one index per block, 0.82 with two, 0.73 with four, 0.76 for the row kernel that gathers x element-wise and keeps it
// in registers for 16 indices.)  The gather reads N vectors of N elements along dim t, transposes the N x N block in registers and
// writes N whole vectors to LDS.
constexpr int kSVecs = 64;                    // tile columns in 16-byte vectors (one wave writes one row piece)
// Tile rows (along dim t), two per wave.  WIDE = 32 rows of 4-byte elements, 1024 lanes: a whole 128-byte line of the transposed
// input per inner-dim position, for an input that is streamed from memory once (16384^2 f32: a + b.transpose() 0.74 -> 0.79 of
// peak, transposing copy 0.68 -> 0.76 against 16 rows).  Otherwise 16 rows, 512 lanes: an input that is re-read from cache for
// every index of a dim along which it does not move (config 3b: 0.89 with 16 rows, 0.87 with 32).
template <class T, bool WIDE> struct StageGeom {
    static constexpr int kRows = (WIDE && sizeof(T) == 4) ? 32 : 16;
    static constexpr int kWaves = kRows / 2;
    static constexpr int kBlock = kWaves * RT_WAVE;
};

// At most two outer dims besides dim t and the inner dim; everything a wave needs from the kernel arguments is fetched in one batch.
struct StageArgs {
    uint32_t L, K, ltiles;
    FastDiv32 ltiles_div;
    // strides by role (0 = the transposed input, 1 = the other input, 2 = dst) along dim t, the inner dim and the two outer dims;
    // every offset inside an operand fits 32 bits (checked on the host)
    int32_t ts[3], is[3], o0s[3], o1s[3];
    uint32_t x_is_left, nt_xt;
};

constexpr int M_BOTH = 3;    // mode of the other input in the staged kernel: transposed like the first one

// grid: x = inner-dim tile + ltiles * (tile along t), y = index along the inner outer dim, z = index along the outer one.  (When t is
// an outer dim of dst beyond those two -- the row-major copy of a (64, 1024, 4096) tensor permuted to (4096, 64, 1024) -- carrying
// the tile along t in y or z instead, so that the blocks in flight write one compact window of dst, only moves the scatter to the
// reads: 0.67 of peak either way.)
// OM == M_BOTH: the other input is transposed in the same way; both are gathered, combined in registers and staged as one tile.
// FULL: K and L are whole numbers of tiles, so no index is clamped and no row or vector is tested against an edge.
// NTO: the other input is a row-wise operand that is read exactly once: non-temporal loads (a compile-time choice, see load_raw).
template <class T, int OP, int OM, bool WIDE, bool FULL, bool NTO>
__global__ __launch_bounds__((StageGeom<T, WIDE>::kBlock)) void bin_stage_kernel(const T* xt, const T* xo, T* d, StageArgs a, int32_t* fault) {
    constexpr int N = 16 / sizeof(T);
    constexpr int kSRows = StageGeom<T, WIDE>::kRows, kSWaves = StageGeom<T, WIDE>::kWaves, kSBlock = StageGeom<T, WIDE>::kBlock;
    constexpr int TK = kSRows, TL = kSVecs * N, KQ = TK / N, NU = kSVecs * KQ, RPL = TK / kSWaves;
    static_assert(TK % N == 0 && TK % kSWaves == 0, "tile shape");
    __shared__ alignas(16) T tile[TK][TL + N];
    uint32_t L = a.L, K = a.K, ltiles = a.ltiles, x_left = a.x_is_left, nt_xt = a.nt_xt, lm = a.ltiles_div.mul, lsh = a.ltiles_div.shift;
    int32_t ts0 = a.ts[0], ts1 = a.ts[1], ts2 = a.ts[2], is0 = a.is[0], is1 = a.is[1];
    int32_t p0 = a.o0s[0], p1 = a.o0s[1], p2 = a.o0s[2], q0 = a.o1s[0], q1 = a.o1s[1], q2 = a.o1s[2];
    RT_PIN(L); RT_PIN(K); RT_PIN(ltiles); RT_PIN(x_left); RT_PIN(nt_xt); RT_PIN(lm); RT_PIN(lsh);
    RT_PIN(ts0); RT_PIN(ts1); RT_PIN(ts2); RT_PIN(is0); RT_PIN(is1);
    RT_PIN(p0); RT_PIN(p1); RT_PIN(p2); RT_PIN(q0); RT_PIN(q1); RT_PIN(q2);
    RT_TOUCH(xt); RT_TOUCH(xo); RT_TOUCH(d);
    const uint32_t ktile = (uint32_t)(((uint64_t)__umulhi(blockIdx.x, lm) + blockIdx.x) >> lsh);
    const uint32_t ltile = blockIdx.x - ktile * ltiles;
    const int32_t i0 = (int32_t)blockIdx.y, i1 = (int32_t)blockIdx.z;
    xt += i1 * q0 + i0 * p0;
    xo += i1 * q1 + i0 * p1;
    T* dp = d + (i1 * q2 + i0 * p2);
    const uint32_t k0 = ktile * TK, l0 = ltile * TL;
    const uint32_t lane = threadIdx.x & (RT_WAVE - 1);
    const uint32_t wv = (uint32_t)__builtin_amdgcn_readfirstlane((int)(threadIdx.x / RT_WAVE));
    const uint32_t c = l0 + lane * N;
    const bool full_vec = FULL || c + N <= L;
    // rows of the other input, issued before the gather so that both are in flight together
    Vec16<T> ov[RPL] = {};
    if constexpr (OP != kOpCopy && OM != M_BOTH) {
        if (full_vec) {
#pragma unroll
            for (int i = 0; i < RPL; ++i) {
                const uint32_t k = FULL ? k0 + wv * RPL + i : min(k0 + wv * RPL + i, K - 1);
                if constexpr (OM == M_VEC && NTO) ov[i] = __builtin_bit_cast(Vec16<T>, rt_ld16u<T, true>(xo + (int32_t)k * ts1 + c));
                else ov[i] = load_vec<T, OM>(xo + (int32_t)k * ts1, c, is1);
            }
        }
    }
    // (the non-temporal hint is a launch-wide fact: one branch around the whole gather, not one per load, so that all loads of a
    // lane are in flight together)
    auto gather = [&](auto nt_c) {
        constexpr bool NTG = decltype(nt_c)::value;
        const bool fwd = ts0 > 0;
#pragma unroll
        for (int u0 = 0; u0 < NU; u0 += kSBlock) {
            const uint32_t v = u0 + threadIdx.x;
            if (NU % kSBlock == 0 || v < (uint32_t)NU) {
                const uint32_t lq = v / KQ, tq = v % KQ;
                const uint32_t t0 = FULL ? k0 + tq * N : min(k0 + tq * N, K - N);   // K % N == 0 here; rows past the end of dim t are never stored
                // lowest address of a vector: element t0 when dim t ascends in memory, element t0 + N - 1 when it descends
                const T* src = xt + (fwd ? (int64_t)t0 : -(int64_t)(t0 + N - 1));
                Vec16<T> g[N];
#pragma unroll
                for (int j = 0; j < N; ++j) {
                    const uint32_t col = FULL ? l0 + lq * N + j : min(l0 + lq * N + j, L - 1);
                    const Vec16<T>* gp = reinterpret_cast<const Vec16<T>*>(src + (int32_t)col * is0);
                    if constexpr (NTG) g[j] = rt_ld16_nt(gp); else g[j] = rt_ld16(gp);
                }
                if constexpr (OM == M_BOTH) {
                    const T* src2 = xo + (fwd ? (int64_t)t0 : -(int64_t)(t0 + N - 1));
                    Vec16<T> h[N];
#pragma unroll
                    for (int j = 0; j < N; ++j) {
                        const uint32_t col = FULL ? l0 + lq * N + j : min(l0 + lq * N + j, L - 1);
                        const Vec16<T>* hp = reinterpret_cast<const Vec16<T>*>(src2 + (int32_t)col * is1);
                        if constexpr (NTG) h[j] = rt_ld16_nt(hp); else h[j] = rt_ld16(hp);
                    }
#pragma unroll
                    for (int j = 0; j < N; ++j) {
                        if (x_left) bin_apply_vec<OP, T>(g[j], h[j], fault);
                        else { bin_apply_vec<OP, T>(h[j], g[j], fault); g[j] = h[j]; }
                    }
                }
#pragma unroll
                for (int e = 0; e < N; ++e) {
                    Vec16<T> w;
#pragma unroll
                    for (int j = 0; j < N; ++j) w.e[j] = g[j].e[e];
                    *reinterpret_cast<Vec16<T>*>(&tile[tq * N + (fwd ? e : N - 1 - e)][lq * N]) = w;
                }
            }
        }
    };
    if (nt_xt) gather(std::true_type{}); else gather(std::false_type{});
    __syncthreads();
    if (!FULL && c >= L) return;
#pragma unroll
    for (int i = 0; i < RPL; ++i) {
        const uint32_t kk = wv * RPL + i;
        if (!FULL && k0 + kk >= K) continue;
        T* drow = dp + (int32_t)(k0 + kk) * ts2;
        if (full_vec) {
            const Vec16<T> xv = *reinterpret_cast<const Vec16<T>*>(&tile[kk][lane * N]);
            Vec16<T> out;
            if constexpr (OM == M_BOTH) out = xv;
            else if (x_left) { out = xv; bin_apply_vec<OP, T>(out, ov[i], fault); }
            else { out = ov[i]; bin_apply_vec<OP, T>(out, xv, fault); }
            rt_st16u_nt<T>(drow + c, __builtin_bit_cast(rt_u32x4, out));
        } else {
            // ragged end of a row: element accesses
            for (uint32_t cc = c; cc < L; ++cc) {
                T xe = tile[kk][cc - l0];
                if constexpr (OM == M_BOTH) {
                    drow[cc] = xe;
                } else {
                    T oe = xe;
                    if constexpr (OP != kOpCopy) oe = (xo + (int32_t)(k0 + kk) * ts1)[(int32_t)cc * is1];
                    drow[cc] = x_left ? bin_apply<OP, T>(xe, oe, fault) : bin_apply<OP, T>(oe, xe, fault);
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
    if (tl < 0 && tr < 0) return false;
    // both inputs transposed: only when they are transposed alike (a.transpose() + b.transpose()); the staged kernel combines them
    // before the transposition
    const bool both = tl >= 0 && tr >= 0;
    if (both && (tl != tr || dsc.stride[0][tl] != dsc.stride[1][tr])) return false;
    const int xt = tl >= 0 ? 0 : 1, o = 1 - xt, tdim = tl >= 0 ? tl : tr;
    int om;
    {
        int64_t is = dsc.stride[o][rank - 1];
        om = both ? M_BOTH : (is == 0 ? (int)M_BCAST : (is == 1 ? (int)M_VEC : (int)M_ELEM));
    }
    // 4- and 8-byte elements whose transposed input can be read with aligned 16-byte vectors along dim t: the staged kernel, also
    // when that input does not move along some dim.  2-byte elements only in that last case, where the input is re-read from cache
    // (config 3b at i16: 0.62 -> 0.74 of peak); when it is streamed once the tile kernel below is faster for them (16384^2 i16
    // a + b.transpose(): 0.68 against 0.54), as it is for 1-byte elements in both cases.
    if constexpr (sizeof(T) >= 2) {
        const T* xbase = (xt == 0 ? l : r) + dsc.offset[xt];
        const int64_t ts = dsc.stride[xt][tdim];
        const T* first = ts > 0 ? xbase : xbase - (N - 1);
        bool ok = (reinterpret_cast<uintptr_t>(first) & 15) == 0 && dsc.shape[tdim] % N == 0;
        bool xstream = true;
        for (int k = 0; k < rank; ++k) {
            if (k != tdim) ok = ok && mult_of(dsc.stride[xt][k], N);
            xstream = xstream && dsc.stride[xt][k] != 0;
        }
        if (sizeof(T) == 2 && (xstream || both)) ok = false;
        if (both) {                                                // the same conditions for the second transposed input
            const T* obase = (o == 0 ? l : r) + dsc.offset[o];
            const T* ofirst = ts > 0 ? obase : obase - (N - 1);
            ok = ok && (reinterpret_cast<uintptr_t>(ofirst) & 15) == 0;
            for (int k = 0; k < rank; ++k) {
                if (k != tdim) ok = ok && mult_of(dsc.stride[o][k], N);
                xstream = xstream && dsc.stride[o][k] != 0;
            }
        }
        for (int q = 0; q < 3 && ok; ++q) {                       // 32-bit offsets inside every operand
            uint64_t reach = 0;
            for (int k = 0; k < rank; ++k) reach += (uint64_t)(dsc.shape[k] - 1) * (uint64_t)(dsc.stride[q][k] < 0 ? -dsc.stride[q][k] : dsc.stride[q][k]);
            ok = reach < (1ull << 31);
        }
        if (ok && rank <= 4) {
            StageArgs a;
            memset(&a, 0, sizeof(a));
            a.L = (uint32_t)dsc.shape[rank - 1];
            a.K = (uint32_t)dsc.shape[tdim];
            const int role[3] = {xt, o, 2};
            a.x_is_left = xt == 0 ? 1u : 0u;
            a.nt_xt = xstream ? 1u : 0u;
            int od[2], nod = 0;                                    // the outer dims, innermost first
            for (int k = rank - 2; k >= 0; --k)
                if (k != tdim) od[nod++] = k;
            const uint64_t n0 = nod >= 1 ? (uint64_t)dsc.shape[od[0]] : 1ull, n1 = nod >= 2 ? (uint64_t)dsc.shape[od[1]] : 1ull;
            for (int q = 0; q < 3; ++q) {
                a.ts[q] = (int32_t)dsc.stride[role[q]][tdim];
                a.is[q] = (int32_t)dsc.stride[role[q]][rank - 1];
                a.o0s[q] = nod >= 1 ? (int32_t)dsc.stride[role[q]][od[0]] : 0;
                a.o1s[q] = nod >= 2 ? (int32_t)dsc.stride[role[q]][od[1]] : 0;
            }
            const bool wide = xstream && sizeof(T) == 4;
            const uint32_t kSRows = wide ? 32u : 16u, kSBlock = kSRows / 2 * RT_WAVE;
            const uint32_t ktiles = (a.K + kSRows - 1) / kSRows;
            a.ltiles = (a.L + kSVecs * (uint32_t)N - 1) / (kSVecs * (uint32_t)N);
            a.ltiles_div = make_fastdiv(a.ltiles);
            const uint64_t gx = (uint64_t)ktiles * a.ltiles;
            if (gx < (1ull << 31) && n0 <= 65535 && n1 <= 65535) {
                const T* xp = (xt == 0 ? l : r) + dsc.offset[xt];
                const T* op = (xt == 0 ? r : l) + dsc.offset[o];
                T* dp = d + dsc.offset[2];
                dim3 grid((unsigned)gx, (unsigned)n0, (unsigned)n1), blk(kSBlock);
                const bool full = a.K % kSRows == 0 && a.L % (kSVecs * (uint32_t)N) == 0;
                bool other_once = om == M_VEC;
                for (int k = 0; k < rank; ++k) other_once = other_once && dsc.stride[o][k] != 0;
                auto go = [&](auto wide_c, auto full_c) {
                    constexpr bool W = decltype(wide_c)::value, F = decltype(full_c)::value;
                    if constexpr (OP == kOpCopy) {
                        hipLaunchKernelGGL((bin_stage_kernel<T, OP, M_BCAST, W, F, false>), grid, blk, 0, ctx->stream, xp, op, dp, a, fault_of<T, OP>(ctx));
                    } else {
                        if (om == M_BOTH) hipLaunchKernelGGL((bin_stage_kernel<T, OP, M_BOTH, W, F, false>), grid, blk, 0, ctx->stream, xp, op, dp, a, fault_of<T, OP>(ctx));
                        else if (om == M_VEC && other_once) hipLaunchKernelGGL((bin_stage_kernel<T, OP, M_VEC, W, F, true>), grid, blk, 0, ctx->stream, xp, op, dp, a, fault_of<T, OP>(ctx));
                        else if (om == M_VEC) hipLaunchKernelGGL((bin_stage_kernel<T, OP, M_VEC, W, F, false>), grid, blk, 0, ctx->stream, xp, op, dp, a, fault_of<T, OP>(ctx));
                        else if (om == M_BCAST) hipLaunchKernelGGL((bin_stage_kernel<T, OP, M_BCAST, W, F, false>), grid, blk, 0, ctx->stream, xp, op, dp, a, fault_of<T, OP>(ctx));
                        else hipLaunchKernelGGL((bin_stage_kernel<T, OP, M_ELEM, W, F, false>), grid, blk, 0, ctx->stream, xp, op, dp, a, fault_of<T, OP>(ctx));
                    }
                };
                auto go_w = [&](auto wide_c) { if (full) go(wide_c, std::true_type{}); else go(wide_c, std::false_type{}); };
                if constexpr (sizeof(T) == 4) { if (wide) go_w(std::true_type{}); else go_w(std::false_type{}); }
                else go_w(std::false_type{});
                hipError_t e = hipGetLastError();
                *status = e == hipSuccess ? RT_OK : rt_hip_fail(e, "broadcast (staged tile kernel) launch");
                return true;
            }
        }
    }
    if (both || hoistable(xt)) return false;
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
        if (sizeof(T) == 2 && (xstream || both)) ok = false;
        if (both) {                                                // the same conditions for the second transposed input
            const T* obase = (o == 0 ? l : r) + dsc.offset[o];
            const T* ofirst = ts > 0 ? obase : obase - (N - 1);
            ok = ok && (reinterpret_cast<uintptr_t>(ofirst) & 15) == 0;
            for (int k = 0; k < rank; ++k) {
                if (k != tdim) ok = ok && mult_of(dsc.stride[o][k], N);
                xstream = xstream && dsc.stride[o][k] != 0;
            }
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
#define RT_TILE(OM) do { if (vec_gather) hipLaunchKernelGGL((bin_tile_kernel<T, OP, OM, true>), grid, blk, 0, s, xp, op, dp, a, fault_of<T, OP>(ctx)); \
                         else hipLaunchKernelGGL((bin_tile_kernel<T, OP, OM, false>), grid, blk, 0, s, xp, op, dp, a, fault_of<T, OP>(ctx)); } while (0)
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
    int64_t off2[2];
    rt_outer_offsets<2>(q, a.nouter, a.oshape, a.odiv, a.ostride, off2);
    const int64_t offs = off2[0], offd = off2[1];
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
RT_TILE_INST(float, RT_DIV) RT_TILE_INST(double, RT_DIV) RT_TILE_INST(u128_t, RT_DIV) RT_TILE_INST(i128_t, RT_DIV)
RT_TILE_INST(uint8_t, kOpCopy) RT_TILE_INST(uint16_t, kOpCopy) RT_TILE_INST(uint32_t, kOpCopy) RT_TILE_INST(uint64_t, kOpCopy)

}  // namespace rtb
