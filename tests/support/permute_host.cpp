// Host-only walk of the permuting tile copy (rtensors_amd/csrc/rt_permute.h), built by tests/test_permute_host.py with hipcc's host
// pass and the address sanitizer.  For every case on stdin -- "es rank shape[rank] stride[rank] offset" (a view of a buffer that is
// exactly as long as the view reaches) -- it plans the copy, runs the three stages of every block lane by lane with an LDS tile and
// tables of exactly the planned sizes, and prints "ok blocks store-width load-width" when dst equals the row-major copy of the view for the planned
// store width and for single-element stores; "skip" when the plan declines the case; a line naming the first mismatch otherwise.
#include <stdint.h>
#include <stdio.h>

#include <vector>

#include "../../rtensors_amd/csrc/rt_permute.h"

using namespace rtp;

template <class T, int W, int V>
static void run_blocks(PermArgs a, uint64_t blocks, const T* src, T* dst) {
    rt_permute_set_widths(&a, V, W);
    // one allocation of exactly the launch's dynamic LDS, carved up as the kernel does
    std::vector<unsigned char> smem(rt_permute_lds_bytes(a, (uint32_t)sizeof(T)));
    unsigned char* tile = smem.data();
    const PermTables tb = pm_tables(a, smem.data(), (uint32_t)sizeof(T));
    for (uint64_t blk = 0; blk < blocks; ++blk) {
        const uint32_t which = pm_remap(a, (uint32_t)blk);
        const PermBlock b = pm_block(a, which);
        for (uint32_t t = 0; t < (uint32_t)kPBlock; ++t) pm_stage0<T>(a, which, t, tb);
        for (uint32_t t = 0; t < (uint32_t)kPBlock; ++t) pm_stage1<T, V>(src, a, b, t, tile, tb);
        for (uint32_t t = 0; t < (uint32_t)kPBlock; ++t) pm_stage2<T, W>(dst, a, b, t, tile, tb, PmCopy{});
    }
}

template <class T>
static void one_case(int rank, const int64_t* shape, const int64_t* stride, int64_t offset) {
    constexpr uint32_t N = 16 / sizeof(T);
    int64_t dstride[RT_MAX_RANK], lo = 0, hi = 0, count = 1;
    for (int k = rank - 1; k >= 0; --k) { dstride[k] = count; count *= shape[k]; }
    for (int k = 0; k < rank; ++k) {
        const int64_t r = (shape[k] - 1) * stride[k];
        if (r < 0) lo += r; else hi += r;
    }
    if (offset + lo != 0) { printf("bad the view does not start at the buffer's first element\n"); return; }
    std::vector<T> src((size_t)(hi - lo + 1));
    for (size_t i = 0; i < src.size(); ++i) src[i] = (T)(i * 2654435761u + 12345u);
    PermArgs a;
    uint64_t blocks = 0;
    if (!rt_permute_plan(rank, shape, stride, dstride, (uint32_t)sizeof(T), &a, &blocks)) { printf("skip\n"); return; }
    if (rt_permute_lds_bytes(a, (uint32_t)sizeof(T)) > 48 * 1024 || a.run1_len > kPTabMax || a.rows1 > kPRowMax || a.rows2 > kPRowMax) { printf("bad the plan exceeds the LDS arrays\n"); return; }
    std::vector<T> want((size_t)count);
    {
        std::vector<int64_t> idx(rank, 0);
        for (int64_t i = 0; i < count; ++i) {
            int64_t off = offset;
            for (int k = 0; k < rank; ++k) off += idx[k] * stride[k];
            want[(size_t)i] = src[(size_t)off];
            for (int k = rank - 1; k >= 0; --k) { if (++idx[k] < shape[k]) break; idx[k] = 0; }
        }
    }
    const uint32_t w = rt_permute_store_width(a, N);
    constexpr uint32_t kWord = sizeof(T) < 4 ? 4 / sizeof(T) : 1;
    const uint32_t v = rt_permute_load_width(a, N);
    for (int pass = 0; pass < 2; ++pass) {
        std::vector<T> dst((size_t)count, (T)0x5a);
        uint32_t used = 1;
        const T* sp = src.data() + offset;
        if (pass == 0 && w == N) {
            if (v == N) run_blocks<T, (int)N, (int)N>(a, blocks, sp, dst.data()); else run_blocks<T, (int)N, 1>(a, blocks, sp, dst.data());
            used = N;
        } else if (pass == 0 && kWord > 1 && w >= kWord) {
            if (v == N) run_blocks<T, (int)kWord, (int)N>(a, blocks, sp, dst.data()); else run_blocks<T, (int)kWord, 1>(a, blocks, sp, dst.data());
            used = kWord;
        } else if (pass == 0) {
            if (v == N) run_blocks<T, 1, (int)N>(a, blocks, sp, dst.data()); else run_blocks<T, 1, 1>(a, blocks, sp, dst.data());
        } else {
            run_blocks<T, 1, 1>(a, blocks, sp, dst.data());
        }
        for (int64_t i = 0; i < count; ++i)
            if (dst[(size_t)i] != want[(size_t)i]) { printf("bad element %lld differs (pass %d, store width %u, load width %u)\n", (long long)i, pass, used, v); return; }
        if (pass == 1) printf("ok %llu %u %u\n", (unsigned long long)blocks, w, v);
    }
}

int main() {
    int es, rank;
    while (scanf("%d %d", &es, &rank) == 2) {
        int64_t shape[RT_MAX_RANK], stride[RT_MAX_RANK], offset = 0;
        if (rank < 1 || rank > RT_MAX_RANK) return 2;
        for (int k = 0; k < rank; ++k) { long long v; if (scanf("%lld", &v) != 1) return 2; shape[k] = v; }
        for (int k = 0; k < rank; ++k) { long long v; if (scanf("%lld", &v) != 1) return 2; stride[k] = v; }
        { long long v; if (scanf("%lld", &v) != 1) return 2; offset = v; }
        switch (es) {
            case 1: one_case<uint8_t>(rank, shape, stride, offset); break;
            case 2: one_case<uint16_t>(rank, shape, stride, offset); break;
            case 4: one_case<uint32_t>(rank, shape, stride, offset); break;
            case 8: one_case<uint64_t>(rank, shape, stride, offset); break;
            default: return 2;
        }
        fflush(stdout);
    }
    return 0;
}
