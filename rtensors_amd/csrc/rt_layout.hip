// Host-side descriptor validation and canonicalisation.
// The checks are those the reference's remote server applies before it lets a request reach a backend
// (backend/remote/server.rs:241-295): a descriptor that addresses anything outside its buffer is refused with an
// error code instead of being launched.
#include "rt_common.h"

#include <algorithm>

int32_t rt_check_extent(const char* what, uint64_t offset, int rank, const uint64_t* shape, const int64_t* strides,
                        uint64_t len, uint64_t* count) {
    if (rank < 0 || rank > RT_MAX_INPUT_RANK) return rt_fail(RT_E_INVALID, "%s: rank %d outside 0..%d", what, rank, RT_MAX_INPUT_RANK);
    if (rank > 0 && (!shape || !strides)) return rt_fail(RT_E_INVALID, "%s: null shape/strides", what);
    // every address of a view that passes lies in [0, len): with len within int64 the signed 64-bit arithmetic of the canonicalisation
    // and of the kernels cannot overflow
    if (len > (uint64_t)INT64_MAX) return rt_fail(RT_E_INVALID, "%s: a buffer of %llu elements is beyond signed 64-bit indexing", what, (unsigned long long)len);
    // element count as the reference folds it (checked_mul over usize, left to right: a product that overflows before a zero dim is
    // met is refused, backend/remote/server.rs:246-248, 272-275)
    unsigned __int128 n = 1;
    bool empty = false;
    for (int i = 0; i < rank; ++i) {
        if (shape[i] == 0) empty = true;
        n *= shape[i];
        if (n > (unsigned __int128)UINT64_MAX) return rt_fail(RT_E_INVALID, "%s: shape has too many elements", what);
    }
    if (empty) {
        if (offset > len) return rt_fail(RT_E_OUT_OF_BOUNDS, "%s: offset %llu is past the end of a buffer with %llu elements", what,
                                         (unsigned long long)offset, (unsigned long long)len);
        if (count) *count = 0;
        return RT_OK;
    }
    // kernels index with signed 64-bit arithmetic
    if (n > (unsigned __int128)INT64_MAX) return rt_fail(RT_E_INVALID, "%s: shape has too many elements", what);
    __int128 lo = (__int128)offset, hi = (__int128)offset;
    for (int i = 0; i < rank; ++i) {
        __int128 span = ((__int128)shape[i] - 1) * (__int128)strides[i];
        if (span < 0) lo += span; else hi += span;
    }
    if (lo < 0 || hi >= (__int128)len)
        return rt_fail(RT_E_OUT_OF_BOUNDS, "%s: addresses elements %lld..=%lld of a buffer with %llu elements", what,
                       (long long)lo, (long long)hi, (unsigned long long)len);
    if (count) *count = (uint64_t)n;
    return RT_OK;
}

ByteSpan rt_view_span(const void* base, int elem_size, uint64_t offset, int rank, const uint64_t* shape, const int64_t* strides) {
    __int128 lo = (__int128)offset, hi = (__int128)offset;
    for (int i = 0; i < rank; ++i) {
        __int128 span = ((__int128)shape[i] - 1) * (__int128)strides[i];
        if (span < 0) lo += span; else hi += span;
    }
    const uintptr_t b = reinterpret_cast<uintptr_t>(base);
    return ByteSpan{b + (uintptr_t)lo * (uintptr_t)elem_size, b + ((uintptr_t)hi + 1) * (uintptr_t)elem_size};
}

bool rt_same_view(const void* a, uint64_t a_offset, const int64_t* a_strides, const void* b, uint64_t b_offset, const int64_t* b_strides,
                  int rank, const uint64_t* shape) {
    if (a != b || a_offset != b_offset) return false;
    for (int i = 0; i < rank; ++i)
        if (shape[i] > 1 && a_strides[i] != b_strides[i]) return false;
    return true;
}

namespace {
struct Dim { int64_t n; int64_t s[3]; };

// size-1 dims dropped, dims optionally flipped / sorted by operand `key`, adjacent dims merged where every operand allows it
void collapse_dims(int nops, int rank, const uint64_t* shape, const int64_t* const* strides, const uint64_t* offsets, bool reorder, int key,
                   std::vector<Dim>* merged_out, int64_t (&off)[3]) {
    std::vector<Dim> dims;
    dims.reserve((size_t)rank);
    off[0] = off[1] = off[2] = 0;
    for (int o = 0; o < nops; ++o) off[o] = (int64_t)offsets[o];
    for (int i = 0; i < rank; ++i) {
        if (shape[i] == 1) continue;                        // size-1 dims never move an address
        Dim d;
        d.n = (int64_t)shape[i];
        for (int o = 0; o < 3; ++o) d.s[o] = o < nops ? strides[o][i] : 0;
        dims.push_back(d);
    }
    if (reorder) {
        for (auto& d : dims) {
            if (d.s[key] < 0) {                             // walk this dim backwards: same element set, ascending addresses
                for (int o = 0; o < nops; ++o) { off[o] += (d.n - 1) * d.s[o]; d.s[o] = -d.s[o]; }
            }
        }
        std::stable_sort(dims.begin(), dims.end(), [key](const Dim& a, const Dim& b) { return a.s[key] > b.s[key]; });
    }
    // merge dim i+1 into dim i when, for every operand, stepping dim i once equals stepping dim i+1 shape[i+1] times
    std::vector<Dim>& merged = *merged_out;
    merged.clear();
    for (const Dim& d : dims) {
        if (!merged.empty()) {
            Dim& p = merged.back();
            bool ok = true;
            for (int o = 0; o < nops; ++o) ok = ok && (p.s[o] == d.s[o] * d.n);
            if (ok) {
                p.n *= d.n;
                for (int o = 0; o < nops; ++o) p.s[o] = d.s[o];
                continue;
            }
        }
        merged.push_back(d);
    }
}
}  // namespace

int32_t rt_collapse(int nops, int rank, const uint64_t* shape, const int64_t* const* strides, const uint64_t* offsets,
                    bool reorder, int key, NdDesc* out) {
    std::vector<Dim> merged;
    int64_t off[3];
    collapse_dims(nops, rank, shape, strides, offsets, reorder, key, &merged, off);
    if ((int)merged.size() > RT_MAX_RANK)
        return rt_fail(RT_E_RANK, "layout needs %d dims after collapsing; the kernel-argument descriptor holds %d", (int)merged.size(), RT_MAX_RANK);
    out->rank = (int)merged.size();
    for (int i = 0; i < RT_MAX_RANK; ++i) {
        out->shape[i] = i < out->rank ? merged[(size_t)i].n : 1;
        for (int o = 0; o < 3; ++o) out->stride[o][i] = i < out->rank ? merged[(size_t)i].s[o] : 0;
    }
    for (int o = 0; o < 3; ++o) out->offset[o] = off[o];
    return RT_OK;
}

// The same for layouts that keep more than RT_MAX_RANK dims (the reference accepts rank <= 128, core/primitives.rs:377-383): the
// descriptor goes to device memory (the context's scratch buffer) as int64 words [shape[rank], stride0[rank], stride1[rank],
// stride2[rank]] and a rank-generic kernel reads it from there.  Caller holds ctx->mu.
int32_t rt_collapse_big(rt_ctx* ctx, int nops, int rank, const uint64_t* shape, const int64_t* const* strides, const uint64_t* offsets,
                        bool reorder, int key, BigDesc* out) {
    std::vector<Dim> merged;
    int64_t off[3];
    collapse_dims(nops, rank, shape, strides, offsets, reorder, key, &merged, off);
    const int r = (int)merged.size();
    std::vector<int64_t> words((size_t)r * 4);
    for (int i = 0; i < r; ++i) {
        words[(size_t)i] = merged[(size_t)i].n;
        for (int o = 0; o < 3; ++o) words[(size_t)(o + 1) * r + i] = merged[(size_t)i].s[o];
    }
    void* dev = nullptr;
    RT_TRY(rt_scratch(ctx, words.size() * sizeof(int64_t) + 8, &dev));
    // a pageable source is staged by the runtime before the call returns; the copy is ordered on the stream like the kernels
    RT_HIP(hipMemcpyAsync(dev, words.data(), words.size() * sizeof(int64_t), hipMemcpyHostToDevice, ctx->stream));
    RT_HIP(hipStreamSynchronize(ctx->stream));
    out->rank = r;
    out->words = (const int64_t*)dev;
    for (int o = 0; o < 3; ++o) out->offset[o] = off[o];
    return RT_OK;
}

// ---- the host-side checks on their own (no context, no device) ---------------------------------------------------------------------
extern "C" int32_t rt_debug_check_view(uint64_t offset, int32_t rank, const uint64_t* shape, const int64_t* strides, uint64_t len, uint64_t* out_count,
                                       int32_t* out_rank, int64_t* out_shape, int64_t* out_strides, int64_t* out_offset) {
    uint64_t count = 0;
    RT_TRY(rt_check_extent("view", offset, rank, shape, strides, len, &count));
    if (out_count) *out_count = count;
    if (out_rank) *out_rank = 0;
    if (count == 0) return RT_OK;
    NdDesc d;
    const int64_t* sp[1] = {strides};
    RT_TRY(rt_collapse(1, rank, shape, sp, &offset, /*reorder=*/true, 0, &d));
    if (out_rank) *out_rank = d.rank;
    for (int i = 0; i < d.rank; ++i) {
        if (out_shape) out_shape[i] = d.shape[i];
        if (out_strides) out_strides[i] = d.stride[0][i];
    }
    if (out_offset) *out_offset = d.offset[0];
    return RT_OK;
}

extern "C" int32_t rt_debug_check_overlap(int32_t elem_size, int32_t rank, const uint64_t* shape, uint64_t a_offset, const int64_t* a_strides, uint64_t b_offset,
                                          const int64_t* b_strides, uint64_t len, int32_t* out_meet, int32_t* out_same) {
    if (elem_size < 1 || elem_size > 16) return rt_fail(RT_E_INVALID, "element size %d", elem_size);
    uint64_t ca = 0, cb = 0;
    RT_TRY(rt_check_extent("view a", a_offset, rank, shape, a_strides, len, &ca));
    RT_TRY(rt_check_extent("view b", b_offset, rank, shape, b_strides, len, &cb));
    int meet = 0, same = 0;
    if (ca != 0) {
        // any base address will do: both views live in one buffer
        const void* base = reinterpret_cast<const void*>((uintptr_t)1 << 40);
        meet = rt_spans_meet(rt_view_span(base, elem_size, a_offset, rank, shape, a_strides), rt_view_span(base, elem_size, b_offset, rank, shape, b_strides)) ? 1 : 0;
        same = rt_same_view(base, a_offset, a_strides, base, b_offset, b_strides, rank, shape) ? 1 : 0;
    }
    if (out_meet) *out_meet = meet;
    if (out_same) *out_same = same;
    return RT_OK;
}
