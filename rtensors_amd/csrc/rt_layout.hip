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
    unsigned __int128 n = 1;
    bool empty = false;
    for (int i = 0; i < rank; ++i) {
        if (shape[i] == 0) empty = true;
        n *= shape[i];
        if (n > (unsigned __int128)INT64_MAX) {
            // keep multiplying only to detect zeros; an overflowing non-empty shape is refused below
            n = (unsigned __int128)INT64_MAX + 1;
        }
    }
    if (empty) {
        if (offset > len) return rt_fail(RT_E_OUT_OF_BOUNDS, "%s: offset %llu is past the end of a buffer with %llu elements", what,
                                         (unsigned long long)offset, (unsigned long long)len);
        if (count) *count = 0;
        return RT_OK;
    }
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

int32_t rt_collapse(int nops, int rank, const uint64_t* shape, const int64_t* const* strides, const uint64_t* offsets,
                    bool reorder, int key, NdDesc* out) {
    struct Dim { int64_t n; int64_t s[3]; };
    std::vector<Dim> dims;
    dims.reserve((size_t)rank);
    int64_t off[3] = {0, 0, 0};
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
    std::vector<Dim> merged;
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
    if ((int)merged.size() > RT_MAX_RANK)
        return rt_fail(RT_E_RANK, "layout needs %d dims after collapsing; at most %d are supported", (int)merged.size(), RT_MAX_RANK);
    out->rank = (int)merged.size();
    for (int i = 0; i < RT_MAX_RANK; ++i) {
        out->shape[i] = i < out->rank ? merged[(size_t)i].n : 1;
        for (int o = 0; o < 3; ++o) out->stride[o][i] = i < out->rank ? merged[(size_t)i].s[o] : 0;
    }
    for (int o = 0; o < 3; ++o) out->offset[o] = off[o];
    return RT_OK;
}
