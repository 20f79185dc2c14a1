// Host-only driver for the descriptor checks of the library (rtensors_amd/csrc/rt_layout.hip), built with AddressSanitizer and
// UndefinedBehaviorSanitizer by tests/test_layout_fuzz_host.py.  Reads one case per line from stdin, answers one line per case:
//   V offset len rank shape[rank] strides[rank]                      -> status count out_rank out_offset shape[out_rank] strides[out_rank]
//   O elem_size len rank shape[rank] a_offset a_strides[rank] b_offset b_strides[rank]   -> status meet same
// The few internals rt_layout.hip needs from the rest of the library (error plumbing, the scratch buffer of the rank-generic path,
// which no case here reaches) are defined below, so that nothing but the unit under test is linked.
#include <stdarg.h>
#include <stdint.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>

#include <string>
#include <vector>

#include <hip/hip_runtime_api.h>

#include "../../include/rt_hip.h"

struct rt_ctx;
int32_t rt_fail(int32_t status, const char* fmt, ...) {
    char buf[512];
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(buf, sizeof(buf), fmt, ap);        // the format strings and their arguments are exercised too
    va_end(ap);
    return status;
}
int32_t rt_hip_fail(hipError_t, const char*) { return RT_E_HIP; }
int32_t rt_scratch(rt_ctx*, size_t, void**) { return RT_E_HIP; }

int main() {
    char kind;
    std::vector<uint64_t> shape;
    std::vector<int64_t> sa, sb;
    while (scanf(" %c", &kind) == 1) {
        if (kind == 'V') {
            unsigned long long offset, len;
            int rank;
            if (scanf("%llu %llu %d", &offset, &len, &rank) != 3) return 2;
            const int r = rank < 0 ? 0 : rank;
            // exactly `rank` entries on the heap: an access past them is an AddressSanitizer report
            uint64_t* sh = (uint64_t*)malloc(sizeof(uint64_t) * (size_t)(r ? r : 1));
            int64_t* st = (int64_t*)malloc(sizeof(int64_t) * (size_t)(r ? r : 1));
            for (int i = 0; i < r; ++i) { unsigned long long v; if (scanf("%llu", &v) != 1) return 2; sh[i] = v; }
            for (int i = 0; i < r; ++i) { long long v; if (scanf("%lld", &v) != 1) return 2; st[i] = v; }
            uint64_t count = 0;
            int32_t orank = 0;
            int64_t oshape[RT_MAX_RANK], ostr[RT_MAX_RANK], ooff = 0;
            const int32_t status = rt_debug_check_view(offset, rank, sh, st, len, &count, &orank, oshape, ostr, &ooff);
            printf("%d %llu %d %lld", status, (unsigned long long)count, orank, (long long)ooff);
            if (status == RT_OK) {
                for (int i = 0; i < orank; ++i) printf(" %lld", (long long)oshape[i]);
                for (int i = 0; i < orank; ++i) printf(" %lld", (long long)ostr[i]);
            }
            printf("\n");
            free(sh);
            free(st);
        } else if (kind == 'O') {
            int es, rank;
            unsigned long long len, aoff, boff;
            if (scanf("%d %llu %d", &es, &len, &rank) != 3) return 2;
            shape.assign((size_t)rank, 0); sa.assign((size_t)rank, 0); sb.assign((size_t)rank, 0);
            for (int i = 0; i < rank; ++i) { unsigned long long v; if (scanf("%llu", &v) != 1) return 2; shape[(size_t)i] = v; }
            if (scanf("%llu", &aoff) != 1) return 2;
            for (int i = 0; i < rank; ++i) { long long v; if (scanf("%lld", &v) != 1) return 2; sa[(size_t)i] = v; }
            if (scanf("%llu", &boff) != 1) return 2;
            for (int i = 0; i < rank; ++i) { long long v; if (scanf("%lld", &v) != 1) return 2; sb[(size_t)i] = v; }
            int32_t meet = -1, same = -1;
            const int32_t status = rt_debug_check_overlap(es, rank, shape.data(), aoff, sa.data(), boff, sb.data(), len, &meet, &same);
            printf("%d %d %d\n", status, meet, same);
        } else {
            return 3;
        }
    }
    return 0;
}
