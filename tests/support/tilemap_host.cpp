// Host-only check of the tiled traversal of the streaming kernels (TileMap, rtensors_amd/csrc/rt_common.h), built by
// tests/test_tilemap_host.py with hipcc's host pass.  For every case on stdin -- "phase_bytes nvec nthreads piece_bytes rows stride_bytes" --
// it walks every lane of every block of the launch and prints "ok blocks" when
//   * the lanes that own a vector own the vectors 0 .. nvec - 1 exactly once (the map is a permutation),
//   * the block-wise form of the index (rt_tile_index_block) agrees with the lane-by-lane form (rt_tile_index) for every lane,
// and a line that names the first violation otherwise.
#include <stdint.h>
#include <stdio.h>

#include <vector>

#include "../../rtensors_amd/csrc/rt_common.h"

int main() {
    unsigned long long phase, nvec;
    unsigned nthreads, piece, rows, stride;
    while (scanf("%llu %llu %u %u %u %u", &phase, &nvec, &nthreads, &piece, &rows, &stride) == 6) {
        const void* body = reinterpret_cast<const void*>((uintptr_t)0x7f0000000000ull + phase);
        const TileMap m = rt_make_tilemap(body, (size_t)nvec, nthreads, piece, rows, stride);
        const size_t blocks = rt_tilemap_blocks(m, (size_t)nvec, nthreads);
        std::vector<uint8_t> seen((size_t)nvec, 0);
        const char* bad = nullptr;
        size_t owned = 0;
        for (size_t b = 0; b < blocks + 2 && !bad; ++b) {              // two blocks past the grid must own nothing
            for (uint32_t t = 0; t < nthreads; ++t) {
                size_t i = 0, j = 0;
                const bool has = rt_tile_index_block(m, (uint32_t)b, nthreads, t, (size_t)nvec, &i);
                const bool has2 = rt_tile_index(m, (uint32_t)b, nthreads, t, (size_t)nvec, &j);
                if (has != has2 || (has && i != j)) { bad = "the two forms disagree"; break; }
                if (!has) continue;
                if (b >= blocks) { bad = "a block beyond the grid owns a vector"; break; }
                if (i >= nvec) { bad = "index out of range"; break; }
                if (seen[i]) { bad = "a vector is owned twice"; break; }
                seen[i] = 1;
                owned += 1;
            }
        }
        if (!bad && owned != nvec) bad = "a vector is owned by no lane";
        if (bad) printf("bad %s\n", bad);
        else printf("ok %zu\n", blocks);
    }
    return 0;
}
