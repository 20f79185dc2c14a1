// Host build of the device's 128-bit division (rtensors_amd/csrc/rt_div128.h) for the CPU test that holds it to exact integer
// arithmetic.  Operands and quotients cross as 16 little-endian bytes each.
#include <stddef.h>
#include <string.h>

#include "../../rtensors_amd/csrc/rt_div128.h"

extern "C" void div128_many(int is_signed, size_t n, const unsigned char* a, const unsigned char* b, unsigned char* q) {
    for (size_t i = 0; i < n; ++i) {
        rt_u128 x, y, r;
        memcpy(&x, a + 16 * i, 16);
        memcpy(&y, b + 16 * i, 16);
        r = is_signed ? (rt_u128)rt_idiv128((rt_i128)x, (rt_i128)y) : rt_udiv128(x, y);
        memcpy(q + 16 * i, &r, 16);
    }
}

extern "C" unsigned long long div_128_by_64(unsigned long long u1, unsigned long long u0, unsigned long long v) {
    return rt_div_128_by_64(u1, u0, v);
}
