// Host build of the device's hand-written f64 routines (rtensors_amd/csrc/rt_math64.h) for the CPU test that measures their error
// against 80-bit arithmetic.
#include <stddef.h>

#include "../../rtensors_amd/csrc/rt_math64.h"

extern "C" void log_many(size_t n, const double* x, double* y) {
    for (size_t i = 0; i < n; ++i) y[i] = rt_log_f64(x[i]);
}
extern "C" void log1p_many(size_t n, const double* x, double* y) {
    for (size_t i = 0; i < n; ++i) y[i] = rt_log1p_f64(x[i]);
}
extern "C" void asin_many(size_t n, const double* x, double* y) {
    for (size_t i = 0; i < n; ++i) y[i] = rt_asin_f64(x[i]);
}
extern "C" void acos_many(size_t n, const double* x, double* y) {
    for (size_t i = 0; i < n; ++i) y[i] = rt_acos_f64(x[i]);
}
extern "C" void sqrt_ge1_many(size_t n, const double* x, double* y) {
    for (size_t i = 0; i < n; ++i) y[i] = rt_sqrt_ge1_f64(x[i]);
}
extern "C" void rcp_many(size_t n, const double* x, double* y) {
    for (size_t i = 0; i < n; ++i) y[i] = rt_rcp_f64(x[i]);
}
extern "C" void quot_many(size_t n, const double* a, const double* d, double* y) {
    for (size_t i = 0; i < n; ++i) y[i] = rt_quot_f64(a[i], d[i]);
}
// sine and cosine of the reduced argument as the tangent's kernels form them (the quadrant is not applied)
extern "C" void sincos_kernel_many(size_t n, const double* x, double* s, double* c) {
    for (size_t i = 0; i < n; ++i) {
        int q;
        const double r = rt_pio2_reduce(x[i], &q);
        rt_sincos_kernel(r, &s[i], &c[i]);
    }
}
extern "C" void tan_many(size_t n, const double* x, double* y) {
    for (size_t i = 0; i < n; ++i) y[i] = rt_tan_f64(x[i]);
}
extern "C" void exp_nonpos_many(size_t n, const double* x, double* y) {
    for (size_t i = 0; i < n; ++i) y[i] = rt_exp_nonpos_f64(x[i]);
}
