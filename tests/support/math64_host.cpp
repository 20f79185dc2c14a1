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
