// Counter-based synthetic data generator (benchmark / test support, separate from librt_hip.so).
// Element i of tensor `stream` under `seed` depends on (seed, stream, i) only, through splitmix64, so the same bits
// come out of this kernel and of the numpy implementation in rtensors_amd/datagen.py on any machine.
//   uniform f32 [-1,1): ((r >> 40) * 2^-23) - 1          uniform f64: ((r >> 11) * 2^-52) - 1
//   normal(0, sigma)  : Irwin-Hall, twelve 24-bit uniforms summed as integers, centred, times sigma * 2^-24
//   integers in [lo, hi]: lo + r mod (hi - lo + 1)
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace {

__host__ __device__ inline uint64_t splitmix64(uint64_t x) {
    x += 0x9E3779B97F4A7C15ull;
    uint64_t z = x;
    z = (z ^ (z >> 30)) * 0xBF58476D1CE4E5B9ull;
    z = (z ^ (z >> 27)) * 0x94D049BB133111EBull;
    return z ^ (z >> 31);
}

__host__ __device__ inline uint64_t stream_key(uint64_t seed, uint64_t stream) {
    return splitmix64(splitmix64(seed) ^ (stream * 0xD1342543DE82EF95ull));
}

__device__ inline int64_t irwin_hall(uint64_t key, uint64_t i) {
    int64_t s = 0;
#pragma unroll
    for (int k = 0; k < 6; ++k) {
        uint64_t r = splitmix64(key + i * 8 + (uint64_t)k);
        s += (int64_t)(r >> 40) + (int64_t)((r >> 16) & 0xFFFFFFull);
    }
    return s - 6 * (1ll << 24);
}

enum { DIST_UNIFORM = 0, DIST_NORMAL = 1, DIST_INT = 2 };
enum { DT_F32 = 10, DT_F64 = 11, DT_I32 = 6 };

__global__ void gen_f32(float* out, size_t n, uint64_t key, int dist, float scale) {
    size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    const size_t step = (size_t)gridDim.x * blockDim.x;
    for (; i < n; i += step) {
        if (dist == DIST_UNIFORM) {
            uint64_t r = splitmix64(key + i * 8);
            out[i] = (float)(r >> 40) * 1.1920928955078125e-07f - 1.0f;       // 2^-23; every step is exact in f32
        } else {
            out[i] = (float)irwin_hall(key, i) * scale;
        }
    }
}

__global__ void gen_f64(double* out, size_t n, uint64_t key, int dist, double scale) {
    size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    const size_t step = (size_t)gridDim.x * blockDim.x;
    for (; i < n; i += step) {
        if (dist == DIST_UNIFORM) {
            uint64_t r = splitmix64(key + i * 8);
            out[i] = (double)(r >> 11) * 2.220446049250313e-16 - 1.0;            // 2^-52
        } else {
            out[i] = (double)irwin_hall(key, i) * scale;
        }
    }
}

__global__ void gen_i32(int32_t* out, size_t n, uint64_t key, int64_t lo, uint64_t span) {
    size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    const size_t step = (size_t)gridDim.x * blockDim.x;
    for (; i < n; i += step) {
        uint64_t r = splitmix64(key + i * 8);
        out[i] = (int32_t)(lo + (int64_t)(r % span));
    }
}

}  // namespace

// dist 0: uniform [-1,1) (p0, p1 ignored); dist 1: normal(0, p0); dist 2 (i32 only): integers in [p0, p1].
// `out` is a device pointer; the call returns after the data is written.
extern "C" int32_t rtd_generate(int32_t dtype, int32_t dist, uint64_t seed, uint64_t stream, double p0, double p1, void* out, uint64_t n) {
    if (!out && n) return 1;
    if (n == 0) return 0;
    const uint64_t key = stream_key(seed, stream);
    size_t blocks = (size_t)((n + 255) / 256);
    if (blocks > 65536) blocks = 65536;
    if (dtype == DT_F32 && (dist == DIST_UNIFORM || dist == DIST_NORMAL)) {
        float scale = (float)(p0 * 5.9604644775390625e-08);                      // sigma * 2^-24, rounded to f32 once
        hipLaunchKernelGGL(gen_f32, dim3((unsigned)blocks), dim3(256), 0, 0, (float*)out, (size_t)n, key, dist, scale);
    } else if (dtype == DT_F64 && (dist == DIST_UNIFORM || dist == DIST_NORMAL)) {
        hipLaunchKernelGGL(gen_f64, dim3((unsigned)blocks), dim3(256), 0, 0, (double*)out, (size_t)n, key, dist, p0 * 5.9604644775390625e-08);
    } else if (dtype == DT_I32 && dist == DIST_INT) {
        int64_t lo = (int64_t)p0, hi = (int64_t)p1;
        if (hi < lo) return 1;
        hipLaunchKernelGGL(gen_i32, dim3((unsigned)blocks), dim3(256), 0, 0, (int32_t*)out, (size_t)n, key, lo, (uint64_t)(hi - lo + 1));
    } else {
        return 2;
    }
    if (hipGetLastError() != hipSuccess) return 3;
    if (hipDeviceSynchronize() != hipSuccess) return 3;
    return 0;
}
