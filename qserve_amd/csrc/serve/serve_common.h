// serve_common.h -- helpers shared by the kernels of libqserve_serve.so (gfx950, 64-wide wavefronts)
#pragma once
#include <hip/hip_runtime.h>
#include <stdarg.h>
#include <stdint.h>
#include <stdio.h>

#include "../../../include/qserve_serve.h"

void qsv_set_error(const char* fmt, ...);

#define QSV_REQUIRE(cond, ...)          \
    do {                                \
        if (!(cond)) {                  \
            qsv_set_error(__VA_ARGS__); \
            return QSV_EINVAL;          \
        }                               \
    } while (0)

static inline int qsv_launch_status(const char* what) {
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) {
        qsv_set_error("%s: launch failed: %s", what, hipGetErrorString(e));
        return (int)e;
    }
    return QSV_OK;
}

typedef uint16_t bf16_t;   // storage only: arithmetic is float

__device__ __forceinline__ float bf2f(bf16_t v) { return __uint_as_float((uint32_t)v << 16); }
__device__ __forceinline__ bf16_t f2bf(float f) {   // round to nearest even; NaN stays NaN
    uint32_t u = __float_as_uint(f);
    if ((u & 0x7fffffffu) > 0x7f800000u) return (bf16_t)0x7fc0;
    u += 0x7fffu + ((u >> 16) & 1u);
    return (bf16_t)(u >> 16);
}
__device__ __forceinline__ float ld(const float* p, size_t i) { return p[i]; }
__device__ __forceinline__ float ld(const bf16_t* p, size_t i) { return bf2f(p[i]); }
__device__ __forceinline__ void st(float* p, size_t i, float v) { p[i] = v; }
__device__ __forceinline__ void st(bf16_t* p, size_t i, float v) { p[i] = f2bf(v); }

__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) v += __shfl_xor(v, o, 64);
    return v;
}
__device__ __forceinline__ float wave_max(float v) {
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) v = fmaxf(v, __shfl_xor(v, o, 64));
    return v;
}
// Sum over a workgroup of NT threads (a multiple of 64); every thread gets the result.  `red` holds NT / 64 + 1 floats.
template <int NT>
__device__ __forceinline__ float block_sum(float v, float* red) {
    v = wave_sum(v);
    __syncthreads();   // (red may still be read from a previous call)
    if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = v;
    __syncthreads();
    float s = 0.f;
#pragma unroll
    for (int i = 0; i < NT / 64; ++i) s += red[i];
    return s;
}

// dtype dispatch of a templated launcher: F<bf16_t>() or F<float>()
#define QSV_DISPATCH(dtype, what, CALL)                                  \
    do {                                                                 \
        if ((dtype) == QSV_BF16) {                                       \
            typedef bf16_t T;                                            \
            CALL;                                                        \
        } else if ((dtype) == QSV_F32) {                                 \
            typedef float T;                                             \
            CALL;                                                        \
        } else {                                                         \
            qsv_set_error("%s: unknown dtype code %d", what, (dtype));   \
            return QSV_EINVAL;                                           \
        }                                                                \
    } while (0)
