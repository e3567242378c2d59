// Shared helpers of the gfx950 kernels: error reporting, element access, launch checks.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>
#include <stdio.h>
#include <stdarg.h>

#include "../../include/hapmi.h"

typedef __bf16 bf16_t;
typedef bf16_t bf16x8 __attribute__((ext_vector_type(8)));
typedef bf16_t bf16x4 __attribute__((ext_vector_type(4)));
typedef bf16_t bf16x2 __attribute__((ext_vector_type(2)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef float f32x2 __attribute__((ext_vector_type(2)));

#define HAPMI_WAVE 64

int hapmi_set_error(int code, const char *fmt, ...);
int hapmi_sumsq_static_setup();   // elementwise.hip: per-device set-up that hapmi_init runs

#define HAPMI_REQUIRE(cond, code, ...)                           \
    do {                                                         \
        if (!(cond)) return hapmi_set_error((code), __VA_ARGS__); \
    } while (0)

#define HAPMI_CHECK_LAUNCH(name)                                                        \
    do {                                                                                \
        hipError_t e__ = hipGetLastError();                                             \
        if (e__ != hipSuccess)                                                          \
            return hapmi_set_error(HAPMI_ELAUNCH, "%s: %s", (name), hipGetErrorString(e__)); \
    } while (0)

static inline int hapmi_dtype_ok(int dtype) { return dtype == HAPMI_F32 || dtype == HAPMI_BF16; }
static inline int64_t hapmi_elem_size(int dtype) { return dtype == HAPMI_F32 ? 4 : 2; }
static inline int64_t hapmi_cdiv(int64_t a, int64_t b) { return (a + b - 1) / b; }

// element load/store as float for either storage type
template <typename T> __device__ __forceinline__ float ld_f(const T *p, int64_t i);
template <> __device__ __forceinline__ float ld_f<float>(const float *p, int64_t i) { return p[i]; }
template <> __device__ __forceinline__ float ld_f<bf16_t>(const bf16_t *p, int64_t i) { return (float)p[i]; }
template <typename T> __device__ __forceinline__ void st_f(T *p, int64_t i, float v);
template <> __device__ __forceinline__ void st_f<float>(float *p, int64_t i, float v) { p[i] = v; }
template <> __device__ __forceinline__ void st_f<bf16_t>(bf16_t *p, int64_t i, float v) { p[i] = (bf16_t)v; }

// 16-byte vector of elements: 4 floats or 8 bf16
template <typename T> struct Vec16;
template <> struct Vec16<float> {
    static constexpr int N = 4;
    f32x4 v;
    __device__ __forceinline__ float get(int i) const { return v[i]; }
    __device__ __forceinline__ void set(int i, float x) { v[i] = x; }
};
template <> struct Vec16<bf16_t> {
    static constexpr int N = 8;
    bf16x8 v;
    __device__ __forceinline__ float get(int i) const { return (float)v[i]; }
    __device__ __forceinline__ void set(int i, float x) { v[i] = (bf16_t)x; }
};

__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) v += __shfl_xor(v, off, 64);
    return v;
}
__device__ __forceinline__ float wave_max(float v) {
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) v = fmaxf(v, __shfl_xor(v, off, 64));
    return v;
}

// block-wide reductions for blocks of up to 1024 threads (16 waves); `red` is 16 floats of LDS
__device__ __forceinline__ float block_sum(float v, float *red) {
    v = wave_sum(v);
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63, nw = (blockDim.x + 63) >> 6;
    __syncthreads();
    if (lane == 0) red[wave] = v;
    __syncthreads();
    float t = 0.f;
    for (int i = 0; i < nw; ++i) t += red[i];
    return t;
}
__device__ __forceinline__ float block_max(float v, float *red) {
    v = wave_max(v);
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63, nw = (blockDim.x + 63) >> 6;
    __syncthreads();
    if (lane == 0) red[wave] = v;
    __syncthreads();
    float t = red[0];
    for (int i = 1; i < nw; ++i) t = fmaxf(t, red[i]);
    return t;
}
