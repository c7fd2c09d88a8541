// Shared device helpers for the gfx950 kernels: storage types, wave/block reductions, checks.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#define TM_WAVE 64

// dtype codes of the C interface
#define TM_F32 0
#define TM_BF16 1
#define TM_NONE (-1)

// error codes of the C interface (0 = ok)
#define TM_OK 0
#define TM_ERR_ARG 1        // an argument the kernel cannot run with
#define TM_ERR_LAUNCH 2     // the runtime refused the launch
#define TM_ERR_UNSUPPORTED 3 // a library has no routine for the request: use another path

typedef uint16_t bf16_t;    // bfloat16 bits

__device__ __forceinline__ float bf16_to_f32(bf16_t v) {
    return __uint_as_float(((uint32_t)v) << 16);
}

// round to nearest even; NaN stays NaN
__device__ __forceinline__ bf16_t f32_to_bf16(float f) {
    uint32_t u = __float_as_uint(f);
    if ((u & 0x7fffffffu) > 0x7f800000u) return (bf16_t)((u >> 16) | 0x0040u);
    u += 0x7fffu + ((u >> 16) & 1u);
    return (bf16_t)(u >> 16);
}

template <typename T> struct Elem;
template <> struct Elem<float> {
    static __device__ __forceinline__ float load(const float* p) { return *p; }
    static __device__ __forceinline__ void store(float* p, float v) { *p = v; }
    static __device__ __forceinline__ float round(float v) { return v; }
};
template <> struct Elem<bf16_t> {
    static __device__ __forceinline__ float load(const bf16_t* p) { return bf16_to_f32(*p); }
    static __device__ __forceinline__ void store(bf16_t* p, float v) { *p = f32_to_bf16(v); }
    static __device__ __forceinline__ float round(float v) { return bf16_to_f32(f32_to_bf16(v)); }
};

// The rotation of a pair (x1, x2) by the angle whose cosine and sine are c and s (reference
// src/infer/model/layers.py:60-64). Every product and each sum is rounded to 32-bit on its own, as a tensor
// library's x1 * cos - x2 * sin is: left to itself the compiler fuses a product into the sum, and which one it
// picks differs from one kernel (or one instantiation of a kernel) to the next, so that the same token would get
// other last bits from the kernel for 8 rows than from the kernel for 40.
__device__ __forceinline__ void rotate_pair(float x1, float x2, float c, float s, float& y1, float& y2) {
#pragma clang fp contract(off)
    const float a = x1 * c, b = x2 * s, d = x2 * c, e = x1 * s;
    y1 = a - b;
    y2 = d + e;
}

__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
    for (int off = TM_WAVE / 2; off > 0; off >>= 1) v += __shfl_xor(v, off, TM_WAVE);
    return v;
}

__device__ __forceinline__ float wave_max(float v) {
#pragma unroll
    for (int off = TM_WAVE / 2; off > 0; off >>= 1) v = fmaxf(v, __shfl_xor(v, off, TM_WAVE));
    return v;
}

// Sum over a block of NT threads (NT a multiple of 64, at most 1024). Every thread gets the result.
// The order of the additions is fixed by the thread layout, never by the data.
template <int NT>
__device__ __forceinline__ float block_sum(float v, float* smem /* NT/64 floats */) {
    v = wave_sum(v);
    const int wave = threadIdx.x / TM_WAVE, lane = threadIdx.x % TM_WAVE;
    __syncthreads();
    if (lane == 0) smem[wave] = v;
    __syncthreads();
    float total = 0.f;
#pragma unroll
    for (int w = 0; w < NT / TM_WAVE; ++w) total += smem[w];
    return total;
}

#define TM_CHECK_LAUNCH()                                        \
    do {                                                         \
        hipError_t e_ = hipGetLastError();                       \
        if (e_ != hipSuccess) return TM_ERR_LAUNCH;              \
    } while (0)
