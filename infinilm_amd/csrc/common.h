// Shared helpers of the gfx950 kernels: element types, conversions, wave reductions and the error
// channel of the C entry points.  Every entry point returns 0 on success and -1 after storing a
// message that ilm_last_error() returns.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>
#include <stdio.h>

#define ILM_DTYPE_F32 0
#define ILM_DTYPE_BF16 1

#define WAVE 64

struct bf16 {
    uint16_t bits;
};

__device__ __host__ __forceinline__ float bf16_bits_to_f32(uint16_t b) {
    union {
        uint32_t u;
        float f;
    } c;
    c.u = ((uint32_t)b) << 16;
    return c.f;
}

// round to nearest even; NaN stays NaN
__device__ __host__ __forceinline__ uint16_t f32_to_bf16_bits(float f) {
    union {
        uint32_t u;
        float f;
    } c;
    c.f = f;
    uint32_t u = c.u;
    if ((u & 0x7fffffffu) > 0x7f800000u) return (uint16_t)((u >> 16) | 0x40u);
    u += 0x7fffu + ((u >> 16) & 1u);
    return (uint16_t)(u >> 16);
}

__device__ __forceinline__ float to_f32(float v) { return v; }
__device__ __forceinline__ float to_f32(bf16 v) { return bf16_bits_to_f32(v.bits); }

template <typename T>
__device__ __forceinline__ T from_f32(float v);
template <>
__device__ __forceinline__ float from_f32<float>(float v) {
    return v;
}
template <>
__device__ __forceinline__ bf16 from_f32<bf16>(float v) {
    // the hardware's conversion (round to nearest even), one instruction on gfx950
    bf16 r;
    r.bits = __builtin_bit_cast(uint16_t, (__bf16)v);
    return r;
}

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

// Sum over a block of NW waves; every thread gets the result.  `red` holds NW floats of LDS.
template <int NW>
__device__ __forceinline__ float block_sum(float v, float* red) {
    v = wave_sum(v);
    const int lane = threadIdx.x & 63, w = threadIdx.x >> 6;
    __syncthreads();
    if (lane == 0) red[w] = v;
    __syncthreads();
    float t = 0.f;
#pragma unroll
    for (int i = 0; i < NW; ++i) t += red[i];
    return t;
}

extern "C" const char* ilm_last_error();
void ilm_set_error(const char* fmt, ...);
// compute units of the current device (looked up once a process; 256 if the runtime does not say)
int ilm_num_cus();

#define ILM_REQUIRE(cond, ...)          \
    do {                                \
        if (!(cond)) {                  \
            ilm_set_error(__VA_ARGS__); \
            return -1;                  \
        }                               \
    } while (0)

#define ILM_LAUNCH_CHECK(name)                                                   \
    do {                                                                         \
        hipError_t e__ = hipGetLastError();                                      \
        if (e__ != hipSuccess) {                                                 \
            ilm_set_error("%s: launch failed: %s", name, hipGetErrorString(e__)); \
            return -1;                                                           \
        }                                                                        \
    } while (0)
