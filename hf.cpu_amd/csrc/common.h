// Shared device helpers for the gfx950 kernels: element types, conversions, wave
// and block reductions, and the launchers' error reporting.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>
#include <stdio.h>

#define HFA_F32 0
#define HFA_BF16 1

#define WAVE 64

// bfloat16 carried as its bits; conversion is round-to-nearest-even, NaN kept.
struct bf16 { uint16_t bits; };

__device__ __forceinline__ float to_f32(float v) { return v; }
__device__ __forceinline__ float to_f32(bf16 v) { return __uint_as_float(((uint32_t)v.bits) << 16); }

__device__ __forceinline__ uint16_t bf16_bits(float f) {
    uint32_t u = __float_as_uint(f);
    if ((u & 0x7fffffffu) > 0x7f800000u) return (uint16_t)((u >> 16) | 0x40u);
    u += 0x7fffu + ((u >> 16) & 1u);
    return (uint16_t)(u >> 16);
}
template <typename T> __device__ __forceinline__ T from_f32(float v);
template <> __device__ __forceinline__ float from_f32<float>(float v) { return v; }
template <> __device__ __forceinline__ bf16 from_f32<bf16>(float v) { bf16 r; r.bits = bf16_bits(v); return r; }

__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
    for (int off = WAVE / 2; off > 0; off >>= 1) v += __shfl_xor(v, off, WAVE);
    return v;
}
__device__ __forceinline__ float wave_max(float v) {
#pragma unroll
    for (int off = WAVE / 2; off > 0; off >>= 1) v = fmaxf(v, __shfl_xor(v, off, WAVE));
    return v;
}

// Sum over a block of up to 1024 threads in a fixed order; every thread gets the result.
// `red` is LDS for 17 floats; the caller may reuse it after the call.
__device__ __forceinline__ float block_sum(float v, float* red) {
    v = wave_sum(v);
    const int lane = threadIdx.x & (WAVE - 1), w = threadIdx.x / WAVE, nw = (blockDim.x + WAVE - 1) / WAVE;
    __syncthreads();
    if (lane == 0) red[w] = v;
    __syncthreads();
    if (threadIdx.x == 0) {
        float s = 0.f;
        for (int i = 0; i < nw; i++) s += red[i];
        red[16] = s;
    }
    __syncthreads();
    return red[16];
}
__device__ __forceinline__ float block_max(float v, float* red) {
    v = wave_max(v);
    const int lane = threadIdx.x & (WAVE - 1), w = threadIdx.x / WAVE, nw = (blockDim.x + WAVE - 1) / WAVE;
    __syncthreads();
    if (lane == 0) red[w] = v;
    __syncthreads();
    if (threadIdx.x == 0) {
        float s = red[0];
        for (int i = 1; i < nw; i++) s = fmaxf(s, red[i]);
        red[16] = s;
    }
    __syncthreads();
    return red[16];
}

// ---- error reporting of the launchers ---------------------------------------------------
// Every extern "C" launcher returns 0, or a non-zero code after leaving a message that
// hfa_last_error() returns. Bad shapes are refused before anything is launched.
extern "C" const char* hfa_last_error(void);
void hfa_set_error(const char* fmt, ...);

#define HFA_REQUIRE(cond, ...)              \
    do {                                    \
        if (!(cond)) {                      \
            hfa_set_error(__VA_ARGS__);     \
            return 1;                       \
        }                                   \
    } while (0)

#define HFA_LAUNCH_CHECK(name)                                                      \
    do {                                                                            \
        hipError_t e_ = hipGetLastError();                                          \
        if (e_ != hipSuccess) {                                                     \
            hfa_set_error("%s: launch failed: %s", name, hipGetErrorString(e_));    \
            return 2;                                                               \
        }                                                                           \
    } while (0)
