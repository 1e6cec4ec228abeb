// Shared device helpers for the gfx950 kernels: element types, wave and block reductions.
//
// A wavefront has 64 lanes.  Activations and weights are float (the 32-bit path) or
// bfloat16 carried as raw 16-bit words (the serving path); all arithmetic is float.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#define SIA_WAVE 64

typedef uint16_t bf16_t;  // raw bfloat16 bits

enum SiaDtype { SIA_F32 = 0, SIA_BF16 = 1 };

__device__ __forceinline__ float bf16_to_float(bf16_t b) {
    return __uint_as_float(((uint32_t)b) << 16);
}

// Round to nearest, ties to even; NaN stays NaN.
__device__ __forceinline__ bf16_t float_to_bf16(float f) {
    uint32_t u = __float_as_uint(f);
    if ((u & 0x7fffffffu) > 0x7f800000u) return (bf16_t)((u >> 16) | 0x0040u);
    u += 0x7fffu + ((u >> 16) & 1u);
    return (bf16_t)(u >> 16);
}

__device__ __forceinline__ float to_float(float x) { return x; }
__device__ __forceinline__ float to_float(bf16_t x) { return bf16_to_float(x); }

template <typename T> __device__ __forceinline__ T from_float(float x);
template <> __device__ __forceinline__ float from_float<float>(float x) { return x; }
template <> __device__ __forceinline__ bf16_t from_float<bf16_t>(float x) { return float_to_bf16(x); }

// Eight consecutive elements of a row as one register value: 32 bytes of float or 16 of bfloat16.
template <typename T> struct Vec8;
template <> struct Vec8<float> {
    float4 a, b;
    __device__ __forceinline__ void load(const float* p) { a = *(const float4*)p; b = *(const float4*)(p + 4); }
    __device__ __forceinline__ void store(float* p) const { *(float4*)p = a; *(float4*)(p + 4) = b; }
    __device__ __forceinline__ void get(float (&x)[8]) const {
        x[0] = a.x; x[1] = a.y; x[2] = a.z; x[3] = a.w; x[4] = b.x; x[5] = b.y; x[6] = b.z; x[7] = b.w;
    }
    __device__ __forceinline__ void set(const float (&x)[8]) {
        a = make_float4(x[0], x[1], x[2], x[3]); b = make_float4(x[4], x[5], x[6], x[7]);
    }
};
template <> struct Vec8<bf16_t> {
    uint4 u;
    __device__ __forceinline__ void load(const bf16_t* p) { u = *(const uint4*)p; }
    __device__ __forceinline__ void store(bf16_t* p) const { *(uint4*)p = u; }
    __device__ __forceinline__ void get(float (&x)[8]) const {
        const uint32_t w[4] = {u.x, u.y, u.z, u.w};
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            x[2 * i] = __uint_as_float(w[i] << 16);
            x[2 * i + 1] = __uint_as_float(w[i] & 0xffff0000u);
        }
    }
    __device__ __forceinline__ void set(const float (&x)[8]) {
        uint32_t w[4];
#pragma unroll
        for (int i = 0; i < 4; ++i) w[i] = (uint32_t)float_to_bf16(x[2 * i]) | ((uint32_t)float_to_bf16(x[2 * i + 1]) << 16);
        u = make_uint4(w[0], w[1], w[2], w[3]);
    }
};

// Butterfly reductions over the 64 lanes of a wave: every lane gets the result, and the
// order of additions is fixed, so a row's result does not depend on what else is in a batch.
__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
    for (int off = SIA_WAVE / 2; off > 0; off >>= 1) v += __shfl_xor(v, off, SIA_WAVE);
    return v;
}

__device__ __forceinline__ float wave_max(float v) {
#pragma unroll
    for (int off = SIA_WAVE / 2; off > 0; off >>= 1) v = fmaxf(v, __shfl_xor(v, off, SIA_WAVE));
    return v;
}

// Sum over a block of up to 1024 threads (16 waves); ``scratch`` holds 16 floats of LDS.
// All threads get the result.  Ends with a barrier, so scratch may be reused after it.
__device__ __forceinline__ float block_sum(float v, float* scratch) {
    v = wave_sum(v);
    const int wave = threadIdx.x / SIA_WAVE, lane = threadIdx.x % SIA_WAVE;
    const int n_waves = (blockDim.x + SIA_WAVE - 1) / SIA_WAVE;
    if (lane == 0) scratch[wave] = v;
    __syncthreads();
    float total = 0.f;
    for (int w = 0; w < n_waves; ++w) total += scratch[w];
    __syncthreads();
    return total;
}

__device__ __forceinline__ float block_max(float v, float* scratch) {
    v = wave_max(v);
    const int wave = threadIdx.x / SIA_WAVE, lane = threadIdx.x % SIA_WAVE;
    const int n_waves = (blockDim.x + SIA_WAVE - 1) / SIA_WAVE;
    if (lane == 0) scratch[wave] = v;
    __syncthreads();
    float total = scratch[0];
    for (int w = 1; w < n_waves; ++w) total = fmaxf(total, scratch[w]);
    __syncthreads();
    return total;
}

// Every entry point returns 0 or a HIP error code; launches are asynchronous on ``stream``.
#define SIA_LAUNCH_CHECK() ((int)hipGetLastError())
#define SIA_EXPORT extern "C" __attribute__((visibility("default")))

// Entry points refuse argument combinations they are not written for with this code
// (outside the range of hipError_t values in use).
#define SIA_BAD_ARGUMENT 10001
