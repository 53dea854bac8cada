// Shared device helpers for the gfx950 kernels: bfloat16 as raw bits, typed loads and
// stores that always compute in float32, 64-lane wave reductions and block reductions.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#define RL_WAVE 64

// Error codes returned by every extern "C" entry point (0 = launched).
#define RL_OK 0
#define RL_ERR_ARG 1     // an argument the kernel cannot take (the host wrapper says which)
#define RL_ERR_LAUNCH 2  // hipGetLastError() after the launch was not hipSuccess

struct bf16_t {
    uint16_t bits;
};

__device__ __host__ inline float bf16_to_float(bf16_t v) {
    union {
        uint32_t u;
        float f;
    } c;
    c.u = ((uint32_t)v.bits) << 16;
    return c.f;
}

// round to nearest, ties to even; NaN stays NaN
__device__ __host__ inline bf16_t float_to_bf16(float f) {
    union {
        uint32_t u;
        float f;
    } c;
    c.f = f;
    uint32_t u = c.u;
    bf16_t r;
    if ((u & 0x7fffffffu) > 0x7f800000u) {
        r.bits = (uint16_t)((u >> 16) | 0x0040u);
        return r;
    }
    u += 0x7fffu + ((u >> 16) & 1u);
    r.bits = (uint16_t)(u >> 16);
    return r;
}

__device__ inline float to_float(float v) { return v; }
__device__ inline float to_float(bf16_t v) { return bf16_to_float(v); }

template <typename T>
__device__ inline T from_float(float v);
template <>
__device__ inline float from_float<float>(float v) {
    return v;
}
template <>
__device__ inline bf16_t from_float<bf16_t>(float v) {
    return float_to_bf16(v);
}

__device__ inline float wave_sum(float v) {
#pragma unroll
    for (int off = RL_WAVE / 2; off > 0; off >>= 1) v += __shfl_xor(v, off, RL_WAVE);
    return v;
}

__device__ inline float wave_max(float v) {
#pragma unroll
    for (int off = RL_WAVE / 2; off > 0; off >>= 1) v = fmaxf(v, __shfl_xor(v, off, RL_WAVE));
    return v;
}

// Block-wide reductions for blocks of up to 1024 threads (16 waves). `scratch` is a
// __shared__ float[16]; every thread of the block must call these.
__device__ inline float block_sum(float v, float* scratch) {
    const int lane = threadIdx.x & (RL_WAVE - 1);
    const int wave = threadIdx.x / RL_WAVE;
    const int nwaves = (blockDim.x + RL_WAVE - 1) / RL_WAVE;
    v = wave_sum(v);
    __syncthreads();  // scratch may still be read from a previous call
    if (lane == 0) scratch[wave] = v;
    __syncthreads();
    float total = 0.f;
    for (int i = 0; i < nwaves; ++i) total += scratch[i];
    return total;
}

__device__ inline float block_max(float v, float* scratch) {
    const int lane = threadIdx.x & (RL_WAVE - 1);
    const int wave = threadIdx.x / RL_WAVE;
    const int nwaves = (blockDim.x + RL_WAVE - 1) / RL_WAVE;
    v = wave_max(v);
    __syncthreads();
    if (lane == 0) scratch[wave] = v;
    __syncthreads();
    float total = scratch[0];
    for (int i = 1; i < nwaves; ++i) total = fmaxf(total, scratch[i]);
    return total;
}

static inline int rl_launch_status() {
    return hipGetLastError() == hipSuccess ? RL_OK : RL_ERR_LAUNCH;
}

// Element type tags passed from the host: 0 = float32, 1 = bfloat16.
#define RL_F32 0
#define RL_BF16 1
