// Shared device helpers for the gfx950 kernels: bfloat16 storage type, conversions,
// wavefront (64 lanes) and block reductions, and the launch-result convention.
//
// Every entry point is extern "C", takes raw device pointers, sizes and a stream, and
// returns 0 or a hipError_t value; the Python side checks shapes before calling.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

#define CELEG_WAVE 64

struct bf16 {
    uint16_t bits;
};

__device__ __forceinline__ float to_float(float x) { return x; }
__device__ __forceinline__ float to_float(bf16 x) {
    return __uint_as_float(static_cast<uint32_t>(x.bits) << 16);
}

template <typename T>
__device__ __forceinline__ T from_float(float x);

template <>
__device__ __forceinline__ float from_float<float>(float x) { return x; }

// round to nearest even (gfx950 converts in hardware: v_cvt_pk_bf16_f32)
template <>
__device__ __forceinline__ bf16 from_float<bf16>(float x) {
    bf16 r;
    r.bits = __builtin_bit_cast(uint16_t, static_cast<__bf16>(x));
    return r;
}

__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
    for (int off = CELEG_WAVE / 2; off > 0; off >>= 1) v += __shfl_xor(v, off, CELEG_WAVE);
    return v;
}

__device__ __forceinline__ float wave_max(float v) {
#pragma unroll
    for (int off = CELEG_WAVE / 2; off > 0; off >>= 1) v = fmaxf(v, __shfl_xor(v, off, CELEG_WAVE));
    return v;
}

// Sum over a block of up to 1024 threads (a multiple of 64).  `scratch` holds 16 floats.
// Every thread receives the total.  The order of additions is fixed by the thread
// layout, so a row's result does not depend on what else is in the batch.
__device__ __forceinline__ float block_sum(float v, float* scratch) {
    const int lane = threadIdx.x & (CELEG_WAVE - 1);
    const int wave = threadIdx.x / CELEG_WAVE;
    const int n_waves = (blockDim.x + CELEG_WAVE - 1) / CELEG_WAVE;
    v = wave_sum(v);
    __syncthreads();
    if (lane == 0) scratch[wave] = v;
    __syncthreads();
    float total = 0.f;
    for (int w = 0; w < n_waves; ++w) total += scratch[w];
    return total;
}

#define CELEG_LAUNCH_RESULT() static_cast<int>(hipGetLastError())

enum CelegDtype { CELEG_F32 = 0, CELEG_BF16 = 1 };
