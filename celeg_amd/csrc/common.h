// Shared device helpers for the gfx950 kernels: bfloat16 storage type, conversions,
// wavefront (64 lanes) and block reductions, and the launch-result convention.
//
// Every entry point is extern "C", takes raw device pointers, sizes and a stream, and
// returns 0 or a hipError_t value; the Python side checks shapes before calling.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>
#include <type_traits>

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

// larger float <-> larger key
__device__ __forceinline__ uint32_t order_key(float f) {
    const uint32_t u = __float_as_uint(f);
    return (u & 0x80000000u) ? ~u : (u | 0x80000000u);
}

// A logit and its index as one number, for the largest logit of a row and, among equal ones,
// the lowest index: the maximum of these over a row is its greedy token.  0 stands for "none".
__device__ __forceinline__ unsigned long long packed_logit(float x, int index) {
    x += 0.0f;                                                       // -0 and +0 are one value
    return (static_cast<unsigned long long>(order_key(x)) << 32) | (0xffffffffu - static_cast<unsigned>(index));
}
__device__ __forceinline__ int packed_logit_index(unsigned long long packed) {
    return static_cast<int>(0xffffffffu - static_cast<unsigned>(packed & 0xffffffffull));
}

// The largest of v over every group of W neighbouring lanes (W = 4, 8, 16, 32 or 64; groups start
// at multiples of W), in all its lanes.  Up to 16 lanes by cross-lane modifiers of the vector
// unit (lanes swapped in pairs and in pairs of pairs, then the halves of 8 and of 16 mirrored);
// each step beyond, one exchange through the LDS crossbar.
template <int W>
__device__ __forceinline__ uint32_t group_max_u32(uint32_t v) {
    static_assert(W == 4 || W == 8 || W == 16 || W == 32 || W == 64, "groups of 4 to 64 lanes");
    auto across = [](uint32_t x, auto ctrl) {
        return static_cast<uint32_t>(__builtin_amdgcn_update_dpp(0, static_cast<int>(x), decltype(ctrl)::value, 0xf, 0xf, false));
    };
    v = max(v, across(v, std::integral_constant<int, 0xB1>{}));              // lanes 1 0 3 2 of every four
    v = max(v, across(v, std::integral_constant<int, 0x4E>{}));              // lanes 2 3 0 1
    if (W >= 8) v = max(v, across(v, std::integral_constant<int, 0x141>{}));   // every half of 8 mirrored
    if (W >= 16) v = max(v, across(v, std::integral_constant<int, 0x140>{}));  // every row of 16 mirrored
    if (W >= 32) v = max(v, static_cast<uint32_t>(__shfl_xor(static_cast<int>(v), 16, 64)));
    if (W >= 64) v = max(v, static_cast<uint32_t>(__shfl_xor(static_cast<int>(v), 32, 64)));
    return v;
}

// The best (logit, index) of a group of W neighbouring lanes, lane j of the group holding the logit
// x of column first + j (have: it holds one): packed as packed_logit packs it, the lowest column
// among equal logits; 0 if no lane holds one.  The same value in every lane of the group.
template <int W>
__device__ __forceinline__ unsigned long long group_best_logit(float x, bool have, int first) {
    x += 0.0f;
    const uint32_t key = have ? order_key(x) : 0u;
    const uint32_t top = group_max_u32<W>(key);
    const unsigned long long holders = __ballot(have && key == top);
    const int lane = static_cast<int>(threadIdx.x) & 63, base = lane & ~(W - 1);
    const unsigned long long mine = W == 64 ? holders : (holders >> base) & ((1ull << (W & 63)) - 1ull);
    if (mine == 0ull) return 0ull;
    const int j = __ffsll(static_cast<long long>(mine)) - 1;
    return (static_cast<unsigned long long>(top) << 32) | (0xffffffffu - static_cast<unsigned>(first + j));
}

#define CELEG_LAUNCH_RESULT() static_cast<int>(hipGetLastError())

enum CelegDtype { CELEG_F32 = 0, CELEG_BF16 = 1 };
