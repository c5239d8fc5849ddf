// Double-gated short causal convolution over the rows of a step, continuing each
// request from its saved state, and the state update that follows.
//
// bcx[t] = [B | C | x] (each `width` wide); bx = B*x;
// conv[t,ch] = sum_tap w[ch,tap] * bx[pos(t) - (taps-1-tap), ch] (+ bias), zero before
// position 0; y = C * conv.   Reference: src/backend/cpu/kernels/convolution.cpp:7-60;
// ragged CUDA form src/backend/cuda/kernels/shortconv.cuh:34-64.
//
// State per request [taps, width] in 32-bit: entry j holds bx at position
// (tokens seen) - taps + j.  The forward kernel reads only the OLD state and the rows
// of the step; the update kernel runs after it on the same stream.  bx is kept as the
// unrounded 32-bit product both in the state and when read from rows, so cutting a
// sequence into steps changes nothing.
#include "common.h"

template <typename T>
__global__ void short_conv_fwd_kernel(
    const T* __restrict__ bcx, int ld_bcx, const float* __restrict__ w,
    const float* __restrict__ bias, const float* __restrict__ state, size_t state_slot_stride,
    T* __restrict__ out, const int* __restrict__ positions, const int* __restrict__ token_seq,
    const int* __restrict__ seq_start, const int* __restrict__ seq_slot,
    const int* __restrict__ cu_seqlens, int width, int taps) {
    const int ch = blockIdx.y * blockDim.x + threadIdx.x;
    if (ch >= width) return;
    const int t = blockIdx.x;
    const int s = token_seq[t];
    const int start = seq_start[s];
    const int row0 = cu_seqlens[s];
    const int pos = positions[t];
    const float* st = state + static_cast<size_t>(seq_slot[s]) * state_slot_stride;
    float conv = 0.f;
    for (int tap = 0; tap < taps; ++tap) {
        const int q = pos - (taps - 1 - tap);
        if (q < 0) continue;
        float bx;
        if (q >= start) {
            const T* row = bcx + static_cast<size_t>(row0 + (q - start)) * ld_bcx;
            bx = to_float(row[ch]) * to_float(row[2 * width + ch]);
        } else {
            bx = st[static_cast<size_t>(q - start + taps) * width + ch];
        }
        conv = fmaf(w[static_cast<size_t>(ch) * taps + tap], bx, conv);
    }
    if (bias) conv += bias[ch];
    const float c = to_float(bcx[static_cast<size_t>(t) * ld_bcx + width + ch]);
    out[static_cast<size_t>(t) * width + ch] = from_float<T>(c * conv);
}

template <typename T>
__global__ void short_conv_state_kernel(
    const T* __restrict__ bcx, int ld_bcx, float* __restrict__ state, size_t state_slot_stride,
    const int* __restrict__ seq_start, const int* __restrict__ seq_slot,
    const int* __restrict__ cu_seqlens, int width, int taps) {
    const int ch = blockIdx.y * blockDim.x + threadIdx.x;
    if (ch >= width) return;
    const int s = blockIdx.x;
    const int start = seq_start[s];
    const int row0 = cu_seqlens[s];
    const int n = cu_seqlens[s + 1] - row0;
    const int end = start + n;
    float* st = state + static_cast<size_t>(seq_slot[s]) * state_slot_stride;
    // ascending j: an old entry is read at index j + n > j, before it is overwritten
    for (int j = 0; j < taps; ++j) {
        const int q = end - taps + j;
        float v = 0.f;
        if (q >= start) {
            const T* row = bcx + static_cast<size_t>(row0 + (q - start)) * ld_bcx;
            v = to_float(row[ch]) * to_float(row[2 * width + ch]);
        } else if (q >= 0) {
            v = st[static_cast<size_t>(q - start + taps) * width + ch];
        }
        st[static_cast<size_t>(j) * width + ch] = v;
    }
}

extern "C" int celeg_short_conv(const void* bcx, int ld_bcx, int dtype, const float* w,
                                const float* bias, float* state, size_t state_slot_stride,
                                void* out, const int* positions, const int* token_seq,
                                const int* seq_start, const int* seq_slot, const int* cu_seqlens,
                                int n_tokens, int n_seqs, int width, int taps,
                                hipStream_t stream) {
    if (n_tokens <= 0 || n_seqs <= 0) return 0;
    dim3 block(256);
    dim3 grid_fwd(n_tokens, (width + 255) / 256), grid_state(n_seqs, (width + 255) / 256);
    if (dtype == CELEG_F32) {
        hipLaunchKernelGGL(short_conv_fwd_kernel<float>, grid_fwd, block, 0, stream,
                           static_cast<const float*>(bcx), ld_bcx, w, bias, state,
                           state_slot_stride, static_cast<float*>(out), positions, token_seq,
                           seq_start, seq_slot, cu_seqlens, width, taps);
        hipLaunchKernelGGL(short_conv_state_kernel<float>, grid_state, block, 0, stream,
                           static_cast<const float*>(bcx), ld_bcx, state, state_slot_stride,
                           seq_start, seq_slot, cu_seqlens, width, taps);
    } else {
        hipLaunchKernelGGL(short_conv_fwd_kernel<bf16>, grid_fwd, block, 0, stream,
                           static_cast<const bf16*>(bcx), ld_bcx, w, bias, state,
                           state_slot_stride, static_cast<bf16*>(out), positions, token_seq,
                           seq_start, seq_slot, cu_seqlens, width, taps);
        hipLaunchKernelGGL(short_conv_state_kernel<bf16>, grid_state, block, 0, stream,
                           static_cast<const bf16*>(bcx), ld_bcx, state, state_slot_stride,
                           seq_start, seq_slot, cu_seqlens, width, taps);
    }
    return CELEG_LAUNCH_RESULT();
}
