// Double-gated short causal convolution over the rows of a step, continuing each
// request from its saved state, and the state update that follows.
//
// bcx[t] = [B | C | x] (each `width` wide); bx = B*x;
// conv[t,ch] = sum_tap w[ch,tap] * bx[pos(t) - (taps-1-tap), ch] (+ bias), zero before
// position 0; y = C * conv.   Reference: src/backend/cpu/kernels/convolution.cpp:7-60;
// ragged CUDA form src/backend/cuda/kernels/shortconv.cuh:34-64.
//
// State per request [taps, width] in 32-bit: entry j holds bx at position
// (tokens seen) - taps + j.  The forward kernels read only the OLD state and the rows
// of the step; the update kernel runs after them on the same stream, except behind the
// kernel for long steps, which updates the state itself (the thread that read a request's
// old state writes its new one).  bx is kept as the unrounded 32-bit product both in the
// state and when read from rows, so cutting a sequence into steps changes nothing.
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

// The same for groups of channels (16 bytes of a row per load): a thread takes VEC
// neighbouring channels of one token.  Tokens whose taps all lie in rows of this step (all
// but the first taps-1 of a portion) ask for every row at once; the others go the slower way
// through the state.
template <typename T> struct ConvVec;
template <> struct ConvVec<float> {
    static constexpr int n = 4;
    typedef float raw __attribute__((ext_vector_type(4)));
    static __device__ __forceinline__ float at(const raw& r, int i) { return r[i]; }
    static __device__ __forceinline__ void set(raw& r, int i, float v) { r[i] = v; }
};
template <> struct ConvVec<bf16> {
    static constexpr int n = 8;
    typedef __bf16 raw __attribute__((ext_vector_type(8)));
    static __device__ __forceinline__ float at(const raw& r, int i) { return static_cast<float>(r[i]); }
    static __device__ __forceinline__ void set(raw& r, int i, float v) { r[i] = static_cast<__bf16>(v); }
};
#define CONV_VEC_MAX_TAPS 8

template <typename T>
__device__ __forceinline__ void short_conv_token_vec(
    int t, int ch, const T* __restrict__ bcx, int ld_bcx, const float* __restrict__ w,
    const float* __restrict__ bias, const float* state, size_t state_slot_stride,
    T* __restrict__ out, const int* __restrict__ positions, const int* __restrict__ token_seq,
    const int* __restrict__ seq_start, const int* __restrict__ seq_slot,
    const int* __restrict__ cu_seqlens, int width, int taps) {
    constexpr int VEC = ConvVec<T>::n;
    typedef typename ConvVec<T>::raw raw;
    const int s = token_seq[t];
    const int start = seq_start[s];
    const int row0 = cu_seqlens[s];
    const int pos = positions[t];
    float conv[VEC];
#pragma unroll
    for (int i = 0; i < VEC; ++i) conv[i] = bias ? bias[ch + i] : 0.f;
    const raw cv = *reinterpret_cast<const raw*>(bcx + static_cast<size_t>(t) * ld_bcx + width + ch);
    if (pos - (taps - 1) >= start) {        // the same for the whole workgroup
        raw bv[CONV_VEC_MAX_TAPS], xv[CONV_VEC_MAX_TAPS];
#pragma unroll
        for (int tap = 0; tap < CONV_VEC_MAX_TAPS; ++tap) {
            // rows t - (taps-1-tap); taps beyond the kernel's length repeat the token's own row
            const int back = max(taps - 1 - tap, 0);
            const T* row = bcx + static_cast<size_t>(t - back) * ld_bcx;
            bv[tap] = *reinterpret_cast<const raw*>(row + ch);
            xv[tap] = *reinterpret_cast<const raw*>(row + 2 * width + ch);
        }
#pragma unroll
        for (int tap = 0; tap < CONV_VEC_MAX_TAPS; ++tap)
            if (tap < taps) {
#pragma unroll
                for (int i = 0; i < VEC; ++i)
                    conv[i] = fmaf(w[static_cast<size_t>(ch + i) * taps + tap],
                                   ConvVec<T>::at(bv[tap], i) * ConvVec<T>::at(xv[tap], i), conv[i]);
            }
    } else {
        const float* st = state + static_cast<size_t>(seq_slot[s]) * state_slot_stride;
        for (int tap = 0; tap < taps; ++tap) {
            const int q = pos - (taps - 1 - tap);
            if (q < 0) continue;
#pragma unroll
            for (int i = 0; i < VEC; ++i) {
                float bx;
                if (q >= start) {
                    const T* row = bcx + static_cast<size_t>(row0 + (q - start)) * ld_bcx;
                    bx = to_float(row[ch + i]) * to_float(row[2 * width + ch + i]);
                } else {
                    bx = st[static_cast<size_t>(q - start + taps) * width + ch + i];
                }
                conv[i] = fmaf(w[static_cast<size_t>(ch + i) * taps + tap], bx, conv[i]);
            }
        }
    }
    raw o;
#pragma unroll
    for (int i = 0; i < VEC; ++i) ConvVec<T>::set(o, i, ConvVec<T>::at(cv, i) * conv[i]);
    *reinterpret_cast<raw*>(out + static_cast<size_t>(t) * width + ch) = o;
}

template <typename T>
__global__ void short_conv_fwd_vec_kernel(
    const T* __restrict__ bcx, int ld_bcx, const float* __restrict__ w,
    const float* __restrict__ bias, const float* __restrict__ state, size_t state_slot_stride,
    T* __restrict__ out, const int* __restrict__ positions, const int* __restrict__ token_seq,
    const int* __restrict__ seq_start, const int* __restrict__ seq_slot,
    const int* __restrict__ cu_seqlens, int width, int taps) {
    const int ch = (blockIdx.y * blockDim.x + threadIdx.x) * ConvVec<T>::n;
    if (ch >= width) return;
    short_conv_token_vec<T>(blockIdx.x, ch, bcx, ld_bcx, w, bias, state, state_slot_stride, out, positions,
                            token_seq, seq_start, seq_slot, cu_seqlens, width, taps);
}

// The state update for VEC neighbouring channels of one request, by the thread that has just
// read the old state for the request's first tokens: entry j becomes bx at position
// end - taps + j, from the step's rows where they reach that far back, else from the old state.
template <typename T>
__device__ __forceinline__ void short_conv_state_vec(
    int s, int ch, const T* __restrict__ bcx, int ld_bcx, float* state, size_t state_slot_stride,
    const int* __restrict__ seq_start, const int* __restrict__ seq_slot,
    const int* __restrict__ cu_seqlens, int width, int taps) {
    constexpr int VEC = ConvVec<T>::n;
    typedef typename ConvVec<T>::raw raw;
    const int start = seq_start[s];
    const int row0 = cu_seqlens[s];
    const int n = cu_seqlens[s + 1] - row0;
    const int end = start + n;
    float* st = state + static_cast<size_t>(seq_slot[s]) * state_slot_stride + ch;
    float v[CONV_VEC_MAX_TAPS][VEC];
#pragma unroll
    for (int j = 0; j < CONV_VEC_MAX_TAPS; ++j) {
        if (j >= taps) break;
        const int q = end - taps + j;
        if (q >= start) {
            const T* row = bcx + static_cast<size_t>(row0 + (q - start)) * ld_bcx;
            const raw bv = *reinterpret_cast<const raw*>(row + ch);
            const raw xv = *reinterpret_cast<const raw*>(row + 2 * width + ch);
#pragma unroll
            for (int i = 0; i < VEC; ++i) v[j][i] = ConvVec<T>::at(bv, i) * ConvVec<T>::at(xv, i);
        } else {
#pragma unroll
            for (int i = 0; i < VEC; ++i) v[j][i] = q >= 0 ? st[static_cast<size_t>(q - start + taps) * width + i] : 0.f;
        }
    }
    // every old entry has been read: now the new ones
#pragma unroll
    for (int j = 0; j < CONV_VEC_MAX_TAPS; ++j) {
        if (j >= taps) break;
#pragma unroll
        for (int i = 0; i < VEC; ++i) st[static_cast<size_t>(j) * width + i] = v[j][i];
    }
}

// The same for TT tokens in a row per thread: where they all belong to one request and every
// tap lies in rows of this step, a row's B and x are read once for all the tokens that use it
// (a window that slides down the rows) instead of once per tap.  The sums are formed in the
// same order as above, so the results are the same bits.  The rows are asked for before it is
// known whether the block is of that kind (their addresses do not depend on it).
// This kernel also updates the state, with no kernel behind it: the first taps-1 tokens of a
// request's rows, the only ones that read the old state, are all computed by the block that
// holds the request's first row (also those that lie in the next block, which skips them), and
// the same thread then writes the new state for its channels.
#define CONV_BLOCK_TOKENS 2     // (2,048 tokens of 1,024 channels, with the state update: 8.8 us with 2, 9.4 with 1 and 10.1 with 4 a thread; more were slower)
template <typename T, int TAPS, int TT>
__global__ __launch_bounds__(256) void short_conv_fwd_block_kernel(
    const T* __restrict__ bcx, int ld_bcx, const float* __restrict__ w,
    const float* __restrict__ bias, float* state, size_t state_slot_stride,
    T* __restrict__ out, const int* __restrict__ positions, const int* __restrict__ token_seq,
    const int* __restrict__ seq_start, const int* __restrict__ seq_slot,
    const int* __restrict__ cu_seqlens, int width, int n_tokens) {
    constexpr int VEC = ConvVec<T>::n;
    typedef typename ConvVec<T>::raw raw;
    const int ch = (blockIdx.y * blockDim.x + threadIdx.x) * VEC;
    if (ch >= width) return;
    // Workgroups go to the chip's 8 dies in turn, and each die has an L2 of its own: die d takes a
    // run of tokens, so that the rows two neighbouring workgroups both read (the taps before a
    // workgroup's first token) come from memory once, not once for each of two dies.  (The grid is
    // 8 runs of gridDim.x / 8 workgroups; those beyond the last token have nothing to do.)
    const int per_die = gridDim.x >> 3;
    const int t0 = ((blockIdx.x & 7) * per_die + (blockIdx.x >> 3)) * TT;
    if (t0 >= n_tokens) return;
    const int n = min(TT, n_tokens - t0);
    // (asked for ahead of the rows; what depends on it is asked for while the rows are on their way)
    const int s = token_seq[t0], s_end = token_seq[min(t0 + TT - 1, n_tokens - 1)];
    raw bv[TT + TAPS - 1], xv[TT + TAPS - 1], cv[TT];
#pragma unroll
    for (int j = 0; j < TT + TAPS - 1; ++j) {
        const T* row = bcx + static_cast<size_t>(min(max(t0 - (TAPS - 1) + j, 0), n_tokens - 1)) * ld_bcx;
        bv[j] = *reinterpret_cast<const raw*>(row + ch);
        xv[j] = *reinterpret_cast<const raw*>(row + 2 * width + ch);
    }
#pragma unroll
    for (int j = 0; j < TT; ++j)
        cv[j] = *reinterpret_cast<const raw*>(bcx + static_cast<size_t>(min(t0 + j, n_tokens - 1)) * ld_bcx + width + ch);
    float wt[VEC][TAPS], b0[VEC];
#pragma unroll
    for (int i = 0; i < VEC; ++i) {
        b0[i] = bias ? bias[ch + i] : 0.f;
#pragma unroll
        for (int tap = 0; tap < TAPS; ++tap) wt[i][tap] = w[static_cast<size_t>(ch + i) * TAPS + tap];
    }
    // the same for the whole workgroup
    if (n < TT || s_end != s || t0 - (TAPS - 1) < cu_seqlens[s]) {
        for (int j = 0; j < n; ++j) {
            const int t = t0 + j;
            const int first = cu_seqlens[token_seq[t]];
            if (t - first < TAPS - 1 && first < t0) continue;      // the block of the request's first row has it
            short_conv_token_vec<T>(t, ch, bcx, ld_bcx, w, bias, state, state_slot_stride, out,
                                    positions, token_seq, seq_start, seq_slot, cu_seqlens, width, TAPS);
        }
        for (int j = 0; j < n; ++j) {
            const int t = t0 + j;
            const int sj = token_seq[t];
            if (cu_seqlens[sj] != t) continue;                     // requests that begin in this block:
            const int last = min(t + TAPS - 1, cu_seqlens[sj + 1]);
            for (int u = t0 + n; u < last; ++u)                    // their tokens in the next block that read the old state,
                short_conv_token_vec<T>(u, ch, bcx, ld_bcx, w, bias, state, state_slot_stride, out,
                                        positions, token_seq, seq_start, seq_slot, cu_seqlens, width, TAPS);
            short_conv_state_vec<T>(sj, ch, bcx, ld_bcx, state, state_slot_stride, seq_start, seq_slot,      // then the new one
                                    cu_seqlens, width, TAPS);
        }
        return;
    }
#pragma unroll
    for (int j = 0; j < TT; ++j) {
        raw o;
#pragma unroll
        for (int i = 0; i < VEC; ++i) {
            float conv = b0[i];
#pragma unroll
            for (int tap = 0; tap < TAPS; ++tap)
                conv = fmaf(wt[i][tap], ConvVec<T>::at(bv[j + tap], i) * ConvVec<T>::at(xv[j + tap], i), conv);
            ConvVec<T>::set(o, i, ConvVec<T>::at(cv[j], i) * conv);
        }
        *reinterpret_cast<raw*>(out + static_cast<size_t>(t0 + j) * width + ch) = o;
    }
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

// For tests and tuning: 4 tokens a thread in the kernel for long steps instead of CONV_BLOCK_TOKENS (0: the default).
static int g_force_block_tokens = 0;
extern "C" void celeg_short_conv_force_block_tokens(int tokens) { g_force_block_tokens = tokens; }

extern "C" int celeg_short_conv(const void* bcx, int ld_bcx, int dtype, const float* w,
                                const float* bias, float* state, size_t state_slot_stride,
                                void* out, const int* positions, const int* token_seq,
                                const int* seq_start, const int* seq_slot, const int* cu_seqlens,
                                int n_tokens, int n_seqs, int width, int taps,
                                hipStream_t stream) {
    if (n_tokens <= 0 || n_seqs <= 0) return 0;
    dim3 block(256);
    dim3 grid_fwd(n_tokens, (width + 255) / 256), grid_state(n_seqs, (width + 255) / 256);
    const int vec = dtype == CELEG_F32 ? 4 : 8;
    const auto aligned = [](const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15) == 0; };
    if (n_tokens >= 16 && taps <= CONV_VEC_MAX_TAPS && width % vec == 0 && ld_bcx % vec == 0 &&
        aligned(bcx) && aligned(out)) {
        const int threads = min(256, (width / vec + 63) / 64 * 64);
        dim3 vblock(threads), vgrid(n_tokens, (width / vec + threads - 1) / threads);
        if (taps >= 2 && taps <= 4) {      // (n_tokens >= 16 here)
            const int tt = g_force_block_tokens == 4 ? 4 : CONV_BLOCK_TOKENS;
            dim3 bgrid(((n_tokens + tt - 1) / tt + 7) / 8 * 8, vgrid.y);      // (8 runs of tokens, one a die)
#define CELEG_CONV_BLOCK(T_, TAPS_)                                                                \
    if (tt == 4) CELEG_CONV_BLOCK_TT(T_, TAPS_, 4); else CELEG_CONV_BLOCK_TT(T_, TAPS_, CONV_BLOCK_TOKENS)
#define CELEG_CONV_BLOCK_TT(T_, TAPS_, TT_)                                                        \
    hipLaunchKernelGGL((short_conv_fwd_block_kernel<T_, TAPS_, TT_>), bgrid, vblock, 0, stream,     \
                       static_cast<const T_*>(bcx), ld_bcx, w, bias, state, state_slot_stride,      \
                       static_cast<T_*>(out), positions, token_seq, seq_start, seq_slot, cu_seqlens, \
                       width, n_tokens)
#define CELEG_CONV_BLOCK_T(T_)                                                                     \
    if (taps == 2) { CELEG_CONV_BLOCK(T_, 2); } else if (taps == 3) { CELEG_CONV_BLOCK(T_, 3); }     \
    else { CELEG_CONV_BLOCK(T_, 4); }
            if (dtype == CELEG_F32) { CELEG_CONV_BLOCK_T(float) } else { CELEG_CONV_BLOCK_T(bf16) }
#undef CELEG_CONV_BLOCK_T
#undef CELEG_CONV_BLOCK_TT
#undef CELEG_CONV_BLOCK
            return CELEG_LAUNCH_RESULT();
        }
        if (dtype == CELEG_F32) {
            hipLaunchKernelGGL(short_conv_fwd_vec_kernel<float>, vgrid, vblock, 0, stream,
                               static_cast<const float*>(bcx), ld_bcx, w, bias, state,
                               state_slot_stride, static_cast<float*>(out), positions, token_seq,
                               seq_start, seq_slot, cu_seqlens, width, taps);
            hipLaunchKernelGGL(short_conv_state_kernel<float>, grid_state, block, 0, stream,
                               static_cast<const float*>(bcx), ld_bcx, state, state_slot_stride,
                               seq_start, seq_slot, cu_seqlens, width, taps);
        } else {
            hipLaunchKernelGGL(short_conv_fwd_vec_kernel<bf16>, vgrid, vblock, 0, stream,
                               static_cast<const bf16*>(bcx), ld_bcx, w, bias, state,
                               state_slot_stride, static_cast<bf16*>(out), positions, token_seq,
                               seq_start, seq_slot, cu_seqlens, width, taps);
            hipLaunchKernelGGL(short_conv_state_kernel<bf16>, grid_state, block, 0, stream,
                               static_cast<const bf16*>(bcx), ld_bcx, state, state_slot_stride,
                               seq_start, seq_slot, cu_seqlens, width, taps);
        }
        return CELEG_LAUNCH_RESULT();
    }
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
