// Row-wise and element-wise kernels: embedding gather, RMSNorm (with the residual
// addition folded in), SwiGLU, bias, dtype conversion, block-table updates.
#include "common.h"

// ---------------------------------------------------------------- embedding gather
// out[row, :] = table[ids[row], :], widened to 32-bit (the residual stream).
// Reference: src/backend/cuda/kernels/embedding.cu:26-37.
template <typename TW>
__global__ void embed_kernel(const TW* __restrict__ table, const int* __restrict__ ids,
                             float* __restrict__ out, int width, int vocab) {
    const int row = blockIdx.x;
    const int id = ids[row];
    float* dst = out + static_cast<size_t>(row) * width;
    if (id < 0 || id >= vocab) {  // the host rejects such ids; never read out of bounds
        for (int i = threadIdx.x; i < width; i += blockDim.x) dst[i] = 0.f;
        return;
    }
    const TW* src = table + static_cast<size_t>(id) * width;
    for (int i = threadIdx.x; i < width; i += blockDim.x) dst[i] = to_float(src[i]);
}

extern "C" int celeg_embed(const void* table, int table_dtype, const int* ids, float* out,
                           int rows, int width, int vocab, hipStream_t stream) {
    if (rows <= 0) return 0;
    dim3 grid(rows), block(256);
    if (table_dtype == CELEG_F32)
        hipLaunchKernelGGL(embed_kernel<float>, grid, block, 0, stream,
                           static_cast<const float*>(table), ids, out, width, vocab);
    else
        hipLaunchKernelGGL(embed_kernel<bf16>, grid, block, 0, stream,
                           static_cast<const bf16*>(table), ids, out, width, vocab);
    return CELEG_LAUNCH_RESULT();
}

// ---------------------------------------------------------------- RMSNorm
// out[r, :] = v * rsqrt(mean(v^2) + eps) * w with v = x[src, :] (+ delta[src, :]),
// src = rows ? rows[r] : r.  With write_back the sum v is stored to x (the 32-bit
// residual stream).  Sum of squares, scaling and the sum itself are 32-bit.
// Reference: src/backend/cpu/kernels/elementwise.cpp:56-76 (eps inside the root,
// (x*inv)*w); CUDA kernels/norm.cuh:1-44.
template <typename TX, typename TD, typename TO>
__global__ void rmsnorm_kernel(TX* __restrict__ x, const TD* __restrict__ delta,
                               const float* __restrict__ w, TO* __restrict__ out,
                               const int* __restrict__ rows, int width, float eps,
                               int write_back) {
    __shared__ float scratch[16];
    const int r = blockIdx.x;
    const size_t src = static_cast<size_t>(rows ? rows[r] : r) * width;
    float sum = 0.f;
    for (int i = threadIdx.x; i < width; i += blockDim.x) {
        float v = to_float(x[src + i]);
        if (delta) {
            v += to_float(delta[src + i]);
            if (write_back) x[src + i] = from_float<TX>(v);
        }
        sum += v * v;
    }
    sum = block_sum(sum, scratch);
    const float inv = 1.0f / sqrtf(sum / static_cast<float>(width) + eps);
    TO* dst = out + static_cast<size_t>(r) * width;
    for (int i = threadIdx.x; i < width; i += blockDim.x) {
        float v = to_float(x[src + i]);
        if (delta && !write_back) v += to_float(delta[src + i]);
        dst[i] = from_float<TO>(v * inv * w[i]);
    }
}

// The same with the row kept in registers: groups of 4 values, up to RMS_NV groups a
// thread (width <= 4 * RMS_NV * 256), every load of a row asked for before the first is used.
#define RMS_NV 4
template <typename T> struct Vec4;
template <> struct Vec4<float> {
    typedef float raw __attribute__((ext_vector_type(4)));
    static __device__ __forceinline__ void load(const float* p, float (&v)[4]) {
        const raw r = *reinterpret_cast<const raw*>(p);
        v[0] = r[0]; v[1] = r[1]; v[2] = r[2]; v[3] = r[3];
    }
    static __device__ __forceinline__ void store(float* p, const float (&v)[4]) {
        *reinterpret_cast<raw*>(p) = raw{v[0], v[1], v[2], v[3]};
    }
};
template <> struct Vec4<bf16> {
    typedef __bf16 raw __attribute__((ext_vector_type(4)));
    static __device__ __forceinline__ void load(const bf16* p, float (&v)[4]) {
        const raw r = *reinterpret_cast<const raw*>(p);
        v[0] = static_cast<float>(r[0]); v[1] = static_cast<float>(r[1]);
        v[2] = static_cast<float>(r[2]); v[3] = static_cast<float>(r[3]);
    }
    static __device__ __forceinline__ void store(bf16* p, const float (&v)[4]) {
        *reinterpret_cast<raw*>(p) = raw{static_cast<__bf16>(v[0]), static_cast<__bf16>(v[1]),
                                         static_cast<__bf16>(v[2]), static_cast<__bf16>(v[3])};
    }
};

template <typename TX, typename TD, typename TO>
__global__ __launch_bounds__(256) void rmsnorm_vec_kernel(
    TX* __restrict__ x, const TD* __restrict__ delta, const float* __restrict__ w,
    TO* __restrict__ out, const int* __restrict__ rows, int width, float eps, int write_back) {
    __shared__ float scratch[16];
    const int r = blockIdx.x;
    const size_t src = static_cast<size_t>(rows ? rows[r] : r) * width;
    const int groups = width >> 2;
    float v[RMS_NV][4], d[RMS_NV][4], wv[RMS_NV][4];
#pragma unroll
    for (int j = 0; j < RMS_NV; ++j) {
        const int g = min(static_cast<int>(threadIdx.x) + j * 256, groups - 1);   // clamped, masked below
        Vec4<TX>::load(x + src + 4 * g, v[j]);
        if (delta) Vec4<TD>::load(delta + src + 4 * g, d[j]);
        Vec4<float>::load(w + 4 * g, wv[j]);
    }
    float sum = 0.f;
#pragma unroll
    for (int j = 0; j < RMS_NV; ++j) {
        const bool in = static_cast<int>(threadIdx.x) + j * 256 < groups;
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            if (delta) v[j][e] += d[j][e];
            if (in) sum += v[j][e] * v[j][e];
        }
        if (in && delta && write_back) Vec4<TX>::store(x + src + 4 * (threadIdx.x + j * 256), v[j]);
    }
    sum = block_sum(sum, scratch);
    const float inv = 1.0f / sqrtf(sum / static_cast<float>(width) + eps);
    TO* dst = out + static_cast<size_t>(r) * width;
#pragma unroll
    for (int j = 0; j < RMS_NV; ++j) {
        if (static_cast<int>(threadIdx.x) + j * 256 < groups) {
            float o[4];
#pragma unroll
            for (int e = 0; e < 4; ++e) o[e] = v[j][e] * inv * wv[j][e];
            Vec4<TO>::store(dst + 4 * (threadIdx.x + j * 256), o);
        }
    }
}

// One wavefront per row (width <= 4 * RMS_NV * 64): no barrier, 4 rows a workgroup.
template <typename TX, typename TD, typename TO>
__global__ __launch_bounds__(256) void rmsnorm_wave_kernel(
    TX* __restrict__ x, const TD* __restrict__ delta, const float* __restrict__ w,
    TO* __restrict__ out, const int* __restrict__ rows, int n_rows, int width, float eps,
    int write_back) {
    const int lane = threadIdx.x & 63;
    const int r = blockIdx.x * 4 + (threadIdx.x >> 6);
    if (r >= n_rows) return;
    const size_t src = static_cast<size_t>(rows ? rows[r] : r) * width;
    const int groups = width >> 2;
    float v[RMS_NV][4], d[RMS_NV][4], wv[RMS_NV][4];
#pragma unroll
    for (int j = 0; j < RMS_NV; ++j) {
        const int g = min(lane + j * 64, groups - 1);   // clamped, masked below
        Vec4<TX>::load(x + src + 4 * g, v[j]);
        if (delta) Vec4<TD>::load(delta + src + 4 * g, d[j]);
        Vec4<float>::load(w + 4 * g, wv[j]);
    }
    float sum = 0.f;
#pragma unroll
    for (int j = 0; j < RMS_NV; ++j) {
        const bool in = lane + j * 64 < groups;
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            if (delta) v[j][e] += d[j][e];
            if (in) sum += v[j][e] * v[j][e];
        }
        if (in && delta && write_back) Vec4<TX>::store(x + src + 4 * (lane + j * 64), v[j]);
    }
    sum = wave_sum(sum);
    const float inv = 1.0f / sqrtf(sum / static_cast<float>(width) + eps);
    TO* dst = out + static_cast<size_t>(r) * width;
#pragma unroll
    for (int j = 0; j < RMS_NV; ++j) {
        if (lane + j * 64 < groups) {
            float o[4];
#pragma unroll
            for (int e = 0; e < 4; ++e) o[e] = v[j][e] * inv * wv[j][e];
            Vec4<TO>::store(dst + 4 * (lane + j * 64), o);
        }
    }
}

template <typename TX, typename TD>
static int rmsnorm_dispatch_out(TX* x, const TD* delta, const float* w, void* out, int out_dtype,
                                const int* rows, int n_rows, int width, float eps,
                                int write_back, hipStream_t stream) {
    dim3 grid(n_rows), block(width >= 1024 ? 256 : (width >= 256 ? 128 : 64));
    const auto aligned = [](const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15) == 0; };
    if (width % 4 == 0 && width >= 256 && width <= 4 * RMS_NV * 256 && aligned(x) && aligned(w) &&
        aligned(out) && (!delta || aligned(delta))) {
        if (width <= 4 * RMS_NV * 64 && n_rows >= 64) {   // many short rows: a wavefront each
            dim3 wgrid((n_rows + 3) / 4);
            if (out_dtype == CELEG_F32)
                hipLaunchKernelGGL((rmsnorm_wave_kernel<TX, TD, float>), wgrid, dim3(256), 0, stream, x,
                                   delta, w, static_cast<float*>(out), rows, n_rows, width, eps, write_back);
            else
                hipLaunchKernelGGL((rmsnorm_wave_kernel<TX, TD, bf16>), wgrid, dim3(256), 0, stream, x,
                                   delta, w, static_cast<bf16*>(out), rows, n_rows, width, eps, write_back);
            return CELEG_LAUNCH_RESULT();
        }
        if (out_dtype == CELEG_F32)
            hipLaunchKernelGGL((rmsnorm_vec_kernel<TX, TD, float>), grid, dim3(256), 0, stream, x, delta,
                               w, static_cast<float*>(out), rows, width, eps, write_back);
        else
            hipLaunchKernelGGL((rmsnorm_vec_kernel<TX, TD, bf16>), grid, dim3(256), 0, stream, x, delta,
                               w, static_cast<bf16*>(out), rows, width, eps, write_back);
        return CELEG_LAUNCH_RESULT();
    }
    if (out_dtype == CELEG_F32)
        hipLaunchKernelGGL((rmsnorm_kernel<TX, TD, float>), grid, block, 0, stream, x, delta, w,
                           static_cast<float*>(out), rows, width, eps, write_back);
    else
        hipLaunchKernelGGL((rmsnorm_kernel<TX, TD, bf16>), grid, block, 0, stream, x, delta, w,
                           static_cast<bf16*>(out), rows, width, eps, write_back);
    return CELEG_LAUNCH_RESULT();
}

// x_dtype: dtype of x; delta_dtype: dtype of delta (ignored if delta is null).
// write_back requires x in 32-bit (it is the residual stream).
extern "C" int celeg_rmsnorm(void* x, int x_dtype, const void* delta, int delta_dtype,
                             const float* w, void* out, int out_dtype, const int* rows,
                             int n_rows, int width, float eps, int write_back,
                             hipStream_t stream) {
    if (n_rows <= 0) return 0;
    if (write_back && x_dtype != CELEG_F32) return static_cast<int>(hipErrorInvalidValue);
    if (x_dtype == CELEG_F32) {
        float* xf = static_cast<float*>(x);
        if (delta && delta_dtype == CELEG_BF16)
            return rmsnorm_dispatch_out<float, bf16>(xf, static_cast<const bf16*>(delta), w, out,
                                                     out_dtype, rows, n_rows, width, eps,
                                                     write_back, stream);
        return rmsnorm_dispatch_out<float, float>(xf, static_cast<const float*>(delta), w, out,
                                                  out_dtype, rows, n_rows, width, eps,
                                                  write_back, stream);
    }
    bf16* xb = static_cast<bf16*>(x);
    if (delta && delta_dtype == CELEG_F32)
        return rmsnorm_dispatch_out<bf16, float>(xb, static_cast<const float*>(delta), w, out,
                                                 out_dtype, rows, n_rows, width, eps, 0, stream);
    return rmsnorm_dispatch_out<bf16, bf16>(xb, static_cast<const bf16*>(delta), w, out,
                                            out_dtype, rows, n_rows, width, eps, 0, stream);
}

// ---------------------------------------------------------------- SwiGLU
// out[t, i] = silu(gu[t, i]) * gu[t, ff + i], silu(g) = g / (1 + exp(-g)); computed in
// 32-bit and rounded once.  Reference: src/backend/cpu/kernels/elementwise.cpp:101-119.
template <typename T>
__global__ void swiglu_kernel(const T* __restrict__ gu, T* __restrict__ out, int ff,
                              size_t total) {
    const size_t i = static_cast<size_t>(blockIdx.x) * blockDim.x + threadIdx.x;
    if (i >= total) return;
    const size_t t = i / ff;
    const int c = static_cast<int>(i - t * ff);
    const float g = to_float(gu[t * 2 * ff + c]);
    const float u = to_float(gu[t * 2 * ff + ff + c]);
    out[i] = from_float<T>((g / (1.0f + expf(-g))) * u);
}

// groups of 8 values a thread (ff % 8 == 0)
template <typename T>
__global__ __launch_bounds__(256) void swiglu_vec_kernel(const T* __restrict__ gu, T* __restrict__ out,
                                                         int ff, size_t groups) {
    const size_t i = static_cast<size_t>(blockIdx.x) * blockDim.x + threadIdx.x;
    if (i >= groups) return;
    const int per_row = ff >> 3;
    const size_t t = i / per_row;
    const int c = static_cast<int>(i - t * per_row) * 8;
    float g[2][4], u[2][4], o[2][4];
#pragma unroll
    for (int h = 0; h < 2; ++h) {
        Vec4<T>::load(gu + t * 2 * ff + c + 4 * h, g[h]);
        Vec4<T>::load(gu + t * 2 * ff + ff + c + 4 * h, u[h]);
    }
#pragma unroll
    for (int h = 0; h < 2; ++h) {
#pragma unroll
        for (int e = 0; e < 4; ++e) o[h][e] = (g[h][e] / (1.0f + expf(-g[h][e]))) * u[h][e];
        Vec4<T>::store(out + t * ff + c + 4 * h, o[h]);
    }
}

extern "C" int celeg_swiglu(const void* gu, void* out, int dtype, int rows, int ff,
                            hipStream_t stream) {
    const size_t total = static_cast<size_t>(rows) * ff;
    if (total == 0) return 0;
    if (ff % 8 == 0 && (reinterpret_cast<uintptr_t>(gu) & 15) == 0 && (reinterpret_cast<uintptr_t>(out) & 15) == 0) {
        const size_t groups = total / 8;
        dim3 vblock(256), vgrid(static_cast<unsigned>((groups + 255) / 256));
        if (dtype == CELEG_F32)
            hipLaunchKernelGGL(swiglu_vec_kernel<float>, vgrid, vblock, 0, stream,
                               static_cast<const float*>(gu), static_cast<float*>(out), ff, groups);
        else
            hipLaunchKernelGGL(swiglu_vec_kernel<bf16>, vgrid, vblock, 0, stream,
                               static_cast<const bf16*>(gu), static_cast<bf16*>(out), ff, groups);
        return CELEG_LAUNCH_RESULT();
    }
    dim3 block(256), grid(static_cast<unsigned>((total + 255) / 256));
    if (dtype == CELEG_F32)
        hipLaunchKernelGGL(swiglu_kernel<float>, grid, block, 0, stream,
                           static_cast<const float*>(gu), static_cast<float*>(out), ff, total);
    else
        hipLaunchKernelGGL(swiglu_kernel<bf16>, grid, block, 0, stream,
                           static_cast<const bf16*>(gu), static_cast<bf16*>(out), ff, total);
    return CELEG_LAUNCH_RESULT();
}

// ---------------------------------------------------------------- bias
template <typename T>
__global__ void add_bias_kernel(T* __restrict__ x, const float* __restrict__ bias, int width,
                                size_t total) {
    const size_t i = static_cast<size_t>(blockIdx.x) * blockDim.x + threadIdx.x;
    if (i >= total) return;
    x[i] = from_float<T>(to_float(x[i]) + bias[i % width]);
}

extern "C" int celeg_add_bias(void* x, int dtype, const float* bias, int rows, int width,
                              hipStream_t stream) {
    const size_t total = static_cast<size_t>(rows) * width;
    if (total == 0) return 0;
    dim3 block(256), grid(static_cast<unsigned>((total + 255) / 256));
    if (dtype == CELEG_F32)
        hipLaunchKernelGGL(add_bias_kernel<float>, grid, block, 0, stream, static_cast<float*>(x),
                           bias, width, total);
    else
        hipLaunchKernelGGL(add_bias_kernel<bf16>, grid, block, 0, stream, static_cast<bf16*>(x),
                           bias, width, total);
    return CELEG_LAUNCH_RESULT();
}

// ---------------------------------------------------------------- conversion
template <typename TS, typename TD>
__global__ void cast_kernel(const TS* __restrict__ src, TD* __restrict__ dst, size_t total) {
    const size_t i = static_cast<size_t>(blockIdx.x) * blockDim.x + threadIdx.x;
    if (i < total) dst[i] = from_float<TD>(to_float(src[i]));
}

extern "C" int celeg_cast(const void* src, int src_dtype, void* dst, int dst_dtype, size_t total,
                          hipStream_t stream) {
    if (total == 0) return 0;
    dim3 block(256), grid(static_cast<unsigned>((total + 255) / 256));
    if (src_dtype == CELEG_BF16 && dst_dtype == CELEG_F32)
        hipLaunchKernelGGL((cast_kernel<bf16, float>), grid, block, 0, stream,
                           static_cast<const bf16*>(src), static_cast<float*>(dst), total);
    else if (src_dtype == CELEG_F32 && dst_dtype == CELEG_BF16)
        hipLaunchKernelGGL((cast_kernel<float, bf16>), grid, block, 0, stream,
                           static_cast<const float*>(src), static_cast<bf16*>(dst), total);
    else if (src_dtype == CELEG_F32 && dst_dtype == CELEG_F32)
        hipLaunchKernelGGL((cast_kernel<float, float>), grid, block, 0, stream,
                           static_cast<const float*>(src), static_cast<float*>(dst), total);
    else
        hipLaunchKernelGGL((cast_kernel<bf16, bf16>), grid, block, 0, stream,
                           static_cast<const bf16*>(src), static_cast<bf16*>(dst), total);
    return CELEG_LAUNCH_RESULT();
}

// ---------------------------------------------------------------- block-table updates
// updates = [n, (slot, logical page, physical page) * n]; table[slot, logical] = physical.
// The launch covers `capacity` triples; threads beyond n do nothing, so a captured
// graph can replay it with any n <= capacity.
__global__ void table_update_kernel(int* __restrict__ table, int stride, int n_slots,
                                    const int* __restrict__ updates, int capacity) {
    const int i = blockIdx.x * blockDim.x + threadIdx.x;
    const int n = min(updates[0], capacity);
    if (i >= n) return;
    const int slot = updates[1 + 3 * i], logical = updates[2 + 3 * i], page = updates[3 + 3 * i];
    if (slot < 0 || slot >= n_slots || logical < 0 || logical >= stride) return;
    table[static_cast<size_t>(slot) * stride + logical] = page;
}

extern "C" int celeg_table_update(int* table, int stride, int n_slots, const int* updates,
                                  int capacity, hipStream_t stream) {
    if (capacity <= 0) return 0;
    dim3 block(64), grid((capacity + 63) / 64);
    hipLaunchKernelGGL(table_update_kernel, grid, block, 0, stream, table, stride, n_slots,
                       updates, capacity);
    return CELEG_LAUNCH_RESULT();
}

// ---------------------------------------------------------------- tokens from the device
// A row whose token id is negative takes the token its request sampled last:
// token_ids[i] = last_tokens[token_slot[i]].  Lets the host launch a decode step before it
// has read the previous step's tokens.
__global__ void resolve_tokens_kernel(int* __restrict__ token_ids, const int* __restrict__ token_slot,
                                      const int* __restrict__ last_tokens, int n) {
    const int i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= n) return;
    if (token_ids[i] < 0) token_ids[i] = last_tokens[token_slot[i]];
}

// Both of the above in one launch (a step begins with them; one kernel fewer in a step that is
// bound by its number of kernels).  Threads [0, capacity) take the triples, threads
// [0, n) the rows; last_tokens null: no rows to resolve.
__global__ void step_prologue_kernel(int* __restrict__ table, int stride, int n_slots,
                                     const int* __restrict__ updates, int capacity,
                                     int* __restrict__ token_ids, const int* __restrict__ token_slot,
                                     const int* __restrict__ last_tokens, int n) {
    const int i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i < min(updates[0], capacity)) {
        const int slot = updates[1 + 3 * i], logical = updates[2 + 3 * i], page = updates[3 + 3 * i];
        if (slot >= 0 && slot < n_slots && logical >= 0 && logical < stride)
            table[static_cast<size_t>(slot) * stride + logical] = page;
    }
    if (last_tokens && i < n && token_ids[i] < 0) token_ids[i] = last_tokens[token_slot[i]];
}

extern "C" int celeg_step_prologue(int* table, int stride, int n_slots, const int* updates, int capacity,
                                   int* token_ids, const int* token_slot, const int* last_tokens, int n,
                                   hipStream_t stream) {
    const int threads = max(capacity, last_tokens ? n : 0);
    if (threads <= 0) return 0;
    if (capacity <= 0) return static_cast<int>(hipErrorInvalidValue);   // the update list is read
    hipLaunchKernelGGL(step_prologue_kernel, dim3((threads + 255) / 256), dim3(256), 0, stream, table,
                       stride, n_slots, updates, capacity, token_ids, token_slot, last_tokens, n);
    return CELEG_LAUNCH_RESULT();
}

extern "C" int celeg_resolve_tokens(int* token_ids, const int* token_slot, const int* last_tokens,
                                    int n, hipStream_t stream) {
    if (n <= 0) return 0;
    hipLaunchKernelGGL(resolve_tokens_kernel, dim3((n + 255) / 256), dim3(256), 0, stream, token_ids,
                       token_slot, last_tokens, n);
    return CELEG_LAUNCH_RESULT();
}

// ---------------------------------------------------------------- weights re-laid at load time
// out = w with column k scaled by scale[k] (a norm's weight folded into the matrix that follows
// it: (x * s) w^T = x (w * s)^T; scale null: a plain copy), rounded to bfloat16 once, either
// with the rows one after the other or in blocks of 32 k-values with the rows side by side
// inside a block ([K/32, rows, 32], what the products for few rows read in whole runs).
__global__ void fold_weight_kernel(const bf16* __restrict__ w, const float* __restrict__ scale,
                                   bf16* __restrict__ out, int rows, int K, int packed) {
    const size_t i = static_cast<size_t>(blockIdx.x) * blockDim.x + threadIdx.x;
    const size_t total = static_cast<size_t>(rows) * K;
    if (i >= total) return;
    const int n = static_cast<int>(i / K), k = static_cast<int>(i % K);
    const float v = scale ? to_float(w[i]) * scale[k] : to_float(w[i]);
    const size_t at = packed ? (static_cast<size_t>(k / 32) * rows + n) * 32 + k % 32 : i;
    out[at] = from_float<bf16>(v);
}

extern "C" int celeg_fold_weight(const void* w, const float* scale, void* out, int rows, int K,
                                 int packed, hipStream_t stream) {
    if (rows <= 0 || K <= 0) return 0;
    if (packed && K % 32) return static_cast<int>(hipErrorInvalidValue);
    const size_t total = static_cast<size_t>(rows) * K;
    hipLaunchKernelGGL(fold_weight_kernel, dim3(static_cast<unsigned>((total + 255) / 256)), dim3(256), 0,
                       stream, static_cast<const bf16*>(w), scale, static_cast<bf16*>(out), rows, K, packed);
    return CELEG_LAUNCH_RESULT();
}

// bytes [0, n) of p set to zero by a kernel (what a recorded graph may hold, unlike a memset node)
__global__ void zero_bytes_kernel(uint32_t* __restrict__ p, size_t words) {
    const size_t i = static_cast<size_t>(blockIdx.x) * blockDim.x + threadIdx.x;
    if (i < words) p[i] = 0u;
}

extern "C" int celeg_zero_words(void* p, size_t words, hipStream_t stream) {
    if (words == 0) return 0;
    hipLaunchKernelGGL(zero_bytes_kernel, dim3(static_cast<unsigned>((words + 255) / 256)), dim3(256), 0,
                       stream, static_cast<uint32_t*>(p), words);
    return CELEG_LAUNCH_RESULT();
}
