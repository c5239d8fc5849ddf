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

template <typename TX, typename TD>
static int rmsnorm_dispatch_out(TX* x, const TD* delta, const float* w, void* out, int out_dtype,
                                const int* rows, int n_rows, int width, float eps,
                                int write_back, hipStream_t stream) {
    dim3 grid(n_rows), block(width >= 1024 ? 256 : (width >= 256 ? 128 : 64));
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

extern "C" int celeg_swiglu(const void* gu, void* out, int dtype, int rows, int ff,
                            hipStream_t stream) {
    const size_t total = static_cast<size_t>(rows) * ff;
    if (total == 0) return 0;
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
