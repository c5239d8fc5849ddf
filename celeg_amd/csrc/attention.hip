// Attention over the paged cache: (1) per-head RMSNorm + rotary encoding of q and k,
// with k and v written into their pages; (2) a general attention kernel that serves
// every kind of row (prompt portions and decode tokens) in both dtypes.
//
// Cache layout of a group: K [pages, layers, kv_heads, page_tokens, head_dim] and
// V [pages, layers, kv_heads, head_dim, page_tokens] (transposed inside the page, which
// is what the matrix-core kernel of attention_fast.hip wants).
// A row at position p of the request in slot s lives in page table[s, p / page_tokens]
// at place p % page_tokens.  (The reference's layout and addressing:
// src/backend/cuda/kernels/kv_cache.cuh:1-7, 215-240.)
#include "common.h"

__device__ __forceinline__ size_t cache_offset(int page, int n_layers, int layer, int kv_heads,
                                               int head, int page_tokens, int in_page,
                                               int head_dim) {
    return (((static_cast<size_t>(page) * n_layers + layer) * kv_heads + head) * page_tokens +
            in_page) * head_dim;
}

// ---------------------------------------------------------------- q/k norm + rope + store
// One wavefront per (row, head); heads [0,Hq) are q, [Hq,Hq+Hkv) are k, the rest are v.
// Per head: inv = 1/sqrt(mean(x^2)+eps); x = x*inv*w (if a norm weight is given);
// split-half rotation of pairs (i, i+rot/2) by angle = float(pos)*inv_freq[i] (if a
// frequency table is given); q goes back in place, k and v go to the cache.
// Reference: src/backend/cpu/kernels/rope.cpp:61-111; CUDA kernels/rope.cuh:333-393.
template <typename T>
__global__ void qk_norm_rope_store_kernel(
    T* __restrict__ q, int ldq, const T* __restrict__ k, int ldk, const T* __restrict__ v, int ldv,
    const float* __restrict__ q_weight, const float* __restrict__ k_weight, float eps,
    const float* __restrict__ inv_freq, int rotary_dim, const int* __restrict__ positions,
    const int* __restrict__ token_slot, const int* __restrict__ table, int table_stride,
    T* __restrict__ k_pool, T* __restrict__ v_pool, int n_layers, int layer, int page_tokens,
    int q_heads, int kv_heads, int head_dim) {
    extern __shared__ float vals[];  // head_dim floats
    const int t = blockIdx.x;
    const int head = blockIdx.y;
    const int lane = threadIdx.x;
    const int pos = positions[t];
    const bool is_q = head < q_heads;
    const bool is_k = !is_q && head < q_heads + kv_heads;
    const int kv_head = is_q ? 0 : (is_k ? head - q_heads : head - q_heads - kv_heads);

    T* dst;
    if (is_q) {
        dst = q + static_cast<size_t>(t) * ldq + static_cast<size_t>(head) * head_dim;
    } else {
        const int page = table[static_cast<size_t>(token_slot[t]) * table_stride + pos / page_tokens];
        if (!is_k) {  // v: copy, transposed inside the page
            T* vdst = v_pool + cache_offset(page, n_layers, layer, kv_heads, kv_head, page_tokens,
                                            0, head_dim) + pos % page_tokens;
            const T* src = v + static_cast<size_t>(t) * ldv + static_cast<size_t>(kv_head) * head_dim;
            for (int d = lane; d < head_dim; d += CELEG_WAVE)
                vdst[static_cast<size_t>(d) * page_tokens] = src[d];
            return;
        }
        dst = k_pool + cache_offset(page, n_layers, layer, kv_heads, kv_head, page_tokens,
                                    pos % page_tokens, head_dim);
    }
    const T* src = is_q ? q + static_cast<size_t>(t) * ldq + static_cast<size_t>(head) * head_dim
                        : k + static_cast<size_t>(t) * ldk + static_cast<size_t>(kv_head) * head_dim;
    const float* weight = is_q ? q_weight : k_weight;
    float sum = 0.f;
    for (int d = lane; d < head_dim; d += CELEG_WAVE) {
        const float x = to_float(src[d]);
        vals[d] = x;
        sum += x * x;
    }
    if (weight) {
        sum = wave_sum(sum);
        const float inv = 1.0f / sqrtf(sum / static_cast<float>(head_dim) + eps);
        for (int d = lane; d < head_dim; d += CELEG_WAVE) vals[d] = vals[d] * inv * weight[d];
    }
    __syncthreads();
    const int half = rotary_dim / 2;
    for (int d = lane; d < head_dim; d += CELEG_WAVE) {
        float y = vals[d];
        if (inv_freq && d < rotary_dim) {
            const int i = d < half ? d : d - half;
            const float angle = static_cast<float>(pos) * inv_freq[i];
            const float c = cosf(angle), s = sinf(angle);
            const float a = vals[i], b = vals[i + half];
            y = d < half ? a * c - b * s : b * c + a * s;
        }
        dst[d] = from_float<T>(y);
    }
}

extern "C" int celeg_qk_norm_rope_store(
    void* q, int ldq, const void* k, int ldk, const void* v, int ldv, int dtype,
    const float* q_weight, const float* k_weight, float eps, const float* inv_freq,
    int rotary_dim, const int* positions, const int* token_slot, const int* table,
    int table_stride, void* k_pool, void* v_pool, int n_layers, int layer, int page_tokens,
    int n_tokens, int q_heads, int kv_heads, int head_dim, int store_kv, hipStream_t stream) {
    if (n_tokens <= 0) return 0;
    dim3 grid(n_tokens, q_heads + (store_kv ? 2 * kv_heads : 0)), block(CELEG_WAVE);
    const size_t lds = static_cast<size_t>(head_dim) * sizeof(float);
    if (dtype == CELEG_F32)
        hipLaunchKernelGGL(qk_norm_rope_store_kernel<float>, grid, block, lds, stream,
                           static_cast<float*>(q), ldq, static_cast<const float*>(k), ldk,
                           static_cast<const float*>(v), ldv, q_weight, k_weight, eps, inv_freq,
                           rotary_dim, positions, token_slot, table, table_stride,
                           static_cast<float*>(k_pool), static_cast<float*>(v_pool), n_layers,
                           layer, page_tokens, q_heads, kv_heads, head_dim);
    else
        hipLaunchKernelGGL(qk_norm_rope_store_kernel<bf16>, grid, block, lds, stream,
                           static_cast<bf16*>(q), ldq, static_cast<const bf16*>(k), ldk,
                           static_cast<const bf16*>(v), ldv, q_weight, k_weight, eps, inv_freq,
                           rotary_dim, positions, token_slot, table, table_stride,
                           static_cast<bf16*>(k_pool), static_cast<bf16*>(v_pool), n_layers,
                           layer, page_tokens, q_heads, kv_heads, head_dim);
    return CELEG_LAUNCH_RESULT();
}

// ---------------------------------------------------------------- general attention
// One wavefront per (row, query head).  Keys at positions [first, pos] of the row's
// request, first = max(0, pos - window + 1) with a window, else 0; 64 keys at a time:
// every lane scores one key, the chunk joins a running (max, sum, accumulator) in
// 32-bit.  The chunking depends only on the row's own position, so a row's result is
// the same whatever else is in the batch.  scores = (q.k)*scale, scale applied once
// (reference: src/backend/cpu/attention/paged_attention.cpp:229-283;
// CUDA kernels/attention_paged.cuh:2-141).
#define ATT_MAX_DIM_CHUNKS 4  // head_dim <= 256

template <typename T>
__global__ void paged_attention_kernel(
    const T* __restrict__ q, int ldq, const T* __restrict__ k_pool, const T* __restrict__ v_pool,
    const int* __restrict__ table, int table_stride, const int* __restrict__ token_slot,
    const int* __restrict__ positions, T* __restrict__ out, int ldo, int q_heads, int kv_heads,
    int head_dim, int page_tokens, int n_layers, int layer, float scale, int window) {
    extern __shared__ float lds[];  // head_dim floats of q, then 64 probabilities
    float* qs = lds;
    float* ps = lds + head_dim;
    const int t = blockIdx.x;
    const int h = blockIdx.y;
    const int lane = threadIdx.x;
    const int kvh = h / (q_heads / kv_heads);
    const int pos = positions[t];
    const int* pages = table + static_cast<size_t>(token_slot[t]) * table_stride;
    const int first = window > 0 ? max(0, pos - window + 1) : 0;

    const T* qrow = q + static_cast<size_t>(t) * ldq + static_cast<size_t>(h) * head_dim;
    for (int d = lane; d < head_dim; d += CELEG_WAVE) qs[d] = to_float(qrow[d]);
    __syncthreads();

    float m = -INFINITY, l = 0.f;
    float acc[ATT_MAX_DIM_CHUNKS];
#pragma unroll
    for (int j = 0; j < ATT_MAX_DIM_CHUNKS; ++j) acc[j] = 0.f;

    for (int base = first; base <= pos; base += CELEG_WAVE) {
        const int key = base + lane;
        const bool valid = key <= pos;
        float s = -INFINITY;
        if (valid) {
            const T* kp = k_pool + cache_offset(pages[key / page_tokens], n_layers, layer, kv_heads,
                                                kvh, page_tokens, key % page_tokens, head_dim);
            float dot = 0.f;
            for (int d = 0; d < head_dim; ++d) dot = fmaf(qs[d], to_float(kp[d]), dot);
            s = dot * scale;
        }
        const float m_new = fmaxf(m, wave_max(s));
        const float p = valid ? expf(s - m_new) : 0.f;
        const float corr = expf(m - m_new);  // m = -inf at the first chunk gives 0
        l = l * corr + wave_sum(p);
        ps[lane] = p;
        __syncthreads();
#pragma unroll
        for (int j = 0; j < ATT_MAX_DIM_CHUNKS; ++j) acc[j] *= corr;
        const int n_keys = min(CELEG_WAVE, pos - base + 1);
        for (int kk = 0; kk < n_keys; ++kk) {
            const int key2 = base + kk;
            const T* vp = v_pool + cache_offset(pages[key2 / page_tokens], n_layers, layer,
                                                kv_heads, kvh, page_tokens, 0, head_dim) +
                          key2 % page_tokens;
            const float pk = ps[kk];
#pragma unroll
            for (int j = 0; j < ATT_MAX_DIM_CHUNKS; ++j) {
                const int d = lane + j * CELEG_WAVE;
                if (d < head_dim)
                    acc[j] = fmaf(pk, to_float(vp[static_cast<size_t>(d) * page_tokens]), acc[j]);
            }
        }
        __syncthreads();
        m = m_new;
    }
    T* orow = out + static_cast<size_t>(t) * ldo + static_cast<size_t>(h) * head_dim;
    const float inv_l = 1.0f / l;
#pragma unroll
    for (int j = 0; j < ATT_MAX_DIM_CHUNKS; ++j) {
        const int d = lane + j * CELEG_WAVE;
        if (d < head_dim) orow[d] = from_float<T>(acc[j] * inv_l);
    }
}

extern "C" int celeg_paged_attention(
    const void* q, int ldq, const void* k_pool, const void* v_pool, int dtype, const int* table,
    int table_stride, const int* token_slot, const int* positions, void* out, int ldo,
    int n_tokens, int q_heads, int kv_heads, int head_dim, int page_tokens, int n_layers,
    int layer, float scale, int window, hipStream_t stream) {
    if (n_tokens <= 0) return 0;
    if (head_dim > ATT_MAX_DIM_CHUNKS * CELEG_WAVE || q_heads % kv_heads)
        return static_cast<int>(hipErrorInvalidValue);
    dim3 grid(n_tokens, q_heads), block(CELEG_WAVE);
    const size_t lds = static_cast<size_t>(head_dim + CELEG_WAVE) * sizeof(float);
    if (dtype == CELEG_F32)
        hipLaunchKernelGGL(paged_attention_kernel<float>, grid, block, lds, stream,
                           static_cast<const float*>(q), ldq, static_cast<const float*>(k_pool),
                           static_cast<const float*>(v_pool), table, table_stride, token_slot,
                           positions, static_cast<float*>(out), ldo, q_heads, kv_heads, head_dim,
                           page_tokens, n_layers, layer, scale, window);
    else
        hipLaunchKernelGGL(paged_attention_kernel<bf16>, grid, block, lds, stream,
                           static_cast<const bf16*>(q), ldq, static_cast<const bf16*>(k_pool),
                           static_cast<const bf16*>(v_pool), table, table_stride, token_slot,
                           positions, static_cast<bf16*>(out), ldo, q_heads, kv_heads, head_dim,
                           page_tokens, n_layers, layer, scale, window);
    return CELEG_LAUNCH_RESULT();
}
