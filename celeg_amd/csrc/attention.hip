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
// rotation of pair i by angle = float(pos)*inv_freq[i] (if a frequency table is given), the
// pair being (i, i+rot/2) (pairing 0: halves) or (2i, 2i+1) (pairing 1: neighbours); q goes
// back in place, k and v go to the cache.
// Reference: src/backend/cpu/kernels/rope.cpp:61-111; CUDA kernels/rope.cuh:333-393.
#define ROPE_WAVES 4
template <typename T>
__global__ __launch_bounds__(ROPE_WAVES * CELEG_WAVE) void qk_norm_rope_store_kernel(
    T* __restrict__ q, int ldq, const T* __restrict__ k, int ldk, const T* __restrict__ v, int ldv,
    const float* __restrict__ q_weight, const float* __restrict__ k_weight, float eps,
    const float* __restrict__ inv_freq, const float* __restrict__ cos_sin, int rotary_dim, int pairing,
    const int* __restrict__ positions,
    const int* __restrict__ token_slot, const int* __restrict__ table, int table_stride,
    T* __restrict__ k_pool, T* __restrict__ v_pool, int n_layers, int layer, int page_tokens,
    int q_heads, int kv_heads, int head_dim, int n_heads) {
    extern __shared__ float lds[];   // head_dim floats for each wavefront
    const int wave = threadIdx.x / CELEG_WAVE, lane = threadIdx.x % CELEG_WAVE;
    float* vals = lds + wave * head_dim;
    const int t = blockIdx.x;
    const int head = blockIdx.y * ROPE_WAVES + wave;     // a wavefront per head, no barrier between them
    if (head >= n_heads) return;
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
    // the wavefront's own part of LDS: its lanes only have to see each other's writes
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
    const int half = rotary_dim / 2;
    for (int d = lane; d < head_dim; d += CELEG_WAVE) {
        float y = vals[d];
        if (inv_freq && d < rotary_dim) {
            // the pair's number, and whether this value is the pair's first
            const int i = pairing ? d >> 1 : (d < half ? d : d - half);
            const bool first = pairing ? !(d & 1) : d < half;
            float c, s;
            if (cos_sin) {       // the table of celeg_rope_table: the same values, computed once
                const float* cs = cos_sin + (static_cast<size_t>(pos) * half + i) * 2;
                c = cs[0];
                s = cs[1];
            } else {
                const float angle = static_cast<float>(pos) * inv_freq[i];
                c = cosf(angle);
                s = sinf(angle);
            }
            const float a = pairing ? vals[2 * i] : vals[i], b = pairing ? vals[2 * i + 1] : vals[i + half];
            y = first ? a * c - b * s : b * c + a * s;
        }
        dst[d] = from_float<T>(y);
    }
}

// The same for head sizes 32, 64 and 128 with rotation over the whole head (or none) and
// the table of cosines and sines: LPH = head_dim / 4 lanes share a head, a lane holds 4
// neighbouring values, a wavefront 64 / LPH heads of one row.  The sum of squares is
// reduced inside the LPH lanes, and the rotation's partner (the value half a head away) sits
// in lane ^ (LPH / 2), so nothing goes through LDS.
template <typename T> struct Quad;
template <> struct Quad<float> {
    typedef float raw __attribute__((ext_vector_type(4)));
    static __device__ __forceinline__ void load(const float* p, float (&v)[4]) {
        const raw r = *reinterpret_cast<const raw*>(p);
        v[0] = r[0]; v[1] = r[1]; v[2] = r[2]; v[3] = r[3];
    }
    static __device__ __forceinline__ void store(float* p, const float (&v)[4]) {
        *reinterpret_cast<raw*>(p) = raw{v[0], v[1], v[2], v[3]};
    }
};
template <> struct Quad<bf16> {
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

// TOKENS rows a thread (rows blockIdx.x * TOKENS ..), everything they read asked for before
// anything is used: a row's chain of position -> page -> address is three trips to memory, and a
// thread that has one row only spends its time waiting for them (2,048 rows: 13.6 us a layer
// with one row a thread).
template <typename T, int LPH, int TOKENS>
__global__ __launch_bounds__(ROPE_WAVES * CELEG_WAVE) void qk_norm_rope_store_quad_kernel(
    T* __restrict__ q, int ldq, const T* __restrict__ k, int ldk, const T* __restrict__ v, int ldv,
    const float* __restrict__ q_weight, const float* __restrict__ k_weight, float eps,
    const float* __restrict__ cos_sin, const int* __restrict__ positions,
    const int* __restrict__ token_slot, const int* __restrict__ table, int table_stride,
    T* __restrict__ k_pool, T* __restrict__ v_pool, int n_layers, int layer, int page_tokens,
    int q_heads, int kv_heads, int n_heads, int n_tokens) {
    constexpr int HD = 4 * LPH, HPW = CELEG_WAVE / LPH, HALF = HD / 2;
    const int wave = threadIdx.x / CELEG_WAVE, lane = threadIdx.x % CELEG_WAVE;
    const int head_raw = (blockIdx.y * ROPE_WAVES + wave) * HPW + lane / LPH;
    const bool live_head = head_raw < n_heads;
    const int head = live_head ? head_raw : n_heads - 1;     // idle lanes repeat the last head
    const int l = lane % LPH, d0 = 4 * l;
    const bool is_q = head < q_heads;
    const bool is_k = !is_q && head < q_heads + kv_heads;
    const int kv_head = is_q ? 0 : (is_k ? head - q_heads : head - q_heads - kv_heads);
    const float* weight = is_q ? q_weight : (is_k ? k_weight : nullptr);
    float w[4] = {1.f, 1.f, 1.f, 1.f};
    if (weight) Quad<float>::load(weight + d0, w);
    const bool rotate = cos_sin && (is_q || is_k);

    int t[TOKENS], pos[TOKENS], page[TOKENS];
    float x[TOKENS][4], cs[TOKENS][8];
#pragma unroll
    for (int i = 0; i < TOKENS; ++i) {
        t[i] = min(static_cast<int>(blockIdx.x) * TOKENS + i, n_tokens - 1);     // past the end: the last row again (not stored)
        pos[i] = positions[t[i]];
    }
#pragma unroll
    for (int i = 0; i < TOKENS; ++i) {
        const T* src = is_q ? q + static_cast<size_t>(t[i]) * ldq + static_cast<size_t>(head) * HD
                            : (is_k ? k + static_cast<size_t>(t[i]) * ldk + static_cast<size_t>(kv_head) * HD
                                    : v + static_cast<size_t>(t[i]) * ldv + static_cast<size_t>(kv_head) * HD);
        Quad<T>::load(src + d0, x[i]);
        page[i] = 0;
        if (!is_q) page[i] = table[static_cast<size_t>(token_slot[t[i]]) * table_stride + pos[i] / page_tokens];
        if (rotate) {
            const float* c = cos_sin + (static_cast<size_t>(pos[i]) * HALF + (d0 % HALF)) * 2;
            float c0[4], c1[4];
            Quad<float>::load(c, c0);
            Quad<float>::load(c + 4, c1);
#pragma unroll
            for (int e = 0; e < 4; ++e) { cs[i][e] = c0[e]; cs[i][4 + e] = c1[e]; }
        }
    }
    // values: four rows that are neighbours in one page leave as one store of four a dimension
    // (the page holds a dimension's keys side by side) instead of sixteen of two bytes
    if (TOKENS == 4 && !is_q && !is_k) {
        const int slot0 = token_slot[t[0]];
        // a page whose size is a multiple of four holds positions 4n .. 4n+3 side by side, at an
        // address the store of four may take; any other page size goes row by row
        bool together = static_cast<int>(blockIdx.x) * TOKENS + 3 < n_tokens && (pos[0] & 3) == 0 &&
                        (page_tokens & 3) == 0;
#pragma unroll
        for (int i = 1; i < TOKENS; ++i) together = together && pos[i] == pos[0] + i && token_slot[t[i]] == slot0;
        if (together) {
            if (!live_head) return;
            T* vdst = v_pool + cache_offset(page[0], n_layers, layer, kv_heads, kv_head, page_tokens, 0, HD) +
                      pos[0] % page_tokens;
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                const float four[4] = {x[0][e], x[1][e], x[2][e], x[3][e]};
                Quad<T>::store(vdst + static_cast<size_t>(d0 + e) * page_tokens, four);
            }
            return;
        }
    }
#pragma unroll
    for (int i = 0; i < TOKENS; ++i) {
        float sum = x[i][0] * x[i][0] + x[i][1] * x[i][1] + x[i][2] * x[i][2] + x[i][3] * x[i][3];
#pragma unroll
        for (int off = LPH / 2; off > 0; off >>= 1) sum += __shfl_xor(sum, off, CELEG_WAVE);
        if (weight) {
            const float inv = 1.0f / sqrtf(sum / static_cast<float>(HD) + eps);
#pragma unroll
            for (int e = 0; e < 4; ++e) x[i][e] = x[i][e] * inv * w[e];
        }
        float y[4];
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            const float other = __shfl_xor(x[i][e], LPH / 2, CELEG_WAVE);
            // first half: a c - b s with b the partner; second half: b c + a s with a the partner
            y[e] = rotate ? (l < LPH / 2 ? x[i][e] * cs[i][2 * e] - other * cs[i][2 * e + 1]
                                         : x[i][e] * cs[i][2 * e] + other * cs[i][2 * e + 1])
                          : x[i][e];
        }
        if (!live_head || static_cast<int>(blockIdx.x) * TOKENS + i >= n_tokens) continue;
        if (is_q) {
            Quad<T>::store(q + static_cast<size_t>(t[i]) * ldq + static_cast<size_t>(head) * HD + d0, y);
        } else if (is_k) {
            Quad<T>::store(k_pool + cache_offset(page[i], n_layers, layer, kv_heads, kv_head, page_tokens,
                                                 pos[i] % page_tokens, HD) + d0, y);
        } else {                               // v: copy, transposed inside the page
            T* vdst = v_pool + cache_offset(page[i], n_layers, layer, kv_heads, kv_head, page_tokens, 0, HD) +
                      pos[i] % page_tokens;
#pragma unroll
            for (int e = 0; e < 4; ++e) vdst[static_cast<size_t>(d0 + e) * page_tokens] = from_float<T>(x[i][e]);
        }
    }
}

template <typename T, int LPH>
static int launch_rope_quad(T* q, int ldq, const T* k, int ldk, const T* v, int ldv,
                            const float* q_weight, const float* k_weight, float eps,
                            const float* cos_sin, const int* positions, const int* token_slot,
                            const int* table, int table_stride, T* k_pool, T* v_pool, int n_layers,
                            int layer, int page_tokens, int n_tokens, int q_heads, int kv_heads,
                            int n_heads, hipStream_t stream) {
    const int per_block = ROPE_WAVES * (CELEG_WAVE / LPH);
    const unsigned head_blocks = (n_heads + per_block - 1) / per_block;
    // four rows a thread once there are enough of them to fill the chip that way
    if (static_cast<long long>(n_tokens) * head_blocks >= 4 * 1024) {
        hipLaunchKernelGGL((qk_norm_rope_store_quad_kernel<T, LPH, 4>), dim3((n_tokens + 3) / 4, head_blocks),
                           dim3(ROPE_WAVES * CELEG_WAVE), 0, stream, q, ldq, k, ldk, v, ldv, q_weight, k_weight, eps,
                           cos_sin, positions, token_slot, table, table_stride, k_pool, v_pool, n_layers, layer,
                           page_tokens, q_heads, kv_heads, n_heads, n_tokens);
    } else {
        hipLaunchKernelGGL((qk_norm_rope_store_quad_kernel<T, LPH, 1>), dim3(n_tokens, head_blocks),
                           dim3(ROPE_WAVES * CELEG_WAVE), 0, stream, q, ldq, k, ldk, v, ldv, q_weight, k_weight, eps,
                           cos_sin, positions, token_slot, table, table_stride, k_pool, v_pool, n_layers, layer,
                           page_tokens, q_heads, kv_heads, n_heads, n_tokens);
    }
    return CELEG_LAUNCH_RESULT();
}

template <typename T>
static int rope_quad_dispatch(void* q, int ldq, const void* k, int ldk, const void* v, int ldv,
                              const float* q_weight, const float* k_weight, float eps,
                              const float* cos_sin, const int* positions, const int* token_slot,
                              const int* table, int table_stride, void* k_pool, void* v_pool,
                              int n_layers, int layer, int page_tokens, int n_tokens, int q_heads,
                              int kv_heads, int head_dim, int n_heads, hipStream_t stream) {
#define CELEG_ROPE_QUAD(LPH_)                                                                     \
    return launch_rope_quad<T, LPH_>(static_cast<T*>(q), ldq, static_cast<const T*>(k), ldk,      \
                                     static_cast<const T*>(v), ldv, q_weight, k_weight, eps,      \
                                     cos_sin, positions, token_slot, table, table_stride,         \
                                     static_cast<T*>(k_pool), static_cast<T*>(v_pool), n_layers,  \
                                     layer, page_tokens, n_tokens, q_heads, kv_heads, n_heads, stream)
    if (head_dim == 32) { CELEG_ROPE_QUAD(8); }
    if (head_dim == 64) { CELEG_ROPE_QUAD(16); }
    CELEG_ROPE_QUAD(32);
#undef CELEG_ROPE_QUAD
}

// cos and sin of position * inv_freq[i] for positions 0 .. n_positions-1, interleaved:
// out[(pos * half + i) * 2 + {0, 1}].  The angle is the 32-bit product of the position and
// the frequency, as in the kernel above when it has no table.
__global__ void rope_table_kernel(const float* __restrict__ inv_freq, int half, int n_positions,
                                  float* __restrict__ out) {
    const size_t idx = static_cast<size_t>(blockIdx.x) * blockDim.x + threadIdx.x;
    if (idx >= static_cast<size_t>(n_positions) * half) return;
    const int pos = static_cast<int>(idx / half), i = static_cast<int>(idx % half);
    const float angle = static_cast<float>(pos) * inv_freq[i];
    out[2 * idx] = cosf(angle);
    out[2 * idx + 1] = sinf(angle);
}

extern "C" int celeg_rope_table(const float* inv_freq, int half, int n_positions, float* out,
                                hipStream_t stream) {
    if (half <= 0 || n_positions <= 0) return 0;
    const size_t total = static_cast<size_t>(n_positions) * half;
    hipLaunchKernelGGL(rope_table_kernel, dim3(static_cast<unsigned>((total + 255) / 256)), dim3(256), 0,
                       stream, inv_freq, half, n_positions, out);
    return CELEG_LAUNCH_RESULT();
}

// cos_sin: the table of celeg_rope_table covering every position of the step, or null.
extern "C" int celeg_qk_norm_rope_store(
    void* q, int ldq, const void* k, int ldk, const void* v, int ldv, int dtype,
    const float* q_weight, const float* k_weight, float eps, const float* inv_freq,
    const float* cos_sin, int rotary_dim, int pairing, const int* positions, const int* token_slot, const int* table,
    int table_stride, void* k_pool, void* v_pool, int n_layers, int layer, int page_tokens,
    int n_tokens, int q_heads, int kv_heads, int head_dim, int store_kv, hipStream_t stream) {
    if (n_tokens <= 0) return 0;
    if (pairing != 0 && pairing != 1) return static_cast<int>(hipErrorInvalidValue);
    const int n_heads = q_heads + (store_kv ? 2 * kv_heads : 0);
    const auto aligned = [](const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15) == 0; };
    const bool whole_rotation = !inv_freq || (cos_sin && rotary_dim == head_dim && pairing == 0);
    if ((head_dim == 32 || head_dim == 64 || head_dim == 128) && whole_rotation && ldq % 4 == 0 &&
        (!store_kv || (ldk % 4 == 0 && ldv % 4 == 0 && aligned(k) && aligned(v))) && aligned(q) &&
        aligned(k_pool) && aligned(v_pool) && (!q_weight || aligned(q_weight)) && (!k_weight || aligned(k_weight)) &&
        (!cos_sin || aligned(cos_sin))) {
        const float* cs = inv_freq ? cos_sin : nullptr;
        if (dtype == CELEG_F32)
            return rope_quad_dispatch<float>(q, ldq, k, ldk, v, ldv, q_weight, k_weight, eps, cs,
                                             positions, token_slot, table, table_stride, k_pool, v_pool,
                                             n_layers, layer, page_tokens, n_tokens, q_heads, kv_heads,
                                             head_dim, n_heads, stream);
        return rope_quad_dispatch<bf16>(q, ldq, k, ldk, v, ldv, q_weight, k_weight, eps, cs, positions,
                                        token_slot, table, table_stride, k_pool, v_pool, n_layers,
                                        layer, page_tokens, n_tokens, q_heads, kv_heads, head_dim,
                                        n_heads, stream);
    }
    dim3 grid(n_tokens, (n_heads + ROPE_WAVES - 1) / ROPE_WAVES), block(ROPE_WAVES * CELEG_WAVE);
    const size_t lds = static_cast<size_t>(ROPE_WAVES) * head_dim * sizeof(float);
    if (dtype == CELEG_F32)
        hipLaunchKernelGGL(qk_norm_rope_store_kernel<float>, grid, block, lds, stream,
                           static_cast<float*>(q), ldq, static_cast<const float*>(k), ldk,
                           static_cast<const float*>(v), ldv, q_weight, k_weight, eps, inv_freq,
                           cos_sin, rotary_dim, pairing, positions, token_slot, table, table_stride,
                           static_cast<float*>(k_pool), static_cast<float*>(v_pool), n_layers,
                           layer, page_tokens, q_heads, kv_heads, head_dim, n_heads);
    else
        hipLaunchKernelGGL(qk_norm_rope_store_kernel<bf16>, grid, block, lds, stream,
                           static_cast<bf16*>(q), ldq, static_cast<const bf16*>(k), ldk,
                           static_cast<const bf16*>(v), ldv, q_weight, k_weight, eps, inv_freq,
                           cos_sin, rotary_dim, pairing, positions, token_slot, table, table_stride,
                           static_cast<bf16*>(k_pool), static_cast<bf16*>(v_pool), n_layers,
                           layer, page_tokens, q_heads, kv_heads, head_dim, n_heads);
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
