// Sampling on the device: penalised argmax, and temperature / top-k / top-p sampling,
// one workgroup per row of logits.  Semantics follow the reference's CPU sampler
// (src/backend/cpu/sampler.cpp:26-101): repetition penalty v >= 0 ? v/p : v*p on seen
// tokens if p > 1; greedy = first (lowest) index of the maximum; otherwise
// score = penalised / temperature, the top_k by (score desc, id asc), p = exp(score -
// max) / sum, the shortest prefix whose mass reaches top_p, and a walk down the list
// with the uniform draw u that the host hands in (its xorshift64* state lives on the
// host, one per request).  top_k <= 128 as in the reference
// (include/celeg/model/runtime_types.hpp:37).
#include "common.h"

#define SAMPLE_THREADS 1024
#define SAMPLE_MAX_K 128
typedef float floatx4_t __attribute__((ext_vector_type(4)));

__device__ __forceinline__ float penalised_logit(const float* __restrict__ row,
                                                 const uint8_t* __restrict__ seen, float penalty,
                                                 int i) {
    float v = row[i];
    if (seen && penalty > 1.0f && seen[i]) v = v >= 0.0f ? v / penalty : v * penalty;
    return v;
}

// larger float <-> larger key
__device__ __forceinline__ uint32_t order_key(float f) {
    const uint32_t u = __float_as_uint(f);
    return (u & 0x80000000u) ? ~u : (u | 0x80000000u);
}

__device__ __forceinline__ bool better(float sa, int ia, float sb, int ib) {
    return sa == sb ? ia < ib : sa > sb;
}

// fparams[row] = {temperature, top_p, penalty, u}; iparams[row] = {top_k, seen_row or -1,
// slot or -1}; the token also goes to last_tokens[slot] (if given and slot >= 0), where the
// next step can take it from without the host in between.
__global__ __launch_bounds__(SAMPLE_THREADS) void sample_kernel(
    const float* __restrict__ logits, int ld, int vocab, const float* __restrict__ fparams,
    const int* __restrict__ iparams, const uint8_t* __restrict__ seen_all, size_t seen_stride,
    int* __restrict__ out_tokens, int* __restrict__ last_tokens) {
    __shared__ float s_val[SAMPLE_THREADS / CELEG_WAVE];
    __shared__ int s_idx[SAMPLE_THREADS / CELEG_WAVE];
    __shared__ unsigned int hist[256];
    __shared__ unsigned int sel[3];       // prefix, remaining, (unused)
    __shared__ int wave_gt[SAMPLE_THREADS / CELEG_WAVE], wave_eq[SAMPLE_THREADS / CELEG_WAVE];
    __shared__ int running[2];
    __shared__ float cand_score[SAMPLE_MAX_K];
    __shared__ int cand_id[SAMPLE_MAX_K];

    const int r = blockIdx.x;
    const int tid = threadIdx.x;
    const int lane = tid & (CELEG_WAVE - 1), wave = tid / CELEG_WAVE;
    const int n_waves = SAMPLE_THREADS / CELEG_WAVE;
    const float* row = logits + static_cast<size_t>(r) * ld;
    const float temperature = fparams[4 * r + 0], top_p = fparams[4 * r + 1];
    const float penalty = fparams[4 * r + 2], u = fparams[4 * r + 3];
    int top_k = iparams[3 * r + 0];
    const int seen_row = iparams[3 * r + 1];
    const int slot = iparams[3 * r + 2];
    const uint8_t* seen = (seen_all && seen_row >= 0)
                              ? seen_all + static_cast<size_t>(seen_row) * seen_stride : nullptr;

    if (temperature <= 0.0f || top_k == 1) {
        // ---- penalised argmax, lowest index wins ties
        // Groups of 4 logits, 8 groups of a thread asked for before any is looked at (a
        // row of 65,536 logits is then two round trips to memory instead of 64).
        float best = -INFINITY;
        int best_i = 0x7fffffff;
        const bool pen = seen && penalty > 1.0f;
        const bool vec = (reinterpret_cast<uintptr_t>(row) & 15) == 0 &&
                         (!pen || (reinterpret_cast<uintptr_t>(seen) & 3) == 0);
        const int n4 = vec ? vocab >> 2 : 0;
        auto take = [&](float v, unsigned seen_byte, int i) {
            if (seen_byte) v = v >= 0.0f ? v / penalty : v * penalty;
            if (best_i == 0x7fffffff || v > best) { best = v; best_i = i; }
        };
        constexpr int UN = 8;
        for (int g0 = tid; g0 < n4; g0 += SAMPLE_THREADS * UN) {
            floatx4_t v[UN];
            unsigned sn[UN];
#pragma unroll
            for (int j = 0; j < UN; ++j) {
                const int g = min(g0 + j * SAMPLE_THREADS, n4 - 1);      // clamped, masked below
                v[j] = reinterpret_cast<const floatx4_t*>(row)[g];
                sn[j] = pen ? reinterpret_cast<const unsigned*>(seen)[g] : 0u;
            }
#pragma unroll
            for (int j = 0; j < UN; ++j) {
                const int g = g0 + j * SAMPLE_THREADS;
                if (g < n4) {
#pragma unroll
                    for (int e = 0; e < 4; ++e) take(v[j][e], (sn[j] >> (8 * e)) & 0xffu, 4 * g + e);
                }
            }
        }
        for (int i = 4 * n4 + tid; i < vocab; i += SAMPLE_THREADS)      // what the groups left
            take(row[i], pen ? seen[i] : 0u, i);
        for (int off = CELEG_WAVE / 2; off > 0; off >>= 1) {
            const float ov = __shfl_xor(best, off, CELEG_WAVE);
            const int oi = __shfl_xor(best_i, off, CELEG_WAVE);
            if (oi != 0x7fffffff && (best_i == 0x7fffffff || better(ov, oi, best, best_i))) {
                best = ov; best_i = oi;
            }
        }
        if (lane == 0) { s_val[wave] = best; s_idx[wave] = best_i; }
        __syncthreads();
        if (tid == 0) {
            for (int w = 1; w < n_waves; ++w)
                if (s_idx[w] != 0x7fffffff &&
                    (best_i == 0x7fffffff || better(s_val[w], s_idx[w], best, best_i))) {
                    best = s_val[w]; best_i = s_idx[w];
                }
            out_tokens[r] = best_i;
            if (last_tokens && slot >= 0) last_tokens[slot] = best_i;
        }
        return;
    }

    top_k = min(min(top_k, vocab), SAMPLE_MAX_K);
    // ---- radix select of the top_k-th largest score
    if (tid == 0) { sel[0] = 0u; sel[1] = static_cast<unsigned>(top_k); }
    unsigned int mask = 0u;
    for (int shift = 24; shift >= 0; shift -= 8) {
        if (tid < 256) hist[tid] = 0u;
        __syncthreads();
        const unsigned int prefix = sel[0];
        for (int i = tid; i < vocab; i += SAMPLE_THREADS) {
            const uint32_t key = order_key(penalised_logit(row, seen, penalty, i) / temperature);
            if ((key & mask) == prefix) atomicAdd(&hist[(key >> shift) & 255u], 1u);
        }
        __syncthreads();
        if (tid == 0) {
            unsigned int remaining = sel[1], above = 0u;
            int bin = 255;
            for (; bin > 0; --bin) {
                if (above + hist[bin] >= remaining) break;
                above += hist[bin];
            }
            sel[0] = prefix | (static_cast<unsigned>(bin) << shift);
            sel[1] = remaining - above;
        }
        mask |= 255u << shift;
        __syncthreads();
    }
    const uint32_t kth = sel[0];
    const int need_eq = static_cast<int>(sel[1]);  // how many of the ties at the threshold to take
    const int n_gt = top_k - need_eq;

    // ---- ordered compaction: all above the threshold, and the lowest-id ties
    if (tid == 0) { running[0] = 0; running[1] = 0; }
    __syncthreads();
    for (int base = 0; base < vocab; base += SAMPLE_THREADS) {
        const int i = base + tid;
        float score = 0.f;
        bool gt = false, eq = false;
        if (i < vocab) {
            score = penalised_logit(row, seen, penalty, i) / temperature;
            const uint32_t key = order_key(score);
            gt = key > kth;
            eq = key == kth;
        }
        const unsigned long long m_gt = __ballot(gt), m_eq = __ballot(eq);
        const unsigned long long below = lane == 0 ? 0ull : (~0ull >> (CELEG_WAVE - lane));
        const int p_gt = __popcll(m_gt & below), p_eq = __popcll(m_eq & below);
        if (lane == 0) { wave_gt[wave] = __popcll(m_gt); wave_eq[wave] = __popcll(m_eq); }
        __syncthreads();
        int off_gt = running[0], off_eq = running[1];
        for (int w = 0; w < wave; ++w) { off_gt += wave_gt[w]; off_eq += wave_eq[w]; }
        if (gt) {
            const int p = off_gt + p_gt;
            if (p < n_gt) { cand_score[p] = score; cand_id[p] = i; }
        } else if (eq) {
            const int e = off_eq + p_eq;
            if (e < need_eq) { cand_score[n_gt + e] = score; cand_id[n_gt + e] = i; }
        }
        __syncthreads();
        if (tid == 0) {
            int a = 0, b = 0;
            for (int w = 0; w < n_waves; ++w) { a += wave_gt[w]; b += wave_eq[w]; }
            running[0] += a; running[1] += b;
        }
        __syncthreads();
    }
    if (tid >= top_k && tid < SAMPLE_MAX_K) { cand_score[tid] = -INFINITY; cand_id[tid] = 0x7fffffff; }
    __syncthreads();

    // ---- bitonic sort of 128 candidates by (score desc, id asc)
    for (int size = 2; size <= SAMPLE_MAX_K; size <<= 1) {
        for (int stride = size >> 1; stride > 0; stride >>= 1) {
            if (tid < SAMPLE_MAX_K) {
                const int partner = tid ^ stride;
                if (partner > tid) {
                    const bool ascending_block = (tid & size) == 0;  // "best first" blocks
                    const float sa = cand_score[tid], sb = cand_score[partner];
                    const int ia = cand_id[tid], ib = cand_id[partner];
                    const bool a_first = better(sa, ia, sb, ib);
                    if (ascending_block ? !a_first : a_first) {
                        cand_score[tid] = sb; cand_id[tid] = ib;
                        cand_score[partner] = sa; cand_id[partner] = ia;
                    }
                }
            }
            __syncthreads();
        }
    }

    // ---- softmax, top-p prefix and the walk, sequentially as the reference does
    if (tid == 0) {
        const float maximum = cand_score[0];
        float total = 0.f;
        for (int i = 0; i < top_k; ++i) {
            cand_score[i] = expf(cand_score[i] - maximum);
            total += cand_score[i];
        }
        for (int i = 0; i < top_k; ++i) cand_score[i] /= total;
        int active = top_k;
        if (top_p < 1.0f) {
            float cumulative = 0.f;
            active = 0;
            do {
                cumulative += cand_score[active++];
            } while (active < top_k && cumulative < top_p);
            total = 0.f;
            for (int i = 0; i < active; ++i) total += cand_score[i];
        } else {
            total = 1.0f;
        }
        float target = u * total;
        int chosen = cand_id[active - 1];
        for (int i = 0; i < active; ++i) {
            target -= cand_score[i];
            if (target <= 0.0f) { chosen = cand_id[i]; break; }
        }
        out_tokens[r] = chosen;
        if (last_tokens && slot >= 0) last_tokens[slot] = chosen;
    }
}

extern "C" int celeg_sample(const float* logits, int ld, int rows, int vocab,
                            const float* fparams, const int* iparams, const uint8_t* seen,
                            size_t seen_stride, int* out_tokens, int* last_tokens,
                            hipStream_t stream) {
    if (rows <= 0) return 0;
    if (vocab <= 0) return static_cast<int>(hipErrorInvalidValue);
    hipLaunchKernelGGL(sample_kernel, dim3(rows), dim3(SAMPLE_THREADS), 0, stream, logits, ld,
                       vocab, fparams, iparams, seen, seen_stride, out_tokens, last_tokens);
    return CELEG_LAUNCH_RESULT();
}

// seen[slot[t], token[t]] = 1 for the rows of a step (prompt and generated tokens alike,
// reference kernels/sampling.cu:45-73)
__global__ void mark_seen_kernel(uint8_t* __restrict__ seen, size_t stride, int n_slots, int vocab,
                                 const int* __restrict__ tokens, const int* __restrict__ slots,
                                 int n) {
    const int i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= n) return;
    const int s = slots[i], t = tokens[i];
    if (s < 0 || s >= n_slots || t < 0 || t >= vocab) return;
    seen[static_cast<size_t>(s) * stride + t] = 1;
}

extern "C" int celeg_mark_seen(uint8_t* seen, size_t stride, int n_slots, int vocab,
                               const int* tokens, const int* slots, int n, hipStream_t stream) {
    if (n <= 0) return 0;
    hipLaunchKernelGGL(mark_seen_kernel, dim3((n + 255) / 256), dim3(256), 0, stream, seen, stride,
                       n_slots, vocab, tokens, slots, n);
    return CELEG_LAUNCH_RESULT();
}
