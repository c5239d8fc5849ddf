// bfloat16 attention over the paged cache for gfx950: an MFMA kernel for the rows of
// prompt portions (and mixed batches), and a split-key kernel for batches in which
// every request brings one row (decode).
//
// Cache layout of a group (one page id covers all layers of the group):
//   K [pages, layers, kv_heads, page_tokens, head_dim]   one key after the other
//   V [pages, layers, kv_heads, head_dim, page_tokens]   transposed inside the page
// K rows feed the MFMA of q.k directly (head_dim runs along the instruction's k), and
// the transposed V feeds the MFMA of p.v directly (keys run along its k), so neither
// operand is shuffled through LDS.
//
// Scores are (q.k)*scale, causal (key position <= row position) and, with a window w,
// key position > row position - w.  Softmax statistics and accumulators are 32-bit; the
// probabilities enter the second product rounded to bfloat16.
// Reference semantics: src/backend/cpu/attention/paged_attention.cpp:229-283; tiled CUDA
// form src/backend/cuda/kernels/attention_gemm.cuh:15-200; split-key CUDA form
// src/backend/cuda/kernels/attention_paged.cuh:287-487.
#include "common.h"

typedef short bf16x4_t __attribute__((ext_vector_type(4)));
typedef float floatx4_t __attribute__((ext_vector_type(4)));

__device__ __forceinline__ size_t kv_block(int page, int n_layers, int layer, int kv_heads,
                                           int head, int page_tokens, int head_dim) {
    return ((static_cast<size_t>(page) * n_layers + layer) * kv_heads + head) *
           static_cast<size_t>(page_tokens) * head_dim;
}

__device__ __forceinline__ short bf16_bits(float x) { return static_cast<short>(from_float<bf16>(x).bits); }

// ================================================================ rows of portions
// One workgroup of 4 wavefronts per (tile of 64 rows of one request, query head); a
// wavefront owns 16 rows.  Per 64 keys: S^T = K Q^T (16x16x16 MFMA: A = 16 keys x 16
// dims, B = 16 dims x 16 rows), online softmax per row (a row is a lane column), then
// O^T += V^T P^T (A = 16 dims x 16 keys from the transposed V, B = P^T straight from the
// accumulator registers of S^T).  The request's page ids are put into LDS once; the keys
// of the next 64 are asked for while the current 64 are worked on, and the values of the
// current 64 before its scores are computed.
template <int HD>
__global__ __launch_bounds__(256) void attention_rows_kernel(
    const bf16* __restrict__ q, int ldq, const bf16* __restrict__ k_pool,
    const bf16* __restrict__ v_pool, const int* __restrict__ table, int table_stride,
    const int* __restrict__ cu_seqlens, const int* __restrict__ seq_slot,
    const int* __restrict__ seq_start, int n_seqs, bf16* __restrict__ out, int ldo, int q_heads,
    int kv_heads, int page_tokens, int page_shift, int n_layers, int layer, float scale_log2e,
    int window) {
    constexpr int DQ = HD / 4;   // dims a lane quad covers in q.k
    constexpr int KS = DQ / 4;   // MFMA steps along head_dim
    constexpr int DT = HD / 16;  // 16-dim tiles of the output
    extern __shared__ int spages[];   // table_stride page ids
    int tile = blockIdx.x;
    const int h = blockIdx.y;
    int s = 0, len = 0;
    bool found = false;
    for (; s < n_seqs; ++s) {
        len = cu_seqlens[s + 1] - cu_seqlens[s];
        const int tiles = (len + 63) >> 6;
        if (tile < tiles) { found = true; break; }
        tile -= tiles;
    }
    if (!found) return;   // the whole workgroup
    const int start = seq_start[s];
    {
        // pages up to the last key this tile of rows can see
        const int last_key = start + min(tile * 64 + 63, len - 1);
        const int* __restrict__ pages = table + static_cast<size_t>(seq_slot[s]) * table_stride;
        for (int i = threadIdx.x; i <= last_key >> page_shift; i += 256) spages[i] = pages[i];
    }
    __syncthreads();
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
    const int c = lane & 15, qd = lane >> 4;
    const int wrow0 = tile * 64 + wave * 16;
    if (wrow0 >= len) return;  // no row of this wavefront exists (no barrier is used below)
    const int row = wrow0 + c;
    const bool row_valid = row < len;
    const int row_c = row_valid ? row : len - 1;
    const int pq = start + row_c;                       // this lane's row position
    const int lo_q = window > 0 ? max(0, pq - window + 1) : 0;
    const int kmax = start + min(wrow0 + 15, len - 1);  // last key any row of the wavefront sees
    const int kmin = window > 0 ? max(0, start + wrow0 - window + 1) : 0;
    const int kvh = h / (q_heads / kv_heads);
    const size_t row_base = static_cast<size_t>(cu_seqlens[s]);
    const size_t head_block = static_cast<size_t>(page_tokens) * HD;
    const size_t page_stride = static_cast<size_t>(n_layers) * kv_heads * head_block;
    const size_t layer_head = (static_cast<size_t>(layer) * kv_heads + kvh) * head_block;

    bf16x4_t qreg[KS];
    {
        const bf16* qrow = q + (row_base + row_c) * ldq + static_cast<size_t>(h) * HD + qd * DQ;
#pragma unroll
        for (int st = 0; st < KS; ++st) qreg[st] = *reinterpret_cast<const bf16x4_t*>(qrow + st * 4);
    }
    floatx4_t oacc[DT];
#pragma unroll
    for (int dt = 0; dt < DT; ++dt) oacc[dt] = floatx4_t{0.f, 0.f, 0.f, 0.f};
    float m = -INFINITY, l = 0.f;

    // A tile of 16 keys lies in one page (page_tokens is a multiple of 16), so its page id
    // is the same for every lane: it is read once into a scalar, and a lane's own offset
    // inside the tile never changes.  Tiles beyond the last key are read from the last
    // key's page (any place there is allocated memory) and masked.
    const int last_page = kmax >> page_shift;
    const size_t k_lane = static_cast<size_t>(c) * HD + qd * DQ;
    const size_t v_lane = static_cast<size_t>(c) * page_tokens + 4 * qd;
    auto load_keys = [&](int kb, bf16x4_t (&dst)[4][KS]) {
#pragma unroll
        for (int kt = 0; kt < 4; ++kt) {
            const int key0 = kb + kt * 16;
            const int page = __builtin_amdgcn_readfirstlane(spages[min(key0 >> page_shift, last_page)]);
            const bf16* kp = k_pool + static_cast<size_t>(page) * page_stride + layer_head +
                             static_cast<size_t>(key0 & (page_tokens - 1)) * HD + k_lane;
#pragma unroll
            for (int st = 0; st < KS; ++st) dst[kt][st] = *reinterpret_cast<const bf16x4_t*>(kp + st * 4);
        }
    };
    const float neg_inf = -INFINITY;
    auto round64 = [&](int kb, bf16x4_t (&kcur)[4][KS], bf16x4_t (&knxt)[4][KS]) {
        // values of this round: lane (dim c of tile dt, quad qd) reads 4 keys' values
        bf16x4_t vreg[4][DT];
#pragma unroll
        for (int kt = 0; kt < 4; ++kt) {
            const int key0 = kb + kt * 16;
            const int page = __builtin_amdgcn_readfirstlane(spages[min(key0 >> page_shift, last_page)]);
            const bf16* vp = v_pool + static_cast<size_t>(page) * page_stride + layer_head +
                             (key0 & (page_tokens - 1)) + v_lane;
#pragma unroll
            for (int dt = 0; dt < DT; ++dt)
                vreg[kt][dt] = *reinterpret_cast<const bf16x4_t*>(vp + static_cast<size_t>(dt) * 16 * page_tokens);
        }
        if (kb + 64 <= kmax) load_keys(kb + 64, knxt);

        floatx4_t sacc[4];
#pragma unroll
        for (int kt = 0; kt < 4; ++kt) {
            sacc[kt] = floatx4_t{0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int st = 0; st < KS; ++st)
                sacc[kt] = __builtin_amdgcn_mfma_f32_16x16x16bf16_1k(kcur[kt][st], qreg[st], sacc[kt], 0, 0, 0);
        }
        // sacc[kt][r] = (key kb + 16 kt + 4 qd + r) . (row c); rounds that lie wholly inside
        // every row's range need no mask
        const bool full = kb + 63 <= start + wrow0 && (window <= 0 || kb >= start + min(wrow0 + 15, len - 1) - window + 1);
        float mx = neg_inf;
        if (full) {
#pragma unroll
            for (int kt = 0; kt < 4; ++kt)
#pragma unroll
                for (int r = 0; r < 4; ++r) mx = fmaxf(mx, sacc[kt][r]);
        } else {
#pragma unroll
            for (int kt = 0; kt < 4; ++kt)
#pragma unroll
                for (int r = 0; r < 4; ++r) {
                    const int key = kb + kt * 16 + 4 * qd + r;
                    const float sv = (key <= pq && key >= lo_q) ? sacc[kt][r] : neg_inf;
                    sacc[kt][r] = sv;
                    mx = fmaxf(mx, sv);
                }
        }
        mx = fmaxf(mx, __shfl_xor(mx, 16, 64));
        mx = fmaxf(mx, __shfl_xor(mx, 32, 64));
        const float m_new = fmaxf(m, mx * scale_log2e);          // the scale is positive
        const float m_use = m_new == neg_inf ? 0.f : m_new;      // a row that has seen no key yet
        const float alpha = __builtin_amdgcn_exp2f(m - m_use);
        float psum = 0.f;
#pragma unroll
        for (int kt = 0; kt < 4; ++kt)
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                const float p = __builtin_amdgcn_exp2f(fmaf(sacc[kt][r], scale_log2e, -m_use));
                sacc[kt][r] = p;
                psum += p;
            }
        l = l * alpha + psum;
        m = m_new;
#pragma unroll
        for (int dt = 0; dt < DT; ++dt) oacc[dt] *= alpha;
#pragma unroll
        for (int kt = 0; kt < 4; ++kt) {
            const bf16x4_t pb = {bf16_bits(sacc[kt][0]), bf16_bits(sacc[kt][1]),
                                 bf16_bits(sacc[kt][2]), bf16_bits(sacc[kt][3])};
#pragma unroll
            for (int dt = 0; dt < DT; ++dt)
                oacc[dt] = __builtin_amdgcn_mfma_f32_16x16x16bf16_1k(vreg[kt][dt], pb, oacc[dt], 0, 0, 0);
        }
    };
    // two sets of key registers take turns: one is multiplied while the other is filled
    bf16x4_t kreg_a[4][KS], kreg_b[4][KS];
    int kb = (kmin >> 6) << 6;
    load_keys(kb, kreg_a);
    while (kb <= kmax) {
        round64(kb, kreg_a, kreg_b);
        kb += 64;
        if (kb > kmax) break;
        round64(kb, kreg_b, kreg_a);
        kb += 64;
    }
    l += __shfl_xor(l, 16, 64);
    l += __shfl_xor(l, 32, 64);
    if (!row_valid) return;
    const float inv_l = 1.0f / l;
    bf16* orow = out + (row_base + row) * ldo + static_cast<size_t>(h) * HD + 4 * qd;
#pragma unroll
    for (int dt = 0; dt < DT; ++dt) {
        const bf16x4_t o = {bf16_bits(oacc[dt][0] * inv_l), bf16_bits(oacc[dt][1] * inv_l),
                            bf16_bits(oacc[dt][2] * inv_l), bf16_bits(oacc[dt][3] * inv_l)};
        *reinterpret_cast<bf16x4_t*>(orow + dt * 16) = o;
    }
}

extern "C" int celeg_attention_rows_bf16(
    const void* q, int ldq, const void* k_pool, const void* v_pool, const int* table,
    int table_stride, const int* cu_seqlens, const int* seq_slot, const int* seq_start,
    int n_seqs, int n_tokens, void* out, int ldo, int q_heads, int kv_heads, int head_dim,
    int page_tokens, int n_layers, int layer, float scale, int window, hipStream_t stream) {
    if (n_tokens <= 0 || n_seqs <= 0) return 0;
    if (page_tokens < 16 || (page_tokens & (page_tokens - 1)) || q_heads % kv_heads || (ldq % 4) ||
        (ldo % 4) || table_stride > 15360)
        return static_cast<int>(hipErrorInvalidValue);
    const int page_shift = __builtin_ctz(page_tokens);
    const int max_tiles = n_tokens / 64 + n_seqs;  // >= sum over requests of ceil(rows / 64)
    dim3 grid(max_tiles, q_heads), block(256);
    const size_t lds = static_cast<size_t>(table_stride) * sizeof(int);
    const float scale_log2e = scale * 1.4426950408889634f;
#define CELEG_ROWS(HD_)                                                                          \
    hipLaunchKernelGGL(attention_rows_kernel<HD_>, grid, block, lds, stream,                     \
                       static_cast<const bf16*>(q), ldq, static_cast<const bf16*>(k_pool),       \
                       static_cast<const bf16*>(v_pool), table, table_stride, cu_seqlens,        \
                       seq_slot, seq_start, n_seqs, static_cast<bf16*>(out), ldo, q_heads,       \
                       kv_heads, page_tokens, page_shift, n_layers, layer, scale_log2e, window)
    switch (head_dim) {
        case 32: CELEG_ROWS(32); break;
        case 64: CELEG_ROWS(64); break;
        case 96: CELEG_ROWS(96); break;
        case 128: CELEG_ROWS(128); break;
        default: return static_cast<int>(hipErrorInvalidValue);
    }
#undef CELEG_ROWS
    return CELEG_LAUNCH_RESULT();
}

// ================================================================ one row per request
// One wavefront per (64 keys, GH query heads that share a key/value head, request): all
// its loads (the page ids, then the 64 keys and the 64 values) are in flight before
// anything is computed.  For q.k a lane owns (key j, an eighth of head_dim) and eight
// lanes add up a score; for p.v a lane owns a dimension and reads its row of the
// transposed V.  Partial (max, sum, accumulator) go to a workspace and a second kernel
// joins the ranges of 64 keys.
#define DEC_KEYS 64

template <int HD, int GH>
__global__ __launch_bounds__(64) void attention_decode_kernel(
    const bf16* __restrict__ q, int ldq, const bf16* __restrict__ k_pool,
    const bf16* __restrict__ v_pool, const int* __restrict__ table, int table_stride,
    const int* __restrict__ token_slot, const int* __restrict__ positions,
    float* __restrict__ ws_o, float* __restrict__ ws_ml, int n_splits,
    int q_heads, int kv_heads, int page_tokens, int page_shift, int n_layers, int layer, float scale,
    int window) {
    constexpr int DL = HD / 8;    // dims of a key a lane multiplies
    constexpr int DD = HD / 64;   // output dims a lane accumulates
    __shared__ float ps[GH][DEC_KEYS];
    const int split = blockIdx.x, hb = blockIdx.y, t = blockIdx.z;
    const int lane = threadIdx.x;
    const int pos = positions[t];
    const int lo = window > 0 ? max(0, pos - window + 1) : 0;
    const int kb = split * DEC_KEYS;
    const int k_lo = max(lo, kb);
    const int k_hi = min(pos, kb + DEC_KEYS - 1);
    if (k_lo > k_hi) return;
    const int h0 = hb * GH;
    const int kvh = h0 / (q_heads / kv_heads);
    const int j8 = lane >> 3, seg = lane & 7;
    const int* __restrict__ pages = table + static_cast<size_t>(token_slot[t]) * table_stride;

    // page ids of the chunk: lane i holds the i-th page that the 64 keys touch
    const int first_page = kb >> page_shift;
    const int last_page = k_hi >> page_shift;
    const int my_page = pages[min(first_page + lane, last_page)];

    // keys: 8 rounds of 8 keys, a lane reads DL values of its key
    uint4 kraw[8][DL / 8];
#pragma unroll
    for (int it = 0; it < 8; ++it) {
        const int keyc = min(max(kb + it * 8 + j8, k_lo), k_hi);
        const int page = __shfl(my_page, (keyc >> page_shift) - first_page, 64);
        const bf16* kp = k_pool + kv_block(page, n_layers, layer, kv_heads, kvh, page_tokens, HD) +
                         static_cast<size_t>(keyc & (page_tokens - 1)) * HD + seg * DL;
#pragma unroll
        for (int v8 = 0; v8 < DL / 8; ++v8) kraw[it][v8] = *reinterpret_cast<const uint4*>(kp + v8 * 8);
    }
    // values: 4 groups of 16 keys, a lane reads the 16 values of its dimension(s)
    uint4 vraw[4][DD][2];
#pragma unroll
    for (int pg = 0; pg < 4; ++pg) {
        const int key0 = min(max(kb + pg * 16, k_lo & ~15), k_hi & ~15);   // a group inside the range
        const int page = __shfl(my_page, (key0 >> page_shift) - first_page, 64);
        const bf16* vbase = v_pool + kv_block(page, n_layers, layer, kv_heads, kvh, page_tokens, HD) +
                            (key0 & (page_tokens - 1));
#pragma unroll
        for (int dd = 0; dd < DD; ++dd)
#pragma unroll
            for (int v8 = 0; v8 < 2; ++v8)
                vraw[pg][dd][v8] = *reinterpret_cast<const uint4*>(
                    vbase + static_cast<size_t>(lane + 64 * dd) * page_tokens + v8 * 8);
    }
    float qf[GH][DL];
#pragma unroll
    for (int g = 0; g < GH; ++g) {
        const bf16* qrow = q + static_cast<size_t>(t) * ldq + static_cast<size_t>(h0 + g) * HD + seg * DL;
#pragma unroll
        for (int d = 0; d < DL; ++d) qf[g][d] = to_float(qrow[d]) * scale;
    }

    float sc[8][GH];
#pragma unroll
    for (int it = 0; it < 8; ++it) {
        const int key = kb + it * 8 + j8;
        const bool valid = key >= k_lo && key <= k_hi;
        float kf[DL];
#pragma unroll
        for (int v8 = 0; v8 < DL / 8; ++v8) {
            const uint32_t w[4] = {kraw[it][v8].x, kraw[it][v8].y, kraw[it][v8].z, kraw[it][v8].w};
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                kf[v8 * 8 + 2 * i] = __uint_as_float(w[i] << 16);
                kf[v8 * 8 + 2 * i + 1] = __uint_as_float(w[i] & 0xffff0000u);
            }
        }
#pragma unroll
        for (int g = 0; g < GH; ++g) {
            float dot = 0.f;
#pragma unroll
            for (int d = 0; d < DL; ++d) dot = fmaf(qf[g][d], kf[d], dot);
            dot += __shfl_xor(dot, 1, 64);
            dot += __shfl_xor(dot, 2, 64);
            dot += __shfl_xor(dot, 4, 64);
            sc[it][g] = valid ? dot : -INFINITY;
        }
    }
    float m[GH], l[GH];
#pragma unroll
    for (int g = 0; g < GH; ++g) {
        float mx = sc[0][g];
#pragma unroll
        for (int it = 1; it < 8; ++it) mx = fmaxf(mx, sc[it][g]);
        mx = fmaxf(mx, __shfl_xor(mx, 8, 64));
        mx = fmaxf(mx, __shfl_xor(mx, 16, 64));
        mx = fmaxf(mx, __shfl_xor(mx, 32, 64));   // finite: the chunk holds a key of the range
        float psum = 0.f;
#pragma unroll
        for (int it = 0; it < 8; ++it) {
            const float p = expf(sc[it][g] - mx);
            psum += p;
            if (seg == 0) ps[g][it * 8 + j8] = p;
        }
        psum += __shfl_xor(psum, 8, 64);    // the eight lanes of a key hold the same p:
        psum += __shfl_xor(psum, 16, 64);   // add over keys only
        psum += __shfl_xor(psum, 32, 64);
        m[g] = mx;
        l[g] = psum;
    }
    __syncthreads();
    float acc[GH][DD];
#pragma unroll
    for (int g = 0; g < GH; ++g)
#pragma unroll
        for (int dd = 0; dd < DD; ++dd) acc[g][dd] = 0.f;
#pragma unroll
    for (int pg = 0; pg < 4; ++pg) {
        // groups outside the range were redirected to one inside: their p are all zero
        const int key0 = kb + pg * 16;
        if (key0 > k_hi || key0 + 15 < k_lo) continue;
#pragma unroll
        for (int dd = 0; dd < DD; ++dd) {
            float vf[16];
#pragma unroll
            for (int v8 = 0; v8 < 2; ++v8) {
                const uint32_t w[4] = {vraw[pg][dd][v8].x, vraw[pg][dd][v8].y, vraw[pg][dd][v8].z,
                                       vraw[pg][dd][v8].w};
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    vf[v8 * 8 + 2 * i] = __uint_as_float(w[i] << 16);
                    vf[v8 * 8 + 2 * i + 1] = __uint_as_float(w[i] & 0xffff0000u);
                }
            }
#pragma unroll
            for (int g = 0; g < GH; ++g)
#pragma unroll
                for (int j = 0; j < 16; ++j) acc[g][dd] = fmaf(ps[g][pg * 16 + j], vf[j], acc[g][dd]);
        }
    }
#pragma unroll
    for (int g = 0; g < GH; ++g) {
        const size_t idx = (static_cast<size_t>(t) * q_heads + h0 + g) * n_splits + split;
        if (lane == 0) { ws_ml[2 * idx] = m[g]; ws_ml[2 * idx + 1] = l[g]; }
#pragma unroll
        for (int dd = 0; dd < DD; ++dd) ws_o[idx * HD + lane + 64 * dd] = acc[g][dd];
    }
}

// Joins the ranges of one (request, query head): out = sum_i e^(m_i - m) o_i / sum_i e^(m_i - m) l_i.
template <int HD>
__global__ __launch_bounds__(64) void attention_decode_reduce_kernel(
    const float* __restrict__ ws_o, const float* __restrict__ ws_ml,
    const int* __restrict__ positions, bf16* __restrict__ out, int ldo, int q_heads, int n_splits,
    int window) {
    const int h = blockIdx.x, t = blockIdx.y, lane = threadIdx.x;
    const int pos = positions[t];
    const int lo = window > 0 ? max(0, pos - window + 1) : 0;
    const int first = lo / DEC_KEYS, last = pos / DEC_KEYS;
    const size_t base = (static_cast<size_t>(t) * q_heads + h) * n_splits;
    float m = -INFINITY;
    for (int i0 = first; i0 <= last; i0 += 64) {
        const int i = i0 + lane;
        m = fmaxf(m, i <= last ? ws_ml[2 * (base + i)] : -INFINITY);
    }
    m = wave_max(m);
    float denom = 0.f, acc[HD / 64];
#pragma unroll
    for (int dd = 0; dd < HD / 64; ++dd) acc[dd] = 0.f;
    for (int i0 = first; i0 <= last; i0 += 64) {
        const int i = i0 + lane;
        float w = 0.f, wl = 0.f;
        if (i <= last) {
            w = expf(ws_ml[2 * (base + i)] - m);
            wl = w * ws_ml[2 * (base + i) + 1];
        }
        denom += wave_sum(wl);
        const int n = min(64, last - i0 + 1);
        for (int j0 = 0; j0 < n; j0 += 8) {     // eight ranges' accumulators are read side by side
            float o[8][HD / 64];
#pragma unroll
            for (int j = 0; j < 8; ++j)
#pragma unroll
                for (int dd = 0; dd < HD / 64; ++dd)
                    o[j][dd] = j0 + j < n ? ws_o[(base + i0 + j0 + j) * HD + lane + 64 * dd] : 0.f;
#pragma unroll
            for (int j = 0; j < 8; ++j) {
                const float wj = __shfl(w, min(j0 + j, 63), 64);
#pragma unroll
                for (int dd = 0; dd < HD / 64; ++dd) acc[dd] = fmaf(j0 + j < n ? wj : 0.f, o[j][dd], acc[dd]);
            }
        }
    }
    bf16* orow = out + static_cast<size_t>(t) * ldo + static_cast<size_t>(h) * HD;
#pragma unroll
    for (int dd = 0; dd < HD / 64; ++dd) orow[lane + 64 * dd] = from_float<bf16>(acc[dd] / denom);
}

// workspace: ws_o [rows, q_heads, n_splits, head_dim] and ws_ml [rows, q_heads, n_splits, 2]
// floats, n_splits = ceil(max_context / 64).
extern "C" int celeg_attention_decode_bf16(
    const void* q, int ldq, const void* k_pool, const void* v_pool, const int* table,
    int table_stride, const int* token_slot, const int* positions, float* ws_o, float* ws_ml,
    int n_splits, void* out, int ldo, int n_rows, int q_heads, int kv_heads,
    int head_dim, int page_tokens, int n_layers, int layer, float scale, int window,
    hipStream_t stream) {
    if (n_rows <= 0) return 0;
    const int group = q_heads / kv_heads;
    if (q_heads % kv_heads || page_tokens < 16 || (page_tokens & (page_tokens - 1)) || n_splits <= 0 ||
        (ldq % 8))
        return static_cast<int>(hipErrorInvalidValue);
    const int page_shift = __builtin_ctz(page_tokens);
    const int gh = (group % 4 == 0) ? 4 : ((group % 2 == 0) ? 2 : 1);
    dim3 grid(n_splits, q_heads / gh, n_rows), block(64);
#define CELEG_DEC(HD_, GH_)                                                                      \
    hipLaunchKernelGGL((attention_decode_kernel<HD_, GH_>), grid, block, 0, stream,              \
                       static_cast<const bf16*>(q), ldq, static_cast<const bf16*>(k_pool),       \
                       static_cast<const bf16*>(v_pool), table, table_stride, token_slot,        \
                       positions, ws_o, ws_ml, n_splits, q_heads, kv_heads,                      \
                       page_tokens, page_shift, n_layers, layer, scale, window)
#define CELEG_DEC_HD(HD_)                                                                        \
    if (gh == 4) CELEG_DEC(HD_, 4); else if (gh == 2) CELEG_DEC(HD_, 2); else CELEG_DEC(HD_, 1);  \
    hipLaunchKernelGGL(attention_decode_reduce_kernel<HD_>, dim3(q_heads, n_rows), dim3(64), 0,  \
                       stream, ws_o, ws_ml, positions, static_cast<bf16*>(out), ldo, q_heads,    \
                       n_splits, window)
    if (head_dim == 64) { CELEG_DEC_HD(64); }
    else if (head_dim == 128) { CELEG_DEC_HD(128); }
    else return static_cast<int>(hipErrorInvalidValue);
#undef CELEG_DEC_HD
#undef CELEG_DEC
    return CELEG_LAUNCH_RESULT();
}
