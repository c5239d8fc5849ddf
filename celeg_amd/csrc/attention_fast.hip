// bfloat16 attention over the paged cache for gfx950: an MFMA kernel for the rows of
// prompt portions (and mixed batches), and MFMA kernels for batches in which every request
// brings one row (decode): the query heads that share a key/value head are the rows.
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

typedef __bf16 bf16x4_t __attribute__((ext_vector_type(4)));
typedef __bf16 bf16x8_t __attribute__((ext_vector_type(8)));
typedef float floatx4_t __attribute__((ext_vector_type(4)));
// (arrays of HIP's own uint4 class are not always kept in registers; this type is)
typedef unsigned int u32x4_t __attribute__((ext_vector_type(4)));

__device__ __forceinline__ size_t kv_block(int page, int n_layers, int layer, int kv_heads,
                                           int head, int page_tokens, int head_dim) {
    return ((static_cast<size_t>(page) * n_layers + layer) * kv_heads + head) *
           static_cast<size_t>(page_tokens) * head_dim;
}

// Rows a workgroup of the portion kernel takes when the caller leaves the choice open.
#define CELEG_ROWS_DEFAULT(n_tokens, n_seqs) 64


// Combining a value with the one that lane ^ 16 (lane ^ 32) holds, by the lane-swap
// instructions of gfx950: both operands start as x; the swap leaves (row 0, row 0, row 2,
// row 2) in one and (row 1, row 1, row 3, row 3) in the other (rows of 16 lanes; halves of
// 32 lanes likewise), so the two results are the lane's own value and its partner's.
__device__ __forceinline__ float max_row16(float x) {
    const unsigned u = __float_as_uint(x);
    const auto r = __builtin_amdgcn_permlane16_swap(u, u, false, false);
    return fmaxf(__uint_as_float(r[0]), __uint_as_float(r[1]));
}
__device__ __forceinline__ float max_half32(float x) {
    const unsigned u = __float_as_uint(x);
    const auto r = __builtin_amdgcn_permlane32_swap(u, u, false, false);
    return fmaxf(__uint_as_float(r[0]), __uint_as_float(r[1]));
}
__device__ __forceinline__ float sum_row16(float x) {
    const unsigned u = __float_as_uint(x);
    const auto r = __builtin_amdgcn_permlane16_swap(u, u, false, false);
    return __uint_as_float(r[0]) + __uint_as_float(r[1]);
}
__device__ __forceinline__ float sum_half32(float x) {
    const unsigned u = __float_as_uint(x);
    const auto r = __builtin_amdgcn_permlane32_swap(u, u, false, false);
    return __uint_as_float(r[0]) + __uint_as_float(r[1]);
}

// ================================================================ rows of portions
// A tile is 64*RT rows of one request for one query head; 4 wavefronts work on it, each
// on RT tiles of 16 rows.  A workgroup of 8 wavefronts takes two tiles of a request, the
// i-th from the front and the i-th from the back: under the causal mask their key counts
// add up to the same for every pair, and the wavefronts are spread over the SIMDs so that
// each SIMD gets one of either tile.  The keys and values of 64 positions are staged in
// LDS once for the 4 wavefronts of a tile (two buffers: the next 64 are fetched into registers
// while the current 64 are worked on, and written to the other buffer before the one
// barrier of the round).  Per 64 keys: S^T = K Q^T (16x16x32 MFMA: A = 16 keys x 32 dims,
// B = 32 dims x 16 rows), online softmax per row (a row is a lane column), then
// O^T += V^T P^T (A = 16 dims x 32 keys from the transposed V, B = P^T straight from the
// accumulator registers of S^T).  The 16 keys of a score tile are chosen so that a lane
// ends up with the probabilities of 8 neighbouring keys, which is what one 16-byte read
// of the transposed V delivers.
template <int HD, int RT>
__global__ __launch_bounds__(512) void attention_rows_kernel(
    const bf16* __restrict__ q, int ldq, const bf16* __restrict__ k_pool,
    const bf16* __restrict__ v_pool, const int* __restrict__ table, int table_stride,
    const int* __restrict__ cu_seqlens, const int* __restrict__ seq_slot,
    const int* __restrict__ seq_start, int n_seqs, bf16* __restrict__ out, int ldo,
    int q_heads, int kv_heads, int page_tokens, int page_shift, int n_layers, int layer,
    float scale_log2e, int window) {
    constexpr int ROWS = 64 * RT;   // rows of a workgroup
    constexpr int WROWS = 16 * RT;  // rows of a wavefront
    constexpr int DQ = HD / 4;      // dims a lane quad covers in q.k
    constexpr int KS = DQ / 8;      // MFMA steps of 32 along head_dim
    constexpr int DT = HD / 16;     // 16-dim tiles of the output
    constexpr int KROW = HD + 8;    // LDS row of a key, padded against bank conflicts
    constexpr int VROW = 64 + 8;    // LDS row of a dimension: 64 keys, padded
    constexpr int CH = HD / 32;     // 16-byte pieces of K, and of V, a thread moves per round
    extern __shared__ int smem[];
    const int half = threadIdx.x >> 8, tid = threadIdx.x & 255;
    __bf16* const sK = reinterpret_cast<__bf16*>(smem) + half * (2 * 64 * KROW);       // [2][2][64][KROW]
    __bf16* const sV = reinterpret_cast<__bf16*>(smem) + 4 * 64 * KROW + half * (2 * HD * VROW);  // [2][2][HD][VROW]
    int* const spages = reinterpret_cast<int*>(reinterpret_cast<__bf16*>(smem) + 4 * 64 * KROW + 4 * HD * VROW);
    int pair = blockIdx.x;
    const int h = blockIdx.y;
    int s = 0, len = 0, tiles = 0;
    bool found = false;
    for (; s < n_seqs; ++s) {
        len = cu_seqlens[s + 1] - cu_seqlens[s];
        tiles = (len + ROWS - 1) / ROWS;
        if (pair < (tiles + 1) / 2) { found = true; break; }
        pair -= (tiles + 1) / 2;
    }
    if (!found) return;   // the whole workgroup
    const int start = seq_start[s];
    // first round and number of rounds of a tile of rows
    auto first_key = [&](int t) { return ((window > 0 ? max(0, start + t * ROWS - window + 1) : 0) >> 6) << 6; };
    auto last_key = [&](int t) { return start + min(t * ROWS + ROWS - 1, len - 1); };
    const int heavy = tiles - 1 - pair;
    const bool has_tile = half == 1 || pair != heavy;   // the middle tile of an odd count has no partner
    const int tile = half == 1 ? heavy : pair;
    const int rounds_heavy = ((last_key(heavy) - first_key(heavy)) >> 6) + 1;
    const int rounds_light = pair != heavy ? ((last_key(pair) - first_key(pair)) >> 6) + 1 : 0;
    const int n_rounds = max(rounds_heavy, rounds_light);
    const int my_rounds = half == 1 ? rounds_heavy : rounds_light;
    const int brow0 = tile * ROWS;
    const int bkmax = last_key(tile);             // last key this half sees
    const int last_page = bkmax >> page_shift;
    {
        const int* __restrict__ pages = table + static_cast<size_t>(seq_slot[s]) * table_stride;
        for (int i = threadIdx.x; i <= last_key(heavy) >> page_shift; i += 512) spages[i] = pages[i];
    }
    __syncthreads();
    const int wave = tid >> 6, lane = tid & 63;
    const int c = lane & 15, qd = lane >> 4;
    const int wrow0 = brow0 + wave * WROWS;
    const bool wave_active = has_tile && wrow0 < len;
    const int wkmax = start + min(wrow0 + WROWS - 1, len - 1);  // last key any row of the wavefront sees
    const int wkmin = window > 0 ? max(0, start + wrow0 - window + 1) : 0;
    const int kvh = h / (q_heads / kv_heads);
    const size_t row_base = static_cast<size_t>(cu_seqlens[s]);
    const size_t head_block = static_cast<size_t>(page_tokens) * HD;
    const size_t page_stride = static_cast<size_t>(n_layers) * kv_heads * head_block;
    const size_t layer_head = (static_cast<size_t>(layer) * kv_heads + kvh) * head_block;

    int pq[RT], lo_q[RT];
    bool row_valid[RT];
    bf16x8_t qreg[RT][KS];
    floatx4_t oacc[RT][DT];
    float m[RT], l[RT];
#pragma unroll
    for (int rt = 0; rt < RT; ++rt) {
        const int row = wrow0 + rt * 16 + c;
        row_valid[rt] = row < len;
        const int row_c = row_valid[rt] ? row : len - 1;
        pq[rt] = start + row_c;
        lo_q[rt] = window > 0 ? max(0, pq[rt] - window + 1) : 0;
        const bf16* qrow = q + (row_base + row_c) * ldq + static_cast<size_t>(h) * HD + qd * DQ;
#pragma unroll
        for (int st = 0; st < KS; ++st) qreg[rt][st] = *reinterpret_cast<const bf16x8_t*>(qrow + st * 8);
#pragma unroll
        for (int dt = 0; dt < DT; ++dt) oacc[rt][dt] = floatx4_t{0.f, 0.f, 0.f, 0.f};
        m[rt] = -INFINITY;
        l[rt] = 0.f;
    }

    // What a thread moves per round: piece i of K is 8 dims of one key; piece i of V is 8
    // keys of one dimension, walked page by page so that neighbouring threads read
    // neighbouring memory.  Positions beyond the last key are read from the last key's
    // page (allocated memory) and masked.
    const int pt_shift = min(page_shift, 6);          // keys of a page inside a round: 1 << pt_shift
    u32x4_t kstage[CH], vstage[CH];
    auto fetch = [&](int kb) __attribute__((always_inline)) {
#pragma unroll
        for (int j = 0; j < CH; ++j) {
            const int i = tid + 256 * j;
            {
                const int key = kb + i / (HD / 8), part = i % (HD / 8);
                const int page = spages[min(key >> page_shift, last_page)];
                kstage[j] = *reinterpret_cast<const u32x4_t*>(
                    k_pool + static_cast<size_t>(page) * page_stride + layer_head +
                    static_cast<size_t>(key & (page_tokens - 1)) * HD + part * 8);
            }
            {
                const int per_dim = 1 << (pt_shift - 3);           // pieces of a dimension inside a page
                const int piece = (i >> (pt_shift - 3)) / HD;      // which page of the round
                const int rem = i - piece * (HD << (pt_shift - 3));
                const int d = rem >> (pt_shift - 3), g = rem & (per_dim - 1);
                const int key0 = kb + (piece << pt_shift) + g * 8;
                const int page = spages[min(key0 >> page_shift, last_page)];
                vstage[j] = *reinterpret_cast<const u32x4_t*>(
                    v_pool + static_cast<size_t>(page) * page_stride + layer_head +
                    static_cast<size_t>(d) * page_tokens + (key0 & (page_tokens - 1)));
            }
        }
    };
    auto stage = [&](int buf) __attribute__((always_inline)) {
#pragma unroll
        for (int j = 0; j < CH; ++j) {
            const int i = tid + 256 * j;
            *reinterpret_cast<u32x4_t*>(sK + (buf * 64 + i / (HD / 8)) * KROW + (i % (HD / 8)) * 8) = kstage[j];
            const int per_dim = 1 << (pt_shift - 3);
            const int piece = (i >> (pt_shift - 3)) / HD;
            const int rem = i - piece * (HD << (pt_shift - 3));
            const int d = rem >> (pt_shift - 3), g = rem & (per_dim - 1);
            *reinterpret_cast<u32x4_t*>(sV + (buf * HD + d) * VROW + (piece << pt_shift) + g * 8) = vstage[j];
        }
    };
    const float neg_inf = -INFINITY;
    // score tile kt, A row i  <->  key 32 (kt/2) + 8 (i/4) + 4 (kt%2) + i%4 of the round, so
    // that accumulator register r of lane quad qd is key 32 (kt/2) + 8 qd + 4 (kt%2) + r
    auto compute = [&](int kb, int buf) __attribute__((always_inline)) {
        floatx4_t sacc[RT][4];
#pragma unroll
        for (int rt = 0; rt < RT; ++rt)
#pragma unroll
            for (int kt = 0; kt < 4; ++kt) sacc[rt][kt] = floatx4_t{0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int kt = 0; kt < 4; ++kt) {
            const int key_row = 32 * (kt >> 1) + 8 * (c >> 2) + 4 * (kt & 1) + (c & 3);
            const __bf16* kp = sK + (buf * 64 + key_row) * KROW + qd * DQ;
#pragma unroll
            for (int st = 0; st < KS; ++st) {
                const bf16x8_t kf = *reinterpret_cast<const bf16x8_t*>(kp + st * 8);
#pragma unroll
                for (int rt = 0; rt < RT; ++rt)
                    sacc[rt][kt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(kf, qreg[rt][st], sacc[rt][kt], 0, 0, 0);
            }
        }
        bf16x8_t pb[RT][2];
#pragma unroll
        for (int rt = 0; rt < RT; ++rt) {
            // rounds that lie wholly inside every row's range need no mask
            const int first_row = start + wrow0 + rt * 16;
            const bool full = kb + 63 <= first_row &&
                              (window <= 0 || kb >= min(first_row + 15, start + len - 1) - window + 1);
            float mx = neg_inf;
            if (full) {
#pragma unroll
                for (int kt = 0; kt < 4; ++kt)
#pragma unroll
                    for (int r = 0; r < 4; ++r) mx = fmaxf(mx, sacc[rt][kt][r]);
            } else {
#pragma unroll
                for (int kt = 0; kt < 4; ++kt)
#pragma unroll
                    for (int r = 0; r < 4; ++r) {
                        const int key = kb + 32 * (kt >> 1) + 8 * qd + 4 * (kt & 1) + r;
                        const float sv = (key <= pq[rt] && key >= lo_q[rt]) ? sacc[rt][kt][r] : neg_inf;
                        sacc[rt][kt][r] = sv;
                        mx = fmaxf(mx, sv);
                    }
            }
            mx = max_half32(max_row16(mx));
            const float m_new = fmaxf(m[rt], mx * scale_log2e);      // the scale is positive
            const float m_use = m_new == neg_inf ? 0.f : m_new;      // a row that has seen no key yet
            const float alpha = __builtin_amdgcn_exp2f(m[rt] - m_use);
            float psum = 0.f;
#pragma unroll
            for (int kt = 0; kt < 4; ++kt)
#pragma unroll
                for (int r = 0; r < 4; ++r) {
                    const float p = __builtin_amdgcn_exp2f(fmaf(sacc[rt][kt][r], scale_log2e, -m_use));
                    sacc[rt][kt][r] = p;
                    psum += p;
                }
            l[rt] = l[rt] * alpha + psum;
            m[rt] = m_new;
#pragma unroll
            for (int dt = 0; dt < DT; ++dt) oacc[rt][dt] *= alpha;
#pragma unroll
            for (int kp = 0; kp < 2; ++kp)
                pb[rt][kp] = bf16x8_t{
                    static_cast<__bf16>(sacc[rt][2 * kp][0]), static_cast<__bf16>(sacc[rt][2 * kp][1]),
                    static_cast<__bf16>(sacc[rt][2 * kp][2]), static_cast<__bf16>(sacc[rt][2 * kp][3]),
                    static_cast<__bf16>(sacc[rt][2 * kp + 1][0]), static_cast<__bf16>(sacc[rt][2 * kp + 1][1]),
                    static_cast<__bf16>(sacc[rt][2 * kp + 1][2]), static_cast<__bf16>(sacc[rt][2 * kp + 1][3])};
        }
#pragma unroll
        for (int kp = 0; kp < 2; ++kp)
#pragma unroll
            for (int dt = 0; dt < DT; ++dt) {
                const bf16x8_t vf = *reinterpret_cast<const bf16x8_t*>(
                    sV + (buf * HD + dt * 16 + c) * VROW + 32 * kp + 8 * qd);
#pragma unroll
                for (int rt = 0; rt < RT; ++rt)
                    oacc[rt][dt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(vf, pb[rt][kp], oacc[rt][dt], 0, 0, 0);
            }
    };

    // Round r works on LDS buffer r % 2 while the registers hold round r + 1 (asked for a
    // whole round earlier); at its end they go to the other buffer and round r + 2 is asked
    // for.  Both halves pass the same barriers; the one with fewer rounds idles at the end.
    int kb = first_key(tile);
    int buf = 0;
    if (my_rounds > 0) { fetch(kb); stage(0); }
    if (my_rounds > 1) fetch(kb + 64);
    __syncthreads();
    for (int it = 0; it < n_rounds; ++it, kb += 64) {
        if (it < my_rounds && wave_active && kb <= wkmax && kb + 63 >= wkmin) compute(kb, buf);
        if (it + 1 < my_rounds) {
            stage(buf ^ 1);
            if (it + 2 < my_rounds) fetch(kb + 128);
        }
        __syncthreads();
        buf ^= 1;
    }
    if (!wave_active) return;
#pragma unroll
    for (int rt = 0; rt < RT; ++rt) {
        float lt = l[rt];
        lt = sum_half32(sum_row16(lt));
        if (!row_valid[rt]) continue;
        const float inv_l = 1.0f / lt;
        bf16* orow = out + (row_base + wrow0 + rt * 16 + c) * ldo + static_cast<size_t>(h) * HD + 4 * qd;
#pragma unroll
        for (int dt = 0; dt < DT; ++dt) {
            const bf16x4_t o = {static_cast<__bf16>(oacc[rt][dt][0] * inv_l), static_cast<__bf16>(oacc[rt][dt][1] * inv_l),
                                static_cast<__bf16>(oacc[rt][dt][2] * inv_l), static_cast<__bf16>(oacc[rt][dt][3] * inv_l)};
            *reinterpret_cast<bf16x4_t*>(orow + dt * 16) = o;
        }
    }
}

template <int HD, int RT>
static int launch_attention_rows(
    const void* q, int ldq, const void* k_pool, const void* v_pool, const int* table,
    int table_stride, const int* cu_seqlens, const int* seq_slot, const int* seq_start,
    int n_seqs, int n_tokens, void* out, int ldo, int q_heads, int kv_heads, int page_tokens,
    int n_layers, int layer, float scale, int window, hipStream_t stream) {
    const size_t lds = (4 * 64 * (HD + 8) + 4 * HD * (64 + 8)) * sizeof(bf16) +
                       static_cast<size_t>(table_stride) * sizeof(int);
    if (lds > 160 * 1024) return static_cast<int>(hipErrorInvalidValue);
    auto kernel = attention_rows_kernel<HD, RT>;
    if (lds > 48 * 1024) {
        const hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(kernel),
                                                 hipFuncAttributeMaxDynamicSharedMemorySize,
                                                 static_cast<int>(lds));
        if (e != hipSuccess) return static_cast<int>(e);
    }
    // >= sum over requests of ceil(tiles / 2), tiles = ceil(rows / (64 RT))
    const int max_pairs = (n_tokens / (64 * RT) + 2 * n_seqs + 1) / 2;
    dim3 grid(max_pairs, q_heads), block(512);
    hipLaunchKernelGGL(kernel, grid, block, lds, stream, static_cast<const bf16*>(q), ldq,
                       static_cast<const bf16*>(k_pool), static_cast<const bf16*>(v_pool), table,
                       table_stride, cu_seqlens, seq_slot, seq_start, n_seqs,
                       static_cast<bf16*>(out), ldo, q_heads, kv_heads, page_tokens,
                       __builtin_ctz(page_tokens), n_layers, layer, scale * 1.4426950408889634f, window);
    return CELEG_LAUNCH_RESULT();
}

// rows_per_tile: 64 or 128 rows a workgroup (0: chosen from the number of rows).
extern "C" int celeg_attention_rows_bf16(
    const void* q, int ldq, const void* k_pool, const void* v_pool, const int* table,
    int table_stride, const int* cu_seqlens, const int* seq_slot, const int* seq_start,
    int n_seqs, int n_tokens, void* out, int ldo, int q_heads, int kv_heads, int head_dim,
    int page_tokens, int n_layers, int layer, float scale, int window, int rows_per_tile,
    hipStream_t stream) {
    if (n_tokens <= 0 || n_seqs <= 0) return 0;
    if (page_tokens < 16 || (page_tokens & (page_tokens - 1)) || q_heads % kv_heads || (ldq % 8) ||
        (ldo % 4))
        return static_cast<int>(hipErrorInvalidValue);
    if (rows_per_tile == 0) rows_per_tile = CELEG_ROWS_DEFAULT(n_tokens, n_seqs);
    if (rows_per_tile != 64 && rows_per_tile != 128) return static_cast<int>(hipErrorInvalidValue);
#define CELEG_ROWS(HD_)                                                                          \
    return rows_per_tile == 64                                                                   \
        ? launch_attention_rows<HD_, 1>(q, ldq, k_pool, v_pool, table, table_stride, cu_seqlens, \
              seq_slot, seq_start, n_seqs, n_tokens, out, ldo, q_heads, kv_heads, page_tokens,   \
              n_layers, layer, scale, window, stream)                                            \
        : launch_attention_rows<HD_, 2>(q, ldq, k_pool, v_pool, table, table_stride, cu_seqlens, \
              seq_slot, seq_start, n_seqs, n_tokens, out, ldo, q_heads, kv_heads, page_tokens,   \
              n_layers, layer, scale, window, stream)
    switch (head_dim) {
        case 32: CELEG_ROWS(32);
        case 64: CELEG_ROWS(64);
        case 96: CELEG_ROWS(96);
        case 128: CELEG_ROWS(128);
        default: return static_cast<int>(hipErrorInvalidValue);
    }
#undef CELEG_ROWS
}

// ================================================================ one row per request
// Decode attention works on rounds of 64 keys.
#define DEC_KEYS 64

// Joins the rounds of one (request, query head): out = sum_i e^(m_i - m) o_i / sum_i e^(m_i - m) l_i.
// A lane owns an output dimension (and the (m, l) of rounds lane, lane + 64, ..).  The rounds'
// outputs are asked for 32 at a time without conditions, the first 32 before anything is
// waited for, so that a context of 2,048 keys costs two trips to memory.
template <int HD>
__global__ __launch_bounds__(64) void attention_decode_reduce_kernel(
    const float* __restrict__ ws_o, const float* __restrict__ ws_ml,
    const int* __restrict__ positions, bf16* __restrict__ out, int ldo, int q_heads, int n_splits,
    int window) {
    constexpr int DD = HD / 64, CH = 32;
    const int h = blockIdx.x, t = blockIdx.y, lane = threadIdx.x;
    const int pos = positions[t];
    const int lo = window > 0 ? max(0, pos - window + 1) : 0;
    const int first = lo / DEC_KEYS, n_all = pos / DEC_KEYS - first + 1;
    const size_t base = (static_cast<size_t>(t) * q_heads + h) * n_splits + first;
    const float* __restrict__ op = ws_o + base * HD + lane;
    float o[CH][DD];
    auto fetch = [&](int j0) {
#pragma unroll
        for (int j = 0; j < CH; ++j) {
            const size_t jj = static_cast<size_t>(min(j0 + j, n_all - 1));     // past the end: the last one, weighted 0
#pragma unroll
            for (int dd = 0; dd < DD; ++dd) o[j][dd] = op[jj * HD + 64 * dd];
        }
    };
    fetch(0);
    float m = -INFINITY;
    for (int i = lane; i < n_all; i += 64) m = fmaxf(m, ws_ml[2 * (base + i)]);
    m = wave_max(m);
    float denom = 0.f, acc[DD];
#pragma unroll
    for (int dd = 0; dd < DD; ++dd) acc[dd] = 0.f;
    for (int i0 = 0; i0 < n_all; i0 += 64) {
        const int i = min(i0 + lane, n_all - 1);
        const float w = i0 + lane < n_all ? expf(ws_ml[2 * (base + i)] - m) : 0.f;
        denom += wave_sum(w * ws_ml[2 * (base + i) + 1]);
        const int n = min(64, n_all - i0);
        for (int j0 = 0; j0 < n; j0 += CH) {
            if (i0 + j0 > 0) fetch(i0 + j0);          // the first 32 are here already
#pragma unroll
            for (int j = 0; j < CH; ++j) {
                const float wj = j0 + j < n ? __shfl(w, min(j0 + j, 63), 64) : 0.f;
#pragma unroll
                for (int dd = 0; dd < DD; ++dd) acc[dd] = fmaf(wj, o[j][dd], acc[dd]);
            }
        }
    }
    bf16* orow = out + static_cast<size_t>(t) * ldo + static_cast<size_t>(h) * HD;
#pragma unroll
    for (int dd = 0; dd < DD; ++dd) orow[lane + 64 * dd] = from_float<bf16>(acc[dd] / denom);
}

// Decode attention: the query heads of a key/value head (up to 16 of them a workgroup) are
// the rows of matrix instructions, so the work per key does not grow with the group.  Two
// forms.  For batches that fill the chip, one workgroup per (request, key/value head, chunk of
// 16 heads) and no second kernel: its wavefronts take rounds of 64 keys in turn, each keeps
// a running maximum, sum and output of its own, and they meet in LDS.  For few requests
// (SPLIT), a workgroup of one wavefront per round of 64 keys, so that a long context spreads
// over the chip; the rounds' (max, sum, output) go to a workspace and
// attention_decode_reduce_kernel joins them.
//   S^T[key, head] = K Q^T : a lane holds head lane%16, keys 4*(lane/16)..+3 of a 16-key tile;
//   O^T[dim, head] = V^T P : P's operand wants 8 keys a lane, which are rows 4q..4q+3 of two
//   tiles: tile 2j holds keys 32j + 8*(row/4) + row%4, tile 2j+1 those + 4, so that a lane's
//   eight p are eight keys in a row and V (stored [dim][key] in a page) is read 16 bytes a lane.
template <int HD, int WAVES, bool SPLIT>
__global__ __launch_bounds__(WAVES * 64) void attention_decode_heads_kernel(
    const bf16* __restrict__ q, int ldq, const bf16* __restrict__ k_pool,
    const bf16* __restrict__ v_pool, const int* __restrict__ table, int table_stride,
    const int* __restrict__ token_slot, const int* __restrict__ positions, bf16* __restrict__ out,
    int ldo, int kv_heads, int group, int page_tokens, int page_shift, int n_layers, int layer,
    float scale, int window, float* __restrict__ ws_o, float* __restrict__ ws_ml, int n_splits) {
    constexpr int KS = HD / 32;   // steps of 32 dims in q.k
    constexpr int DT = HD / 16;   // 16-dim tiles of the output
    extern __shared__ float smem_heads[];
    const int chunks = (group + 15) >> 4;
    const int kvh = blockIdx.x / chunks, chunk = blockIdx.x % chunks;
    const int gp = min(group - chunk * 16, 16);          // heads of this workgroup
    const int h0 = kvh * group + chunk * 16;
    const int t = blockIdx.y;
    float* const part_o = smem_heads;                                      // [waves][gp][HD]
    float* const part_ml = smem_heads + static_cast<size_t>(WAVES) * gp * HD;   // [waves][gp][2]
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6), lane = threadIdx.x & 63;
    const int c = lane & 15, qd = lane >> 4;
    const int pos = positions[t];
    const int lo = window > 0 ? max(0, pos - window + 1) : 0;
    const int* __restrict__ pages = table + static_cast<size_t>(token_slot[t]) * table_stride;
    const int page_mask = page_tokens - 1;

    bf16x8_t qf[KS];
    {
        const bf16* qrow = q + static_cast<size_t>(t) * ldq + static_cast<size_t>(h0 + min(c, gp - 1)) * HD + qd * 8;
#pragma unroll
        for (int s = 0; s < KS; ++s) qf[s] = *reinterpret_cast<const bf16x8_t*>(qrow + s * 32);
    }
    float m_run = -INFINITY, l_run = 0.f;
    floatx4_t o[DT];
#pragma unroll
    for (int dt = 0; dt < DT; ++dt) o[dt] = floatx4_t{0.f, 0.f, 0.f, 0.f};

    const int r_first = SPLIT ? static_cast<int>(blockIdx.z) : lo / DEC_KEYS + wave;
    if (SPLIT && (r_first < lo / DEC_KEYS || r_first > pos / DEC_KEYS)) return;     // the whole workgroup
    for (int r = r_first; r <= pos / DEC_KEYS; r += SPLIT ? (1 << 30) : WAVES) {
        const int kb = r * DEC_KEYS;
        const int k_lo = max(lo, kb), k_hi = min(pos, kb + DEC_KEYS - 1);
        const int first_page = kb >> page_shift, last_page = k_hi >> page_shift;
        const int my_page = pages[min(first_page + lane, last_page)];
        bf16x8_t kf[4][KS], vf[DT][2];
#pragma unroll
        for (int T = 0; T < 4; ++T) {
            const int keyc = min(max(kb + 32 * (T >> 1) + 8 * (c >> 2) + 4 * (T & 1) + (c & 3), k_lo), k_hi);
            const int page = __shfl(my_page, (keyc >> page_shift) - first_page, 64);
            const bf16* kp = k_pool + kv_block(page, n_layers, layer, kv_heads, kvh, page_tokens, HD) +
                             static_cast<size_t>(keyc & page_mask) * HD + qd * 8;
#pragma unroll
            for (int s = 0; s < KS; ++s) kf[T][s] = *reinterpret_cast<const bf16x8_t*>(kp + s * 32);
        }
#pragma unroll
        for (int j = 0; j < 2; ++j) {
            // eight keys in a row; a group outside the range reads one inside (its p are zero)
            const int key0 = min(max(kb + 32 * j + 8 * qd, k_lo & ~7), k_hi & ~7);
            const int page = __shfl(my_page, (key0 >> page_shift) - first_page, 64);
            const bf16* vbase = v_pool + kv_block(page, n_layers, layer, kv_heads, kvh, page_tokens, HD) +
                                (key0 & page_mask);
#pragma unroll
            for (int dt = 0; dt < DT; ++dt)
                vf[dt][j] = *reinterpret_cast<const bf16x8_t*>(vbase + static_cast<size_t>(16 * dt + c) * page_tokens);
        }
        float sc[4][4];
        float mx = -INFINITY;
#pragma unroll
        for (int T = 0; T < 4; ++T) {
            floatx4_t acc = floatx4_t{0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int s = 0; s < KS; ++s) acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(kf[T][s], qf[s], acc, 0, 0, 0);
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                const int key = kb + 32 * (T >> 1) + 8 * qd + 4 * (T & 1) + i;
                sc[T][i] = (key >= k_lo && key <= k_hi) ? acc[i] * scale : -INFINITY;
                mx = fmaxf(mx, sc[T][i]);
            }
        }
        mx = fmaxf(mx, __shfl_xor(mx, 16, 64));
        mx = fmaxf(mx, __shfl_xor(mx, 32, 64));        // finite: the round holds a key
        const float m_new = fmaxf(m_run, mx);
        const float keep = expf(m_run - m_new);         // e^(-inf) = 0 the first time
        float psum = 0.f;
#pragma unroll
        for (int T = 0; T < 4; ++T)
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                sc[T][i] = expf(sc[T][i] - m_new);
                psum += sc[T][i];
            }
        psum += __shfl_xor(psum, 16, 64);
        psum += __shfl_xor(psum, 32, 64);
        l_run = l_run * keep + psum;
        m_run = m_new;
#pragma unroll
        for (int dt = 0; dt < DT; ++dt)
#pragma unroll
            for (int i = 0; i < 4; ++i) o[dt][i] *= keep;
#pragma unroll
        for (int j = 0; j < 2; ++j) {
            bf16x8_t pb;
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                pb[i] = static_cast<__bf16>(sc[2 * j][i]);
                pb[4 + i] = static_cast<__bf16>(sc[2 * j + 1][i]);
            }
#pragma unroll
            for (int dt = 0; dt < DT; ++dt)
                o[dt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(vf[dt][j], pb, o[dt], 0, 0, 0);
        }
    }
    if (SPLIT) {
        if (c < gp) {
            const size_t idx = (static_cast<size_t>(t) * (kv_heads * group) + h0 + c) * n_splits + blockIdx.z;
            if (qd == 0) { ws_ml[2 * idx] = m_run; ws_ml[2 * idx + 1] = l_run; }
#pragma unroll
            for (int dt = 0; dt < DT; ++dt)
                *reinterpret_cast<floatx4_t*>(ws_o + idx * HD + 16 * dt + 4 * qd) = o[dt];
        }
        return;
    }
    if (c < gp) {
        if (qd == 0) {
            part_ml[(wave * gp + c) * 2] = m_run;
            part_ml[(wave * gp + c) * 2 + 1] = l_run;
        }
#pragma unroll
        for (int dt = 0; dt < DT; ++dt)
#pragma unroll
            for (int i = 0; i < 4; ++i)
                part_o[(static_cast<size_t>(wave) * gp + c) * HD + 16 * dt + 4 * qd + i] = o[dt][i];
    }
    __syncthreads();
    for (int e = threadIdx.x; e < gp * HD; e += WAVES * 64) {
        const int g = e / HD, d = e % HD;
        float mxw = -INFINITY;
        for (int w = 0; w < WAVES; ++w) mxw = fmaxf(mxw, part_ml[(w * gp + g) * 2]);
        float denom = 0.f, val = 0.f;
        for (int w = 0; w < WAVES; ++w) {
            const float wgt = expf(part_ml[(w * gp + g) * 2] - mxw);   // a wavefront without a round: e^(-inf) = 0
            denom += wgt * part_ml[(w * gp + g) * 2 + 1];
            val = fmaf(wgt, part_o[(static_cast<size_t>(w) * gp + g) * HD + d], val);
        }
        out[static_cast<size_t>(t) * ldo + static_cast<size_t>(h0 + g) * HD + d] = from_float<bf16>(val / denom);
    }
}

template <int HD>
static int launch_decode_heads(const void* q, int ldq, const void* k_pool, const void* v_pool,
                               const int* table, int table_stride, const int* token_slot,
                               const int* positions, void* out, int ldo, int n_rows, int kv_heads,
                               int group, int page_tokens, int page_shift, int n_layers, int layer,
                               float scale, int window, hipStream_t stream) {
    constexpr int WAVES = HD <= 64 ? 16 : 8;   // what the registers of a CU hold of this head size
    const int chunks = (group + 15) / 16;
    const size_t lds = static_cast<size_t>(WAVES) * min(group, 16) * (HD + 2) * sizeof(float);
    static bool raised = false;
    if (lds > 48 * 1024 && !raised) {
        hipError_t err = hipFuncSetAttribute(reinterpret_cast<const void*>(&attention_decode_heads_kernel<HD, WAVES, false>),
                                             hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024);
        if (err != hipSuccess) return static_cast<int>(err);
        raised = true;
    }
    hipLaunchKernelGGL((attention_decode_heads_kernel<HD, WAVES, false>), dim3(kv_heads * chunks, n_rows),
                       dim3(WAVES * 64), lds, stream, static_cast<const bf16*>(q), ldq,
                       static_cast<const bf16*>(k_pool), static_cast<const bf16*>(v_pool), table,
                       table_stride, token_slot, positions, static_cast<bf16*>(out), ldo, kv_heads,
                       group, page_tokens, page_shift, n_layers, layer, scale, window, nullptr, nullptr, 0);
    return CELEG_LAUNCH_RESULT();
}

extern "C" int celeg_attention_decode_bf16(
    const void* q, int ldq, const void* k_pool, const void* v_pool, const int* table,
    int table_stride, const int* token_slot, const int* positions, float* ws_o, float* ws_ml,
    int n_splits, void* out, int ldo, int n_rows, int q_heads, int kv_heads,
    int head_dim, int page_tokens, int n_layers, int layer, float scale, int window, int whole,
    hipStream_t stream) {
    if (n_rows <= 0) return 0;
    const int group = q_heads / kv_heads;
    if (q_heads % kv_heads || page_tokens < 16 || (page_tokens & (page_tokens - 1)) || n_splits <= 0 ||
        (ldq % 8) || (reinterpret_cast<uintptr_t>(q) & 15))     // q is read 16 bytes at a time
        return static_cast<int>(hipErrorInvalidValue);
    const int page_shift = __builtin_ctz(page_tokens);
    const int chunks = (group + 15) / 16;
    // whole: 0 a workgroup per round of 64 keys and a second kernel, 1 one workgroup per
    // (request, key/value head), -1 decide here: the latter once there are enough of them to
    // fill the chip (measured at context 2,100 with 8 key/value heads, groups of 2 and of 4
    // heads: equal at 16 requests, one workgroup each 5 to 8 % of a decode step faster at 32
    // and 64 requests, a workgroup per round 2 to 5 % faster at 1 to 8).
    if (whole < 0) whole = kv_heads * chunks * n_rows >= 192 ? 1 : 0;
    if (whole) {
        if (head_dim == 64)
            return launch_decode_heads<64>(q, ldq, k_pool, v_pool, table, table_stride, token_slot, positions,
                                           out, ldo, n_rows, kv_heads, group, page_tokens, page_shift,
                                           n_layers, layer, scale, window, stream);
        if (head_dim == 128)
            return launch_decode_heads<128>(q, ldq, k_pool, v_pool, table, table_stride, token_slot, positions,
                                            out, ldo, n_rows, kv_heads, group, page_tokens, page_shift,
                                            n_layers, layer, scale, window, stream);
        return static_cast<int>(hipErrorInvalidValue);
    }
    dim3 sgrid(kv_heads * chunks, n_rows, n_splits);
#define CELEG_SPLIT_HEADS(HD_)                                                                   \
    hipLaunchKernelGGL((attention_decode_heads_kernel<HD_, 1, true>), sgrid, dim3(64), 0, stream, \
                       static_cast<const bf16*>(q), ldq, static_cast<const bf16*>(k_pool),       \
                       static_cast<const bf16*>(v_pool), table, table_stride, token_slot,        \
                       positions, static_cast<bf16*>(out), ldo, kv_heads, group, page_tokens,    \
                       page_shift, n_layers, layer, scale, window, ws_o, ws_ml, n_splits);       \
    hipLaunchKernelGGL(attention_decode_reduce_kernel<HD_>, dim3(q_heads, n_rows), dim3(64), 0,  \
                       stream, ws_o, ws_ml, positions, static_cast<bf16*>(out), ldo, q_heads,    \
                       n_splits, window)
    if (head_dim == 64) { CELEG_SPLIT_HEADS(64); }
    else if (head_dim == 128) { CELEG_SPLIT_HEADS(128); }
    else return static_cast<int>(hipErrorInvalidValue);
#undef CELEG_SPLIT_HEADS
    return CELEG_LAUNCH_RESULT();
}
