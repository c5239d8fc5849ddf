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
#include "no_alloc.h"
#include <mutex>

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
// A workgroup takes a tile of 64*RT rows of one request for one query head.  Its 8
// wavefronts are two halves of 4; the wavefronts of a half each own RT tiles of 16 rows of
// the same 64*RT rows, and the halves take the rounds of 64 keys in turn (half 0 the even
// rounds of the tile's key range, half 1 the odd ones), each with a running maximum, sum
// and output of its own.  At the end half 1 hands its (maximum, sum, output) over through
// LDS, and half 0 joins the two and writes.  Under the causal mask the last tile of a
// request sees the most keys, so a request's tiles are handed out last first.
// The keys and values of a round are staged in LDS once for the 4 wavefronts of a half
// (two buffers a half: the half's next round is fetched into registers while the current
// one is worked on, and written to the other buffer before the one barrier of the
// round).  Per 64 keys: S^T = K Q^T (16x16x32 MFMA: A = 16 keys x 32 dims,
// B = 32 dims x 16 rows), online softmax per row (a row is a lane column), then
// O^T += V^T P^T (A = 16 dims x 32 keys from the transposed V, B = P^T straight from the
// accumulator registers of S^T).  The 16 keys of a score tile are chosen so that a lane
// ends up with the probabilities of 8 neighbouring keys, which is what one 16-byte read
// of the transposed V delivers; in LDS the keys lie in the order of the score tiles, so
// that the 16 lanes of a read touch 16 rows in a row (no bank is asked twice).
// The running maximum of a row follows the scores only when some row's grows by more than
// 8 (a factor 2^8): until then probabilities are taken against the older value, stay below
// 2^8, and numerator and denominator carry the same factor.
template <int HD, int RT, int NH, bool SHARE>
__global__ __launch_bounds__(256 * NH) void attention_rows_kernel(
    const bf16* __restrict__ q, int ldq, const bf16* __restrict__ k_pool,
    const bf16* __restrict__ v_pool, const int* __restrict__ table, int table_stride,
    const int* __restrict__ cu_seqlens, const int* __restrict__ seq_slot,
    const int* __restrict__ seq_start, int n_seqs, bf16* __restrict__ out, int ldo,
    int q_heads, int kv_heads, int page_tokens, int page_shift, int n_layers, int layer,
    float scale_log2e, int window, int pages_room) {
    constexpr int ROWS = 64 * RT;   // rows of a workgroup
    constexpr int WROWS = 16 * RT;  // rows of a wavefront
    constexpr int DQ = HD / 4;      // dims a lane quad covers in q.k
    constexpr int KS = DQ / 8;      // MFMA steps of 32 along head_dim
    constexpr int DT = HD / 16;     // 16-dim tiles of the output
    constexpr int KROW = HD + 8;    // LDS row of a key, padded against bank conflicts
    constexpr int VROW = 64 + 8;    // LDS row of a dimension: 64 keys, padded
    constexpr int NSET = SHARE ? 1 : NH;          // sets of staging buffers
    constexpr int NT = SHARE ? 256 * NH : 256;    // threads that fill a set
    constexpr int CH = (8 * HD + NT - 1) / NT;    // 16-byte pieces of K, and of V, a thread moves per round
    constexpr float LAZY = 8.f;     // growth of a row's maximum that is let pass
    extern __shared__ int smem[];
    // wavefront-uniform values are kept in scalar registers
    const int half = NH == 1 ? 0 : __builtin_amdgcn_readfirstlane(static_cast<int>(threadIdx.x) >> 8);
    const int tid = threadIdx.x & 255;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6), lane = tid & 63;
    const int set = SHARE ? 0 : half;
    __bf16* const sK = reinterpret_cast<__bf16*>(smem) + set * (2 * 64 * KROW);       // [NSET][2][64][KROW]
    __bf16* const sV = reinterpret_cast<__bf16*>(smem) + NSET * 2 * 64 * KROW + set * (2 * HD * VROW);  // [NSET][2][HD][VROW]
    int* const spages = reinterpret_cast<int*>(reinterpret_cast<__bf16*>(smem) + NSET * 2 * (64 * KROW + HD * VROW));
    // Which tile and head.  Workgroups go to the chip's 8 dies in turn (number % 8), and each
    // die has an L2 of its own; so the list of all (key/value head, tile, query head of the
    // group, or NH of them where the halves share the staged keys), in this order, is cut into 8
    // runs, one per die: a die then reads the keys and values of few heads, and workgroups that
    // start together read the same ones.
    int all_tiles = 0;
    for (int i = 0; i < n_seqs; ++i) all_tiles += (cu_seqlens[i + 1] - cu_seqlens[i] + ROWS - 1) / ROWS;
    const int group = q_heads / kv_heads;
    const int per_group = SHARE ? (group + NH - 1) / NH : group;   // workgroups a tile of a key/value head takes
    const long long all_items = static_cast<long long>(all_tiles) * kv_heads * per_group;
    const int die = blockIdx.x & 7;
    const long long item = (all_items * die + 7) / 8 + (blockIdx.x >> 3);
    if (item >= (all_items * (die + 1) + 7) / 8) return;   // the whole workgroup
    const int in_group = static_cast<int>(item % per_group) * (SHARE ? NH : 1) + (SHARE ? half : 0);
    const bool head_valid = in_group < group;      // a group that the halves do not divide
    const int h = static_cast<int>(item / per_group / all_tiles) * group + min(in_group, group - 1);
    int idx = static_cast<int>(item / per_group % all_tiles);
    int s = 0, len = 0, tiles = 0;
    for (;; ++s) {
        len = cu_seqlens[s + 1] - cu_seqlens[s];
        tiles = (len + ROWS - 1) / ROWS;
        if (idx < tiles) break;
        idx -= tiles;
    }
    const int tile = tiles - 1 - idx;
    const int start = seq_start[s];
    const int brow0 = tile * ROWS;
    const int first = ((window > 0 ? max(0, start + brow0 - window + 1) : 0) >> 6) << 6;   // first key of the first round
    const int bkmax = start + min(brow0 + ROWS - 1, len - 1);                              // last key the tile sees
    const int total_rounds = ((bkmax - first) >> 6) + 1;
    constexpr int TURNS = SHARE ? 1 : NH;          // halves that take the rounds in turn
    const int my_rounds = SHARE ? total_rounds : (total_rounds - half + NH - 1) / NH;   // rounds half, half + NH, ..
    const int n_it = (total_rounds + TURNS - 1) / TURNS;
    // the pages of the tile's rounds; behind the last key's page, that page again (allocated
    // memory for the positions of the last round that are masked anyway), and before the
    // first page that a row of the tile can still see (the first round starts at a multiple of
    // 64 keys, which may lie in a page that a window has passed and the request has given
    // back), that page.  They are copied to LDS where they fit its room; a tile with more
    // pages than that (a context of several ten thousand tokens) looks them up in memory.
    const int page0 = first >> page_shift;
    const int* __restrict__ const pages = table + static_cast<size_t>(seq_slot[s]) * table_stride;
    const int last_page = bkmax >> page_shift;
    const int live_page = (window > 0 ? max(0, start + brow0 - window + 1) : 0) >> page_shift;
    const int n_fill = ((first + 64 * total_rounds - 1) >> page_shift) - page0 + 1;
    const bool pages_in_lds = n_fill <= pages_room;
    if (pages_in_lds)
        for (int i = threadIdx.x; i < n_fill; i += 256 * NH)
            spages[i] = pages[min(max(page0 + i, live_page), last_page)];
    __syncthreads();
    auto page_at = [&](int i) __attribute__((always_inline)) -> unsigned {
        return pages_in_lds ? spages[i] : pages[min(max(page0 + i, live_page), last_page)];
    };
    const int c = lane & 15, qd = lane >> 4;
    const int wrow0 = brow0 + wave * WROWS;
    const bool wave_active = wrow0 < len && head_valid;
    const int wkmax = start + min(wrow0 + WROWS - 1, len - 1);  // last key any row of the wavefront sees
    const int wkmin = window > 0 ? max(0, start + wrow0 - window + 1) : 0;
    const int kvh = h / (q_heads / kv_heads);
    const size_t row_base = static_cast<size_t>(cu_seqlens[s]);
    const size_t head_block = static_cast<size_t>(page_tokens) * HD;
    const unsigned page_stride = static_cast<unsigned>(n_layers * kv_heads) * static_cast<unsigned>(head_block);   // the host has checked that it fits
    const size_t layer_head = (static_cast<size_t>(layer) * kv_heads + kvh) * head_block;
    const bf16* __restrict__ const kbase = k_pool + layer_head;
    const bf16* __restrict__ const vbase = v_pool + layer_head;

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
    // neighbouring memory.  What does not change from round to round is worked out here:
    // the page of the round a piece lies in, its place inside the page, its place in LDS.
    const int pt_shift = min(page_shift, 6);          // keys of a page inside a round: 1 << pt_shift
    const int in_page = page_tokens - 1;
    int k_pg[CH], k_off[CH], k_lds[CH], v_pg[CH], v_off[CH], v_lds[CH];
    bool has_piece[CH];      // the last one may be past the end
#pragma unroll
    for (int j = 0; j < CH; ++j) {
        const int i_all = (SHARE ? static_cast<int>(threadIdx.x) : tid) + NT * j;
        has_piece[j] = (8 * HD) % NT == 0 || i_all < 8 * HD;
        const int i = min(i_all, 8 * HD - 1);
        const int key = i / (HD / 8), part = i % (HD / 8);
        k_pg[j] = key >> page_shift;
        k_off[j] = (key & in_page) * HD + part * 8;
        // key 32 a + 8 b + 4 t + r of the round is row b*4 + r of score tile 2 a + t
        const int krow = 16 * (2 * (key >> 5) + ((key >> 2) & 1)) + 4 * ((key >> 3) & 3) + (key & 3);
        k_lds[j] = krow * KROW + part * 8;
        const int piece = (i >> (pt_shift - 3)) / HD;      // which page of the round
        const int rem = i - piece * (HD << (pt_shift - 3));
        const int d = rem >> (pt_shift - 3), g = rem & ((1 << (pt_shift - 3)) - 1);
        v_pg[j] = piece;
        v_off[j] = d * page_tokens + g * 8;
        v_lds[j] = d * VROW + (piece << pt_shift) + g * 8;
    }
    u32x4_t kstage[CH], vstage[CH];
    auto fetch = [&](int kb) __attribute__((always_inline)) {
        const int pg = (kb >> page_shift) - page0;
        const int inp = kb & in_page;     // a round inside a longer page starts here
#pragma unroll
        for (int j = 0; j < CH; ++j) {
            if (!has_piece[j]) continue;
            const unsigned kpage = page_at(pg + k_pg[j]);
            kstage[j] = *reinterpret_cast<const u32x4_t*>(
                kbase + (static_cast<unsigned long long>(kpage) * page_stride + static_cast<unsigned>(inp * HD + k_off[j])));
            const unsigned vpage = page_at(pg + v_pg[j]);
            vstage[j] = *reinterpret_cast<const u32x4_t*>(
                vbase + (static_cast<unsigned long long>(vpage) * page_stride + static_cast<unsigned>(inp + v_off[j])));
        }
    };
    auto stage = [&](int buf) __attribute__((always_inline)) {
#pragma unroll
        for (int j = 0; j < CH; ++j) {
            if (!has_piece[j]) continue;
            *reinterpret_cast<u32x4_t*>(sK + buf * 64 * KROW + k_lds[j]) = kstage[j];
            *reinterpret_cast<u32x4_t*>(sV + buf * HD * VROW + v_lds[j]) = vstage[j];
        }
    };
    const float neg_inf = -INFINITY;
    // accumulator register r of lane quad qd, score tile kt, is key 32 (kt/2) + 8 qd + 4 (kt%2) + r
    auto compute = [&](int kb, int buf) __attribute__((always_inline)) {
        floatx4_t sacc[RT][4];
#pragma unroll
        for (int rt = 0; rt < RT; ++rt)
#pragma unroll
            for (int kt = 0; kt < 4; ++kt) sacc[rt][kt] = floatx4_t{0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int kt = 0; kt < 4; ++kt) {
            const __bf16* kp = sK + (buf * 64 + 16 * kt + c) * KROW + qd * DQ;
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
            if (!full) {
#pragma unroll
                for (int kt = 0; kt < 4; ++kt)
#pragma unroll
                    for (int r = 0; r < 4; ++r) {
                        const int key = kb + 32 * (kt >> 1) + 8 * qd + 4 * (kt & 1) + r;
                        if (key > pq[rt] || key < lo_q[rt]) sacc[rt][kt][r] = neg_inf;
                    }
            }
            float mx = neg_inf;
#pragma unroll
            for (int kt = 0; kt < 4; ++kt)
#pragma unroll
                for (int r = 0; r < 4; ++r) mx = fmaxf(mx, sacc[rt][kt][r]);
            mx = max_half32(max_row16(mx)) * scale_log2e;      // the scale is positive
            if (__builtin_amdgcn_ballot_w64(mx > m[rt] + LAZY) != 0) {
                const float m_new = fmaxf(m[rt], mx);
                const float alpha = __builtin_amdgcn_exp2f(m[rt] - (m_new == neg_inf ? 0.f : m_new));
                l[rt] *= alpha;
                m[rt] = m_new;
#pragma unroll
                for (int dt = 0; dt < DT; ++dt) oacc[rt][dt] *= alpha;
            }
            const float m_use = m[rt] == neg_inf ? 0.f : m[rt];      // a row that has seen no key yet
            float psum = 0.f;
#pragma unroll
            for (int kt = 0; kt < 4; ++kt)
#pragma unroll
                for (int r = 0; r < 4; ++r) {
                    const float p = __builtin_amdgcn_exp2f(fmaf(sacc[rt][kt][r], scale_log2e, -m_use));
                    sacc[rt][kt][r] = p;
                    psum += p;
                }
            l[rt] += psum;
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

    // Round r of a set of staging buffers works on LDS buffer r % 2 while the registers hold
    // round r + 1 (asked for a whole round earlier); at its end they go to the other buffer and
    // round r + 2 is asked for.  Halves that take the rounds in turn have a set each (round r
    // of half i is key block first + 64 (i + NH r)), and all pass the same barriers.
    int kb = first + (SHARE ? 0 : 64 * half);
    int buf = 0;
    if (my_rounds > 0) { fetch(kb); stage(0); }
    if (my_rounds > 1) fetch(kb + 64 * TURNS);
    __syncthreads();
    for (int it = 0; it < n_it; ++it, kb += 64 * TURNS) {
        if (it < my_rounds && wave_active && kb <= wkmax && kb + 63 >= wkmin) compute(kb, buf);
        if (it + 1 < my_rounds) {
            stage(buf ^ 1);
            if (it + 2 < my_rounds) fetch(kb + 128 * TURNS);
        }
        __syncthreads();
        buf ^= 1;
    }
    // the sets behind the first hand over: register by register, a lane to the same lane (the
    // sets' wavefronts of one number own the same rows; a set that had no round hands over
    // nothing: maximum -inf, sum and output 0).  The staging buffers are free after the last barrier.
    constexpr int XSET = 4 * RT * (4 * DT + 2) * 64;      // floats a set hands over
    float* const xch = reinterpret_cast<float*>(smem) + wave * (RT * (4 * DT + 2) * 64) + lane;
    if (TURNS > 1 && total_rounds > 1) {
        if (half >= 1 && wave_active) {
#pragma unroll
            for (int rt = 0; rt < RT; ++rt) {
                float* x = xch + (half - 1) * XSET + rt * (4 * DT + 2) * 64;
                x[0] = m[rt];
                x[64] = l[rt];
#pragma unroll
                for (int dt = 0; dt < DT; ++dt)
#pragma unroll
                    for (int r = 0; r < 4; ++r) x[(2 + 4 * dt + r) * 64] = oacc[rt][dt][r];
            }
        }
        __syncthreads();
    }
    if ((TURNS > 1 && half >= 1) || !wave_active) return;
#pragma unroll
    for (int rt = 0; rt < RT; ++rt) {
#pragma unroll
        for (int other = 1; other < TURNS; ++other) {
            if (total_rounds <= 1) break;
            const float* x = xch + (other - 1) * XSET + rt * (4 * DT + 2) * 64;
            const float m1 = x[0];
            const float m_new = fmaxf(m[rt], m1);
            const float m_use = m_new == neg_inf ? 0.f : m_new;
            const float a0 = __builtin_amdgcn_exp2f(m[rt] - m_use), a1 = __builtin_amdgcn_exp2f(m1 - m_use);
            l[rt] = l[rt] * a0 + x[64] * a1;
            m[rt] = m_new;
#pragma unroll
            for (int dt = 0; dt < DT; ++dt)
#pragma unroll
                for (int r = 0; r < 4; ++r)
                    oacc[rt][dt][r] = oacc[rt][dt][r] * a0 + x[(2 + 4 * dt + r) * 64] * a1;
        }
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

// Most entries of a block-table row that a workgroup of attention_rows_kernel copies to LDS.
// celeg_attention_rows_pages_in_lds() lets a test lower it, so that the lookup in memory runs
// at small sizes too.
static int ROWS_MAX_PAGES_IN_LDS = 4096;
extern "C" void celeg_attention_rows_pages_in_lds(int entries) {
    ROWS_MAX_PAGES_IN_LDS = entries > 0 ? min(entries, 4096) : 4096;
}

// LDS bytes that a launch with these sizes asks for (what the host-side check of the limit
// of 160 KB works with): form 1 or 2 = sets of staging buffers.
extern "C" long long celeg_attention_rows_lds_bytes(int head_dim, int sets, int table_stride) {
    const long long staging = static_cast<long long>(sets) * 2 * (64 * (head_dim + 8) + head_dim * (64 + 8)) * 2;
    const long long room = staging < 160 * 1024 ? (160 * 1024 - staging) / 4 : 0;
    return staging + min(static_cast<long long>(min(table_stride + 8, ROWS_MAX_PAGES_IN_LDS)), room) * 4;
}

template <int HD, int RT, int NH, bool SHARE>
static int launch_attention_rows(
    const void* q, int ldq, const void* k_pool, const void* v_pool, const int* table,
    int table_stride, const int* cu_seqlens, const int* seq_slot, const int* seq_start,
    int n_seqs, int n_tokens, void* out, int ldo, int q_heads, int kv_heads, int page_tokens,
    int n_layers, int layer, float scale, int window, hipStream_t stream) {
    // staging buffers, and a tile's pages with room for a round's worth behind the last: the
    // whole of a request's block-table row where that is at most ROWS_MAX_PAGES_IN_LDS entries
    // (16 KB; with the largest staging buffers, 143,360 bytes, still inside 160 KB)
    const size_t staging = static_cast<size_t>(SHARE ? 1 : NH) * 2 * (64 * (HD + 8) + HD * (64 + 8)) * sizeof(bf16);
    const int pages_room = min(min(table_stride + 8, ROWS_MAX_PAGES_IN_LDS),
                               staging < 160 * 1024 ? static_cast<int>((160 * 1024 - staging) / sizeof(int)) : 0);
    const size_t lds = staging + static_cast<size_t>(pages_room) * sizeof(int);
    static_assert(SHARE || static_cast<size_t>(NH - 1) * 4 * RT * (4 * (HD / 16) + 2) * 64 * sizeof(float) <=
                               static_cast<size_t>(NH) * 2 * (64 * (HD + 8) + HD * (64 + 8)) * sizeof(bf16),
                  "what the sets hand over fits the staging buffers");
    if (lds > 160 * 1024) return static_cast<int>(hipErrorInvalidValue);
    // the kernel multiplies page numbers by the elements of a page in 32 x 32 -> 64 bits
    if (static_cast<size_t>(n_layers) * kv_heads * page_tokens * HD >= (size_t{1} << 31))
        return static_cast<int>(hipErrorInvalidValue);
    auto kernel = attention_rows_kernel<HD, RT, NH, SHARE>;
    if (lds > 48 * 1024) {
        const hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(kernel),
                                                 hipFuncAttributeMaxDynamicSharedMemorySize,
                                                 static_cast<int>(lds));
        if (e != hipSuccess) return static_cast<int>(e);
    }
    // >= sum over requests of ceil(rows / (64 RT))
    const int max_tiles = n_tokens / (64 * RT) + n_seqs;
    const int group = q_heads / kv_heads;
    const long long max_items = static_cast<long long>(max_tiles) * kv_heads * (SHARE ? (group + NH - 1) / NH : group);
    dim3 grid(static_cast<unsigned>(8 * ((max_items + 7) / 8 + 1))), block(256 * NH);
    hipLaunchKernelGGL(kernel, grid, block, lds, stream, static_cast<const bf16*>(q), ldq,
                       static_cast<const bf16*>(k_pool), static_cast<const bf16*>(v_pool), table,
                       table_stride, cu_seqlens, seq_slot, seq_start, n_seqs,
                       static_cast<bf16*>(out), ldo, q_heads, kv_heads, page_tokens,
                       __builtin_ctz(page_tokens), n_layers, layer, scale * 1.4426950408889634f, window,
                       pages_room);
    return CELEG_LAUNCH_RESULT();
}

// rows_per_tile: 64 or 128 rows a workgroup.  form: 1, a workgroup of 4 wavefronts takes all
// rounds of keys of its tile for one query head; 2, two such sets take the rounds in turn and
// join at the end (more workgroups in flight and half as long a way for a tile with many
// keys: for few rows); 3, two sets take a query head each of those that share a key/value
// head, and the staged keys and values with it (half the traffic: for many rows); 4, four
// sets take the rounds in turn (tiles of 64 rows, heads of 32 or 64; never chosen here: a
// prompt of 2,048 tokens gives about as many tiles as the chip holds workgroups, so its time
// is that of the tile with the most rounds, which four sets walk in half as many steps as
// two, but one workgroup of 16 wavefronts a compute unit instead of two of 8 made the six
// attention layers of such a prefill 40 us slower, not faster).  0 leaves
// a choice to this function, which then goes by the number of rows and by context_hint, the
// longest context among the step's requests (0: not known).
extern "C" int celeg_attention_rows_bf16(
    const void* q, int ldq, const void* k_pool, const void* v_pool, const int* table,
    int table_stride, const int* cu_seqlens, const int* seq_slot, const int* seq_start,
    int n_seqs, int n_tokens, void* out, int ldo, int q_heads, int kv_heads, int head_dim,
    int page_tokens, int n_layers, int layer, float scale, int window, int rows_per_tile,
    int form, int context_hint, hipStream_t stream) {
    if (n_tokens <= 0 || n_seqs <= 0) return 0;
    if (page_tokens < 16 || (page_tokens & (page_tokens - 1)) || q_heads % kv_heads || (ldq % 8) ||
        (ldo % 4))
        return static_cast<int>(hipErrorInvalidValue);
    if (rows_per_tile == 0) {
        // tiles of 128 rows read the staged keys for twice the rows, tiles of 64 rows put twice
        // the workgroups on the chip: the larger ones once there are enough, sooner if each
        // has many keys to go through
        const long long small_tiles = static_cast<long long>(n_tokens / 64 + n_seqs) * q_heads;
        int keys = context_hint > 0 ? context_hint : n_tokens;
        if (window > 0 && window < keys) keys = window;
        rows_per_tile = small_tiles >= 1024 || (small_tiles >= 512 && keys >= 4096) ? 128 : 64;
    }
    if (rows_per_tile != 64 && rows_per_tile != 128) return static_cast<int>(hipErrorInvalidValue);
    if (form == 0) {
        const int group = q_heads / kv_heads;
        const long long shared = static_cast<long long>(n_tokens / rows_per_tile + n_seqs) * kv_heads * ((group + 1) / 2);
        form = group >= 2 && shared >= 1024 ? 3 : 2;
    }
    if (form < 1 || form > 4) return static_cast<int>(hipErrorInvalidValue);
    if (form == 4 && (rows_per_tile != 64 || head_dim > 64)) return static_cast<int>(hipErrorInvalidValue);
#define CELEG_ROWS_ARGS                                                                            \
    q, ldq, k_pool, v_pool, table, table_stride, cu_seqlens, seq_slot, seq_start, n_seqs, n_tokens, \
        out, ldo, q_heads, kv_heads, page_tokens, n_layers, layer, scale, window, stream
#define CELEG_ROWS_RT(HD_, RT_)                                                              \
    (form == 1 ? launch_attention_rows<HD_, RT_, 1, false>(CELEG_ROWS_ARGS)                   \
     : form == 2 ? launch_attention_rows<HD_, RT_, 2, false>(CELEG_ROWS_ARGS)                 \
                 : launch_attention_rows<HD_, RT_, 2, true>(CELEG_ROWS_ARGS))
#define CELEG_ROWS(HD_) return rows_per_tile == 64 ? CELEG_ROWS_RT(HD_, 1) : CELEG_ROWS_RT(HD_, 2)
    if (form == 4)
        return head_dim == 32 ? launch_attention_rows<32, 1, 4, false>(CELEG_ROWS_ARGS)
                              : launch_attention_rows<64, 1, 4, false>(CELEG_ROWS_ARGS);
    switch (head_dim) {
        case 32: CELEG_ROWS(32);
        case 64: CELEG_ROWS(64);
        case 96: CELEG_ROWS(96);
        case 128: CELEG_ROWS(128);
        default: return static_cast<int>(hipErrorInvalidValue);
    }
#undef CELEG_ROWS
#undef CELEG_ROWS_RT
#undef CELEG_ROWS_ARGS
}

// ================================================================ one row per request
// Decode attention works on rounds of 64 keys.
#define DEC_KEYS 64

// Joins the parts of one (request, query head), a part being some rounds of 64 keys:
// out = sum_i e^(m_i - m) o_i / sum_i e^(m_i - m) l_i.
// A lane owns an output dimension (and the (m, l) of parts lane, lane + 64, ..).  The parts'
// outputs are asked for 32 at a time without conditions, the first 32 before anything is
// waited for, so that a context of 2,048 keys in parts of one round costs two trips to memory.
template <int HD>
__global__ __launch_bounds__(64) void attention_decode_reduce_kernel(
    const float* __restrict__ ws_o, const float* __restrict__ ws_ml,
    const int* __restrict__ positions, bf16* __restrict__ out, int ldo, int q_heads, int n_splits,
    int window, int n_parts) {
    constexpr int DD = HD / 64, CH = 32;
    const int h = blockIdx.x, t = blockIdx.y, lane = threadIdx.x;
    const int pos = positions[t];
    const int lo = window > 0 ? max(0, pos - window + 1) : 0;
    // the request's rounds were shared out evenly over the parts (the same arithmetic as in attention_decode_heads_kernel)
    const int total = pos / DEC_KEYS - lo / DEC_KEYS + 1, per = (total + n_parts - 1) / n_parts;
    const int n_all = (total + per - 1) / per;
    const size_t base = (static_cast<size_t>(t) * q_heads + h) * n_splits;
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
// (SPLIT), a workgroup per part of the context (1, 4 or 16 rounds of 64 keys, a wavefront
// per round), so that a long context spreads over the chip; the parts' (max, sum, output) go
// to a workspace and attention_decode_reduce_kernel joins them.
//   S^T[key, head] = K Q^T : a lane holds head lane%16, keys 4*(lane/16)..+3 of a 16-key tile;
//   O^T[dim, head] = V^T P : P's operand wants 8 keys a lane, which are rows 4q..4q+3 of two
//   tiles: tile 2j holds keys 32j + 8*(row/4) + row%4, tile 2j+1 those + 4, so that a lane's
//   eight p are eight keys in a row and V (stored [dim][key] in a page) is read 16 bytes a lane.
// The step's own token where its key and value are not in the cache yet (k set): q and k come
// as the q/k/v product left them; the kernel then normalises and turns the query heads itself,
// takes the rounds of keys up to the position before the token's, and the workgroup (and
// wavefront) whose part holds the token's position prepares the new key, adds it and the new
// value to its running sums as one more key, and writes both into the request's page: what
// qk_norm_rope_store does as a kernel of its own before the attention.
struct DecodeFresh {
    const bf16* k;            // [rows, ldk] or null: the cache holds the step's keys and values already
    const bf16* v;            // [rows, ldv]
    int ldk, ldv;
    const float* q_weight;    // [HD] or null: no norm
    const float* k_weight;
    float eps;
    const float* cos_sin;     // [positions, HD / 2, 2] or null: no rotation
    bf16* k_pool;             // the pools again, to write to
    bf16* v_pool;
};

// A head's HD values spread over the four lanes qd = 0..3 of a head's lane group as the matrix
// instruction wants them (x[s][e] is dimension 32 s + 8 qd + e): norm (weight w in the same
// layout; null: none) and rotation by split halves (cs: (cos, sin) of pair 32 s + 8 qd + e for
// s < KS / 2; null: none), as qk_norm_rope_store makes them.
// What decode_prepare_head needs from memory, asked for early: the weight at the lane's
// dimensions and the (cos, sin) of its pairs.
template <int KS>
struct DecodeHeadOperands {
    floatx4_t w[KS][2];
    floatx4_t cs[KS / 2][4];
};
template <int KS>
__device__ __forceinline__ void decode_head_operands(DecodeHeadOperands<KS>& o, const float* __restrict__ w,
                                                     const float* __restrict__ cs, const int qd) {
    if (w) {
#pragma unroll
        for (int s = 0; s < KS; ++s) {
            o.w[s][0] = *reinterpret_cast<const floatx4_t*>(w + 32 * s + 8 * qd);
            o.w[s][1] = *reinterpret_cast<const floatx4_t*>(w + 32 * s + 8 * qd + 4);
        }
    }
    if (cs) {
#pragma unroll
        for (int s = 0; s < KS / 2; ++s)
#pragma unroll
            for (int e4 = 0; e4 < 4; ++e4) o.cs[s][e4] = *reinterpret_cast<const floatx4_t*>(cs + (32 * s + 8 * qd) * 2 + 4 * e4);
    }
}

template <int KS>
__device__ __forceinline__ void decode_prepare_head(float (&x)[KS][8], const bool normed, const bool rotate,
                                                    const floatx4_t (&w)[KS][2], const floatx4_t (&cs)[KS / 2][4], const float eps) {
    constexpr int HD = 32 * KS;
    if (normed) {
        float ssq = 0.f;
#pragma unroll
        for (int s = 0; s < KS; ++s)
#pragma unroll
            for (int e = 0; e < 8; ++e) ssq += x[s][e] * x[s][e];
        ssq += __shfl_xor(ssq, 16, 64);
        ssq += __shfl_xor(ssq, 32, 64);
        const float inv = 1.0f / sqrtf(ssq / static_cast<float>(HD) + eps);
#pragma unroll
        for (int s = 0; s < KS; ++s) {
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                x[s][e] = x[s][e] * inv * w[s][0][e];
                x[s][4 + e] = x[s][4 + e] * inv * w[s][1][e];
            }
        }
    }
    if (rotate) {
#pragma unroll
        for (int s = 0; s < KS / 2; ++s) {
#pragma unroll
            for (int e4 = 0; e4 < 4; ++e4) {          // two pairs a load
                const floatx4_t t = cs[s][e4];
#pragma unroll
                for (int h = 0; h < 2; ++h) {
                    const int e = 2 * e4 + h;
                    const float a = x[s][e], b = x[s + KS / 2][e];
                    x[s][e] = a * t[2 * h] - b * t[2 * h + 1];
                    x[s + KS / 2][e] = b * t[2 * h] + a * t[2 * h + 1];
                }
            }
        }
    }
}

template <int HD, int WAVES, bool SPLIT, bool FRESH>
__global__ __launch_bounds__(WAVES * 64) void attention_decode_heads_kernel(
    // (the pointers that the first loads go through first: the leading 14 words of the arguments
    // arrive in registers with the launch)
    const bf16* __restrict__ q, const bf16* __restrict__ k_pool, const bf16* __restrict__ v_pool,
    const int* __restrict__ table, const int* __restrict__ token_slot, const int* __restrict__ positions,
    int ldq, int table_stride, bf16* __restrict__ out, int ldo, int kv_heads, int group, int page_tokens, int page_shift, int n_layers, int layer,
    float scale, int window, float* __restrict__ ws_o, float* __restrict__ ws_ml, int n_splits,
    int n_parts, const DecodeFresh fresh) {
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

    // The query heads as the product left them: norm and rotation here.  A workgroup of one
    // wavefront (one round of keys) asks for what that needs now, does the arithmetic once its
    // round's keys have been asked for, and asks for the new key and value ahead of the round
    // too (LAZY).  In a workgroup of many wavefronts the first one (which starts first) prepares q
    // for all and adds the new token, and takes the last turn at the rounds: the others ask for the
    // keys and values of their first round at once, meet it at a barrier and take q from LDS, so
    // that q's preparation and the keys' way from memory overlap (a decode step of one request
    // 0.385 -> 0.374 ms, of four 0.417 -> 0.406, of 64 0.849 -> 0.843).  Parts of 16 wavefronts were
    // 0.35 us a launch slower that way (8 requests): there every wavefront prepares q for itself.
    constexpr bool LAZY = WAVES == 1;
    constexpr bool SHARED_Q = FRESH && !LAZY && !(SPLIT && WAVES == 16);
    const bool prepares_q = !SHARED_Q || wave == 0;
    const int turn = SHARED_Q ? (wave + WAVES - 1) % WAVES : wave;     // which of the rounds are the wavefront's
    bf16x8_t* const q_share = reinterpret_cast<bf16x8_t*>(smem_heads + static_cast<size_t>(WAVES) * gp * (HD + 2));   // [KS][64]
    bf16x8_t qf[KS];
#pragma unroll
    for (int s = 0; s < KS; ++s) qf[s] = bf16x8_t{};
    if (prepares_q) {
        const bf16* qrow = q + static_cast<size_t>(t) * ldq + static_cast<size_t>(h0 + min(c, gp - 1)) * HD + qd * 8;
#pragma unroll
        for (int s = 0; s < KS; ++s) qf[s] = *reinterpret_cast<const bf16x8_t*>(qrow + s * 32);
    }
    const float* const fresh_cs = FRESH && fresh.cos_sin ? fresh.cos_sin + static_cast<size_t>(pos) * HD : nullptr;
    DecodeHeadOperands<KS> q_operands;
    if (FRESH && prepares_q) decode_head_operands<KS>(q_operands, fresh.q_weight, fresh_cs, qd);
    bool q_ready = !FRESH;
    auto prepare_q = [&]() {
        float x[KS][8];
#pragma unroll
        for (int s = 0; s < KS; ++s)
#pragma unroll
            for (int e = 0; e < 8; ++e) x[s][e] = static_cast<float>(qf[s][e]);
        decode_prepare_head<KS>(x, fresh.q_weight != nullptr, fresh_cs != nullptr, q_operands.w, q_operands.cs, fresh.eps);
#pragma unroll
        for (int s = 0; s < KS; ++s)
#pragma unroll
            for (int e = 0; e < 8; ++e) qf[s][e] = static_cast<__bf16>(x[s][e]);
        q_ready = true;
    };
    // (with a fresh token the rounds end at the position before it)
    const int last_key = FRESH ? pos - 1 : pos;
    float m_run = -INFINITY, l_run = 0.f;
    floatx4_t o[DT];
#pragma unroll
    for (int dt = 0; dt < DT; ++dt) o[dt] = floatx4_t{0.f, 0.f, 0.f, 0.f};

    // the workgroup's rounds: all of the request's, or (SPLIT) part blockIdx.z of them; its
    // wavefronts take them in turn
    // (SPLIT: the request's rounds, from the first of its window to the one of its own position, are
    // shared out evenly over the n_parts workgroups, so that a context well below what the launch was
    // sized for still keeps all of them busy: `per` rounds each, the last parts none)
    const int first_round = lo / DEC_KEYS;
    const int total = pos / DEC_KEYS - first_round + 1, per = SPLIT ? (total + n_parts - 1) / n_parts : 0;
    const int r_begin = SPLIT ? first_round + static_cast<int>(blockIdx.z) * per : first_round;
    const int last_round = last_key < 0 ? -1 : last_key / DEC_KEYS;
    const int r_end = SPLIT ? min(last_round, r_begin + per - 1) : last_round;
    // the fresh token belongs to the part that holds its position (which may hold no other key)
    const bool part_of_fresh = FRESH && (!SPLIT || static_cast<int>(blockIdx.z) == (pos / DEC_KEYS - first_round) / per);
    const bool adds_fresh = part_of_fresh && wave == 0;
    if (SPLIT && r_begin > r_end && !part_of_fresh) return;     // the whole workgroup
    // the new key and value of the wavefront that adds them: asked for ahead of the rounds
    bf16x8_t k_raw[KS];
    bf16x4_t v_raw[DT];
    DecodeHeadOperands<KS> k_operands;
    if (adds_fresh && LAZY) {
        const bf16* krow = fresh.k + static_cast<size_t>(t) * fresh.ldk + static_cast<size_t>(kvh) * HD + qd * 8;
#pragma unroll
        for (int s = 0; s < KS; ++s) k_raw[s] = *reinterpret_cast<const bf16x8_t*>(krow + s * 32);
        const bf16* vrow = fresh.v + static_cast<size_t>(t) * fresh.ldv + static_cast<size_t>(kvh) * HD + 4 * qd;
#pragma unroll
        for (int dt = 0; dt < DT; ++dt) v_raw[dt] = *reinterpret_cast<const bf16x4_t*>(vrow + 16 * dt);
        decode_head_operands<KS>(k_operands, fresh.k_weight, nullptr, qd);
    }
    // The new token as one more key: before the rounds where the wavefront has many (what it
    // needs from memory arrives with q), after its one round otherwise.
    auto add_fresh = [&]() {
        if (!SHARED_Q && !q_ready) prepare_q();    // (a part that holds no other key; where one wavefront prepares q for all it is ready by now)
        if (!LAZY) {
            const bf16* krow = fresh.k + static_cast<size_t>(t) * fresh.ldk + static_cast<size_t>(kvh) * HD + qd * 8;
#pragma unroll
            for (int s = 0; s < KS; ++s) k_raw[s] = *reinterpret_cast<const bf16x8_t*>(krow + s * 32);
            const bf16* vrow = fresh.v + static_cast<size_t>(t) * fresh.ldv + static_cast<size_t>(kvh) * HD + 4 * qd;
#pragma unroll
            for (int dt = 0; dt < DT; ++dt) v_raw[dt] = *reinterpret_cast<const bf16x4_t*>(vrow + 16 * dt);
            decode_head_operands<KS>(k_operands, fresh.k_weight, fresh_cs, qd);
        }
        // the new key in the layout of a query head (every head's lanes prepare it alike)
        float kx[KS][8];
#pragma unroll
        for (int s = 0; s < KS; ++s)
#pragma unroll
            for (int e = 0; e < 8; ++e) kx[s][e] = static_cast<float>(k_raw[s][e]);
        decode_prepare_head<KS>(kx, fresh.k_weight != nullptr, fresh_cs != nullptr, k_operands.w, LAZY ? q_operands.cs : k_operands.cs,
                                fresh.eps);
        const int page = pages[pos >> page_shift];
        const size_t block = kv_block(page, n_layers, layer, kv_heads, kvh, page_tokens, HD);
        float dot = 0.f;
#pragma unroll
        for (int s = 0; s < KS; ++s) {
            bf16x8_t kb16;
#pragma unroll
            for (int e = 0; e < 8; ++e) {
                kb16[e] = static_cast<__bf16>(kx[s][e]);
                dot = fmaf(static_cast<float>(qf[s][e]), static_cast<float>(kb16[e]), dot);
            }
            if (chunk == 0 && c == 0)        // one copy into the page
                *reinterpret_cast<bf16x8_t*>(fresh.k_pool + block + static_cast<size_t>(pos & page_mask) * HD + s * 32 + qd * 8) = kb16;
        }
        dot += __shfl_xor(dot, 16, 64);
        dot += __shfl_xor(dot, 32, 64);
        const float s_new = dot * scale;
        const float m_new = fmaxf(m_run, s_new);
        const float keep = expf(m_run - m_new);         // e^(-inf) = 0 where the part holds no other key
        const float p_exact = expf(s_new - m_new);
        const float p_new = static_cast<float>(static_cast<__bf16>(p_exact));     // as the rounds round theirs for the output
        l_run = l_run * keep + p_exact;
        m_run = m_new;
        // the new value: this lane's dimensions of the output, 16 dt + 4 qd + i
#pragma unroll
        for (int dt = 0; dt < DT; ++dt) {
            const bf16x4_t vv = v_raw[dt];
#pragma unroll
            for (int i = 0; i < 4; ++i) o[dt][i] = o[dt][i] * keep + p_new * static_cast<float>(vv[i]);
            if (chunk == 0 && c == 0) {
#pragma unroll
                for (int i = 0; i < 4; ++i)
                    reinterpret_cast<__bf16*>(fresh.v_pool)[block + static_cast<size_t>(16 * dt + 4 * qd + i) * page_tokens + (pos & page_mask)] = vv[i];
            }
        }
    };
    // One round of 64 keys in two steps: its keys and values asked for (false: the round holds no
    // key: a window of one key with a fresh token), and the arithmetic.
    bf16x8_t kf[4][KS], vf[DT][2];
    auto round_loads = [&](const int r) {
        const int kb = r * DEC_KEYS;
        const int k_lo = max(lo, kb), k_hi = min(last_key, kb + DEC_KEYS - 1);
        if (k_lo > k_hi) return false;
        const int first_page = kb >> page_shift, last_page = k_hi >> page_shift;
        const int my_page = pages[min(first_page + lane, last_page)];
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
        return true;
    };
    auto round_arithmetic = [&](const int r) {
        const int kb = r * DEC_KEYS;
        const int k_lo = max(lo, kb), k_hi = min(last_key, kb + DEC_KEYS - 1);
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
    };
    // after_loads runs once the round's keys and values have been asked for
    auto one_round = [&](const int r, auto&& after_loads) {
        if (!round_loads(r)) return;
        after_loads();
        round_arithmetic(r);
    };
    if constexpr (SHARED_Q) {
        int r = r_begin + turn;
        bool asked = false;
        if (!prepares_q && r <= r_end) asked = round_loads(r);       // on their way while q is prepared
        if (prepares_q) {
            prepare_q();
#pragma unroll
            for (int s = 0; s < KS; ++s) q_share[s * 64 + lane] = qf[s];
        }
        __syncthreads();
        if (!prepares_q) {
#pragma unroll
            for (int s = 0; s < KS; ++s) qf[s] = q_share[s * 64 + lane];
            q_ready = true;
            if (r <= r_end) {
                if (asked) round_arithmetic(r);
                r += WAVES;
            }
        }
        if (adds_fresh) add_fresh();
        for (; r <= r_end; r += WAVES) one_round(r, []() {});
    } else if constexpr (SPLIT && WAVES == 1) {       // a part of one round (more, if the caller gave fewer parts than rounds)
        for (int r = r_begin; r <= r_end; ++r) one_round(r, [&]() { if (FRESH && !q_ready) prepare_q(); });
    } else {
        if (FRESH && !LAZY) prepare_q();               // (every wavefront for itself)
        if (adds_fresh && !LAZY) add_fresh();
        for (int r = r_begin + wave; r <= r_end; r += WAVES) one_round(r, []() {});
    }
    if (adds_fresh && LAZY) add_fresh();
    if (SPLIT && WAVES == 1) {
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
        if (SPLIT) {       // the part's (max, sum, output) for the second kernel
            const size_t idx = (static_cast<size_t>(t) * (kv_heads * group) + h0 + g) * n_splits + blockIdx.z;
            if (d == 0) { ws_ml[2 * idx] = mxw; ws_ml[2 * idx + 1] = denom; }
            ws_o[idx * HD + d] = val;
        } else {
            out[static_cast<size_t>(t) * ldo + static_cast<size_t>(h0 + g) * HD + d] = from_float<bf16>(val / denom);
        }
    }
}

template <int HD, int WAVES>
static int launch_decode_heads(const void* q, int ldq, const void* k_pool, const void* v_pool,
                               const int* table, int table_stride, const int* token_slot,
                               const int* positions, void* out, int ldo, int n_rows, int kv_heads,
                               int group, int page_tokens, int page_shift, int n_layers, int layer,
                               float scale, int window, const DecodeFresh& fresh, hipStream_t stream) {
    const int chunks = (group + 15) / 16;
    // (the wavefronts' partial results, and the prepared q that one of them leaves for the others)
    const size_t lds = static_cast<size_t>(WAVES) * min(group, 16) * (HD + 2) * sizeof(float) + (fresh.k ? HD / 32 * 1024 : 0);
    static bool raised = false;
    if (lds > 48 * 1024 && !raised) {
        hipError_t err = hipFuncSetAttribute(reinterpret_cast<const void*>(&attention_decode_heads_kernel<HD, WAVES, false, false>),
                                             hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024);
        if (err == hipSuccess)
            err = hipFuncSetAttribute(reinterpret_cast<const void*>(&attention_decode_heads_kernel<HD, WAVES, false, true>),
                                      hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024);
        if (err != hipSuccess) return static_cast<int>(err);
        raised = true;
    }
    auto kernel = fresh.k ? &attention_decode_heads_kernel<HD, WAVES, false, true> : &attention_decode_heads_kernel<HD, WAVES, false, false>;
    hipLaunchKernelGGL(kernel, dim3(kv_heads * chunks, n_rows),
                       dim3(WAVES * 64), lds, stream, static_cast<const bf16*>(q),
                       static_cast<const bf16*>(k_pool), static_cast<const bf16*>(v_pool), table,
                       token_slot, positions, ldq, table_stride, static_cast<bf16*>(out), ldo, kv_heads,
                       group, page_tokens, page_shift, n_layers, layer, scale, window, nullptr, nullptr, 0, 1, fresh);
    return CELEG_LAUNCH_RESULT();
}

template <int HD, int WAVES>
static int launch_decode_parts(const void* q, int ldq, const void* k_pool, const void* v_pool,
                               const int* table, int table_stride, const int* token_slot,
                               const int* positions, float* ws_o, float* ws_ml, int n_splits, void* out,
                               int ldo, int n_rows, int kv_heads, int group, int page_tokens,
                               int page_shift, int n_layers, int layer, float scale, int window,
                               int split_rounds, int n_parts, const DecodeFresh& fresh, hipStream_t stream) {
    const int chunks = (group + 15) / 16;
    const size_t lds = WAVES == 1 ? 0 : static_cast<size_t>(WAVES) * min(group, 16) * (HD + 2) * sizeof(float) + (fresh.k ? HD / 32 * 1024 : 0);
    static bool raised = false;
    if (lds > 48 * 1024 && !raised) {
        hipError_t err = hipFuncSetAttribute(reinterpret_cast<const void*>(&attention_decode_heads_kernel<HD, WAVES, true, false>),
                                             hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024);
        if (err == hipSuccess)
            err = hipFuncSetAttribute(reinterpret_cast<const void*>(&attention_decode_heads_kernel<HD, WAVES, true, true>),
                                      hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024);
        if (err != hipSuccess) return static_cast<int>(err);
        raised = true;
    }
    auto kernel = fresh.k ? &attention_decode_heads_kernel<HD, WAVES, true, true> : &attention_decode_heads_kernel<HD, WAVES, true, false>;
    hipLaunchKernelGGL(kernel, dim3(kv_heads * chunks, n_rows, n_parts),
                       dim3(WAVES * 64), lds, stream, static_cast<const bf16*>(q),
                       static_cast<const bf16*>(k_pool), static_cast<const bf16*>(v_pool), table,
                       token_slot, positions, ldq, table_stride, static_cast<bf16*>(out), ldo, kv_heads,
                       group, page_tokens, page_shift, n_layers, layer, scale, window, ws_o, ws_ml,
                       n_splits, n_parts, fresh);
    return 0;
}

static int attention_decode(
    const void* q, int ldq, const void* k_pool, const void* v_pool, const int* table,
    int table_stride, const int* token_slot, const int* positions, float* ws_o, float* ws_ml,
    int n_splits, void* out, int ldo, int n_rows, int q_heads, int kv_heads,
    int head_dim, int page_tokens, int n_layers, int layer, float scale, int window, int whole,
    int split_rounds, int n_parts, const DecodeFresh& fresh, hipStream_t stream) {
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
        // 16 wavefronts a workgroup (what the registers of a compute unit hold at this head size),
        // 8 once there are more workgroups than compute units: two of them then share a compute unit
        // where workgroups of 16 would take a second round (64 requests x 8 heads: 4 to 6 % faster at
        // contexts of 1,000 to 4,000; 36 to 60 requests: 1.2 to 2 % of a decode step; equal at 32 requests)
        if (head_dim == 64 && kv_heads * chunks * n_rows > 256)
            return launch_decode_heads<64, 8>(q, ldq, k_pool, v_pool, table, table_stride, token_slot, positions,
                                              out, ldo, n_rows, kv_heads, group, page_tokens, page_shift,
                                              n_layers, layer, scale, window, fresh, stream);
        if (head_dim == 64)
            return launch_decode_heads<64, 16>(q, ldq, k_pool, v_pool, table, table_stride, token_slot, positions,
                                           out, ldo, n_rows, kv_heads, group, page_tokens, page_shift,
                                           n_layers, layer, scale, window, fresh, stream);
        if (head_dim == 128)
            return launch_decode_heads<128, 8>(q, ldq, k_pool, v_pool, table, table_stride, token_slot, positions,
                                            out, ldo, n_rows, kv_heads, group, page_tokens, page_shift,
                                            n_layers, layer, scale, window, fresh, stream);
        return static_cast<int>(hipErrorInvalidValue);
    }
    // n_parts workgroups per request and key/value head, of 1, 4 or 16 wavefronts (split_rounds; 8
    // at most for heads of 128) that take a round of 64 keys each at a time: the caller chooses both
    // so that n_parts * split_rounds * 64 keys cover the longest context the launch is meant for, and
    // a longer context gets longer parts instead of more of them.  A request's rounds are shared
    // out evenly over its workgroups, whatever its context.
    if ((split_rounds != 1 && split_rounds != 4 && split_rounds != 16) || n_parts <= 0 || n_parts > n_splits)
        return static_cast<int>(hipErrorInvalidValue);
#define CELEG_SPLIT_ARGS                                                                           \
    q, ldq, k_pool, v_pool, table, table_stride, token_slot, positions, ws_o, ws_ml, n_splits, out, \
        ldo, n_rows, kv_heads, group, page_tokens, page_shift, n_layers, layer, scale, window,     \
        split_rounds, n_parts, fresh, stream
#define CELEG_SPLIT_HEADS(HD_, MOST_)                                                              \
    {                                                                                              \
        const int code = split_rounds == 1 ? launch_decode_parts<HD_, 1>(CELEG_SPLIT_ARGS)         \
                         : split_rounds == 4 ? launch_decode_parts<HD_, 4>(CELEG_SPLIT_ARGS)       \
                                             : launch_decode_parts<HD_, MOST_>(CELEG_SPLIT_ARGS);  \
        if (code) return code;                                                                     \
    }                                                                                              \
    hipLaunchKernelGGL(attention_decode_reduce_kernel<HD_>, dim3(q_heads, n_rows), dim3(64), 0,   \
                       stream, ws_o, ws_ml, positions, static_cast<bf16*>(out), ldo, q_heads,     \
                       n_splits, window, n_parts)
    if (head_dim == 64) { CELEG_SPLIT_HEADS(64, 16); }
    else if (head_dim == 128) { CELEG_SPLIT_HEADS(128, 8); }
    else return static_cast<int>(hipErrorInvalidValue);
#undef CELEG_SPLIT_ARGS
#undef CELEG_SPLIT_HEADS
    return CELEG_LAUNCH_RESULT();
}

extern "C" int celeg_attention_decode_bf16(
    const void* q, int ldq, const void* k_pool, const void* v_pool, const int* table,
    int table_stride, const int* token_slot, const int* positions, float* ws_o, float* ws_ml,
    int n_splits, void* out, int ldo, int n_rows, int q_heads, int kv_heads,
    int head_dim, int page_tokens, int n_layers, int layer, float scale, int window, int whole,
    int split_rounds, int n_parts, hipStream_t stream) {
    return attention_decode(q, ldq, k_pool, v_pool, table, table_stride, token_slot, positions, ws_o, ws_ml, n_splits, out,
                            ldo, n_rows, q_heads, kv_heads, head_dim, page_tokens, n_layers, layer, scale, window, whole,
                            split_rounds, n_parts, DecodeFresh{}, stream);
}

// The same for a step whose own keys and values are not in the cache yet: q, k and v as the
// q/k/v product left them ([rows, ld..]); the kernel normalises (weights of head_dim 32-bit
// values, or null) and turns (cos_sin [positions, head_dim / 2, 2], or null) the query heads
// and the new key itself and writes the new key and value into the pages (DecodeFresh).
extern "C" int celeg_attention_decode_fresh_bf16(
    const void* q, int ldq, const void* k, int ldk, const void* v, int ldv, const float* q_weight,
    const float* k_weight, float eps, const float* cos_sin, void* k_pool, void* v_pool, const int* table,
    int table_stride, const int* token_slot, const int* positions, float* ws_o, float* ws_ml,
    int n_splits, void* out, int ldo, int n_rows, int q_heads, int kv_heads,
    int head_dim, int page_tokens, int n_layers, int layer, float scale, int window, int whole,
    int split_rounds, int n_parts, hipStream_t stream) {
    const auto misaligned = [](const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15) != 0; };
    if (!k || !v || (ldk % 8) || (ldv % 4) || misaligned(k) || (reinterpret_cast<uintptr_t>(v) & 7) || misaligned(q_weight) ||
        misaligned(k_weight) || misaligned(cos_sin) || misaligned(k_pool))
        return static_cast<int>(hipErrorInvalidValue);
    DecodeFresh fresh{};
    fresh.k = static_cast<const bf16*>(k);
    fresh.v = static_cast<const bf16*>(v);
    fresh.ldk = ldk;
    fresh.ldv = ldv;
    fresh.q_weight = q_weight;
    fresh.k_weight = k_weight;
    fresh.eps = eps;
    fresh.cos_sin = cos_sin;
    fresh.k_pool = static_cast<bf16*>(k_pool);
    fresh.v_pool = static_cast<bf16*>(v_pool);
    return attention_decode(q, ldq, k_pool, v_pool, table, table_stride, token_slot, positions, ws_o, ws_ml, n_splits, out,
                            ldo, n_rows, q_heads, kv_heads, head_dim, page_tokens, n_layers, layer, scale, window, whole,
                            split_rounds, n_parts, fresh, stream);
}

// ================================================================ without allocation
// (declared in no_alloc.h: no counterpart in the reference; for callers that cannot allocate)
static __device__ __align__(256) float scratch[CELEG_NO_ALLOC_SCRATCH_BYTES / sizeof(float)];

namespace {
constexpr int NO_ALLOC_MAX_DEVICES = 64;
float* scratch_of_device[NO_ALLOC_MAX_DEVICES];     // the array's address on each device, once looked up
std::mutex scratch_lock;

// The address of `scratch` on the current device.  In host code the array's name is only a
// handle for hipGetSymbolAddress; kernels and copies get the address it returns.
int scratch_address(float** ptr) {
    int device = 0;
    hipError_t err = hipGetDevice(&device);
    if (err != hipSuccess) return static_cast<int>(err);
    if (device < 0 || device >= NO_ALLOC_MAX_DEVICES) return static_cast<int>(hipErrorInvalidDevice);
    std::lock_guard<std::mutex> guard(scratch_lock);
    if (scratch_of_device[device] == nullptr) {
        void* address = nullptr;
        err = hipGetSymbolAddress(&address, HIP_SYMBOL(scratch));
        if (err != hipSuccess) return static_cast<int>(err);
        if (address == nullptr) return static_cast<int>(hipErrorInvalidSymbol);
        scratch_of_device[device] = static_cast<float*>(address);
    }
    *ptr = scratch_of_device[device];
    return 0;
}
}  // namespace

extern "C" int celeg_attention_decode_no_alloc_init(void) {
    float* ptr = nullptr;
    return scratch_address(&ptr);
}

extern "C" int celeg_attention_decode_bf16_no_alloc(
    const void* q, int ldq, const void* k_pool, const void* v_pool, const int* table,
    int table_stride, const int* token_slot, const int* positions, void* out, int ldo,
    int n_rows, int q_heads, int kv_heads, int head_dim, int page_tokens, int n_layers, int layer,
    float scale, int window, int split_rounds, int n_parts, hipStream_t stream) {
    if (n_rows <= 0) return 0;
    if (q_heads <= 0 || kv_heads <= 0 || n_parts <= 0 || (head_dim != 64 && head_dim != 128))
        return static_cast<int>(hipErrorInvalidValue);
    // partial outputs [rows, heads, parts, head_dim] then (maximum, sum) [rows, heads, parts, 2]
    const unsigned long long parts = static_cast<unsigned long long>(n_rows) * q_heads * n_parts;
    if (parts * (head_dim + 2) > CELEG_NO_ALLOC_SCRATCH_BYTES / sizeof(float))
        return static_cast<int>(hipErrorInvalidValue);
    float* ws = nullptr;
    const int code = scratch_address(&ws);
    if (code) return code;
    return celeg_attention_decode_bf16(q, ldq, k_pool, v_pool, table, table_stride, token_slot, positions,
                                       ws, ws + parts * head_dim, n_parts, out, ldo, n_rows, q_heads,
                                       kv_heads, head_dim, page_tokens, n_layers, layer, scale, window,
                                       /*whole=*/0, split_rounds, n_parts, stream);
}
