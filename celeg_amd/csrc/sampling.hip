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
#define SAMPLE_HIST_COPIES 16
typedef float floatx4_t __attribute__((ext_vector_type(4)));

__device__ __forceinline__ bool better(float sa, int ia, float sb, int ib) {
    return sa == sb ? ia < ib : sa > sb;
}

// Walks a row of logits: f(penalised value, index) for this thread's share, groups of 4
// logits, 8 groups of a thread asked for before any is looked at (a row of 65,536 logits is
// then two round trips to memory instead of 64).  A thread's indices come in rising order.
template <typename F>
__device__ __forceinline__ void for_each_logit(const float* __restrict__ row,
                                               const uint8_t* __restrict__ seen, float penalty,
                                               int vocab, int tid, F f) {
    const bool pen = seen && penalty > 1.0f;
    const bool vec = (reinterpret_cast<uintptr_t>(row) & 15) == 0 &&
                     (!pen || (reinterpret_cast<uintptr_t>(seen) & 3) == 0);
    const int n4 = vec ? vocab >> 2 : 0;
    auto take = [&](float v, unsigned seen_byte, int i) {
        if (seen_byte) v = v >= 0.0f ? v / penalty : v * penalty;
        f(v, i);
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
}

__device__ __forceinline__ float key_score(uint32_t key) {      // the inverse of order_key
    return __uint_as_float((key & 0x80000000u) ? (key & 0x7fffffffu) : ~key);
}

// The top_k scores of a row (score = penalised logit / temperature) by (score desc, id
// asc), left unordered in cand_score / cand_id [0, top_k).  All threads of the workgroup
// call it.  KPT > 0: the row's keys are held in registers, KPT a thread, element
// tid + SAMPLE_THREADS * j in place j (vocab <= SAMPLE_THREADS * KPT); KPT == 0: every pass
// walks the row in memory.
template <int KPT>
__device__ __forceinline__ void top_k_candidates(
    const float* __restrict__ row, const uint8_t* __restrict__ seen, float penalty, float temperature,
    int vocab, int top_k, unsigned int* hist, unsigned int* sel, int* running, float* cand_score,
    int* cand_id) {
    const int tid = threadIdx.x;
    const int lane = tid & (CELEG_WAVE - 1);
    constexpr int NK = KPT > 0 ? KPT : 1;
    uint32_t keys[NK];
    if (KPT > 0) {
        const bool pen = seen && penalty > 1.0f;
        float v[NK];
        unsigned char sn[NK];
#pragma unroll
        for (int j = 0; j < NK; ++j) {
            const int i = min(tid + SAMPLE_THREADS * j, vocab - 1);      // clamped, masked below
            v[j] = row[i];
            sn[j] = pen ? seen[i] : 0;
        }
#pragma unroll
        for (int j = 0; j < NK; ++j) {
            float x = v[j];
            if (sn[j]) x = x >= 0.0f ? x / penalty : x * penalty;
            keys[j] = tid + SAMPLE_THREADS * j < vocab ? order_key(x / temperature) : 0u;
        }
    }
    // f(key, index) for this thread's share of the row
    auto walk = [&](auto f) {
        if (KPT > 0) {
#pragma unroll
            for (int j = 0; j < NK; ++j)
                if (tid + SAMPLE_THREADS * j < vocab) f(keys[j], tid + SAMPLE_THREADS * j);
        } else {
            for_each_logit(row, seen, penalty, vocab, tid,
                           [&](float x, int i) { f(order_key(x / temperature), i); });
        }
    };
    // One counting pass: bins of bin_of(key, index) >= 0.  The counts go to
    // SAMPLE_HIST_COPIES copies of the 256 bins, a lane using copy lane % copies: scores
    // crowd into a few bins of the top byte, and lanes that hit one address take turns.
    auto count_pass = [&](auto bin_of) {
        for (int i = tid; i < 256 * SAMPLE_HIST_COPIES; i += SAMPLE_THREADS) hist[i] = 0u;
        __syncthreads();
        unsigned int* mine = hist + (lane % SAMPLE_HIST_COPIES) * 256;
        walk([&](uint32_t key, int i) {
            const int bin = bin_of(key, i);
            if (bin >= 0) atomicAdd(&mine[bin], 1u);
        });
        __syncthreads();
        if (tid < 256) {
            unsigned int total = 0u;
#pragma unroll
            for (int c = 0; c < SAMPLE_HIST_COPIES; ++c) total += hist[c * 256 + tid];
            hist[tid] = total;
        }
        __syncthreads();
    };
    // after a pass: the bin in which the sought place lies, counted from the top (largest
    // first) or from the bottom; sel = {prefix so far, places still to go, size of that bin}
    auto choose_bin = [&](int shift, bool from_top) {
        if (tid < CELEG_WAVE) {       // one wavefront: lane l takes the l-th four bins of the walk
            const unsigned int remaining = sel[1];
            unsigned int c[4], mine = 0u;
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                const int pos = 4 * lane + e;
                c[e] = hist[from_top ? 255 - pos : pos];
                mine += c[e];
            }
            unsigned int before = mine;      // inclusive sum over the lanes in front, then exclusive
#pragma unroll
            for (int off = 1; off < CELEG_WAVE; off <<= 1) {
                const unsigned int o = __shfl_up(before, off, CELEG_WAVE);
                if (lane >= off) before += o;
            }
            before -= mine;
            // the first place of the walk at which the running count reaches what is sought;
            // if none does (it cannot, the counts add up to at least that), the last bin
            const bool here = before < remaining && before + mine >= remaining;
            const unsigned long long found = __ballot(here);
            const int owner = found ? __ffsll(static_cast<long long>(found)) - 1 : CELEG_WAVE - 1;
            if (lane == owner) {
                unsigned int passed = before;
                int e = 0;
                for (; e < 3; ++e) {
                    if (passed + c[e] >= remaining) break;
                    passed += c[e];
                }
                const int pos = 4 * lane + e;
                const int bin = from_top ? 255 - pos : pos;
                sel[0] |= static_cast<unsigned>(bin) << shift;
                sel[1] = remaining - passed;
                sel[2] = c[e];
            }
        }
        __syncthreads();
    };

    // ---- a bound from below first, so that few scores take part in the counting: every
    // thread's largest score is a score of its own, so the top_k-th largest of these maxima is
    // not above the top_k-th largest score overall.  Found by the same selection (8 bits a
    // pass, from the top), one count a thread a pass.
    uint32_t my_max = 0u;
    walk([&](uint32_t key, int) { my_max = max(my_max, key); });
    if (tid == 0) { sel[0] = 0u; sel[1] = static_cast<unsigned>(top_k); }
    __syncthreads();
    unsigned int mask = 0u;
    for (int shift = 24; shift >= 0; shift -= 8) {
        const unsigned int prefix = sel[0];
        for (int i = tid; i < 256; i += SAMPLE_THREADS) hist[i] = 0u;
        __syncthreads();
        if ((my_max & mask) == prefix) atomicAdd(&hist[(my_max >> shift) & 255u], 1u);
        __syncthreads();
        choose_bin(shift, true);
        mask |= 255u << shift;
    }
    const uint32_t lower = sel[0];
    __syncthreads();

    // ---- the top_k-th largest score itself
    if (tid == 0) { sel[0] = 0u; sel[1] = static_cast<unsigned>(top_k); }
    __syncthreads();
    mask = 0u;
    for (int shift = 24; shift >= 0; shift -= 8) {
        const unsigned int prefix = sel[0];
        count_pass([&](uint32_t key, int) {
            return (key >= lower && (key & mask) == prefix) ? static_cast<int>((key >> shift) & 255u) : -1;
        });
        choose_bin(shift, true);
        mask |= 255u << shift;
    }
    const uint32_t kth = sel[0];
    const int need_eq = static_cast<int>(sel[1]);  // how many of the ties at the threshold to take
    const int n_eq = static_cast<int>(sel[2]);     // how many scores equal the threshold
    const int n_gt = top_k - need_eq;
    __syncthreads();

    // ---- of the ties at the threshold the lowest ids are taken: if not all of them, the
    // need_eq-th lowest id is found the same way (ids rising, 8 bits a pass)
    int last_tie = 0x7fffffff;
    if (need_eq < n_eq) {
        if (tid == 0) { sel[0] = 0u; sel[1] = static_cast<unsigned>(need_eq); }
        __syncthreads();
        unsigned int imask = 0u;
        for (int shift = 24; shift >= 0; shift -= 8) {
            const unsigned int prefix = sel[0];
            count_pass([&](uint32_t key, int i) {
                return (key == kth && (static_cast<unsigned>(i) & imask) == prefix)
                           ? static_cast<int>((static_cast<unsigned>(i) >> shift) & 255u) : -1;
            });
            choose_bin(shift, false);
            imask |= 255u << shift;
        }
        last_tie = static_cast<int>(sel[0]);
        __syncthreads();
    }

    // ---- the candidates, in any order (the caller sorts them)
    if (tid == 0) { running[0] = 0; running[1] = 0; }
    __syncthreads();
    walk([&](uint32_t key, int i) {
        if (key > kth) {
            const int p = atomicAdd(&running[0], 1);
            if (p < n_gt) { cand_score[p] = key_score(key); cand_id[p] = i; }
        } else if (key == kth && i <= last_tie) {
            const int e = atomicAdd(&running[1], 1);
            if (e < need_eq) { cand_score[n_gt + e] = key_score(key); cand_id[n_gt + e] = i; }
        }
    });
    __syncthreads();
}

// The same candidates by ranking, for rows whose logits fit in registers, already in the
// order (score desc, id asc); false (nothing written) if more logits than SAMPLE_RANK_CAP
// reach the bound from below, as when very many are equal: the caller then selects by
// counting passes as above.
//   1. Every thread keeps its logits as ordered keys of a cheap stand-in for the score
//      (the penalty applied by multiplication, no division by the temperature: the same
//      order up to a unit or two in the last place) and finds its largest.
//   2. A bound from below: with c = ceil(top_k / 16), the c-th largest thread maximum of
//      each of the 16 wavefronts; at least 16 c >= top_k logits reach the smallest of these
//      16 values, so the top_k-th largest stand-in does too.  Eight units in the last place
//      are taken off, which covers what the stand-in can differ from the score by.
//   3. The logits at or above the bound (two or three times top_k of them as a rule) are
//      gathered; their exact scores are computed as the reference does (true divisions), and
//      a thread per such logit counts the ones that come before it: that is its place.
// Five workgroup barriers instead of about forty, and two divisions per gathered logit
// instead of per logit.
#define SAMPLE_RANK_CAP 2048
__device__ __forceinline__ void rank_gathered(const float* __restrict__ row, const uint8_t* __restrict__ seen, bool pen,
                                              float penalty, float temperature, int top_k, int n, uint2* gathered,
                                              float* cand_score, int* cand_id);
template <int KPT>
__device__ __forceinline__ bool top_k_ranked(
    const float* __restrict__ row, const uint8_t* __restrict__ seen, float penalty, float temperature,
    int vocab, int top_k, uint32_t* wave_bound, uint2* gathered, unsigned int* sel, float* cand_score,
    int* cand_id) {
    const int tid = threadIdx.x;
    const int lane = tid & (CELEG_WAVE - 1), wave = tid / CELEG_WAVE;
    const bool pen = seen && penalty > 1.0f;
    const float inv_penalty = 1.0f / penalty;
    // Place j of a thread holds element tid + SAMPLE_THREADS * j, or, where the row can be read 16
    // bytes a lane (and the seen marks 4), element 4 * (tid + SAMPLE_THREADS * (j / 4)) + j % 4: a
    // load of one logit or one mark a lane costs the vector cache as much as one of four (a row of
    // 65,536 logits with its marks: 2,048 loads of a wavefront instead of 512).
    const bool by_fours = (vocab & 3) == 0 && (reinterpret_cast<uintptr_t>(row) & 15) == 0 &&
                          (!pen || (reinterpret_cast<uintptr_t>(seen) & 3) == 0);
    auto index_of = [&](int j) { return by_fours ? 4 * (tid + SAMPLE_THREADS * (j >> 2)) + (j & 3) : tid + SAMPLE_THREADS * j; };
    uint32_t keys[KPT];
    if (by_fours) {
        floatx4_t v[KPT / 4];
        unsigned sn[KPT / 4];
        const int n4 = vocab >> 2;
#pragma unroll
        for (int jj = 0; jj < KPT / 4; ++jj) {
            const int g = min(tid + SAMPLE_THREADS * jj, n4 - 1);       // clamped, masked below
            v[jj] = reinterpret_cast<const floatx4_t*>(row)[g];
            sn[jj] = pen ? reinterpret_cast<const unsigned*>(seen)[g] : 0u;
        }
#pragma unroll
        for (int jj = 0; jj < KPT / 4; ++jj)
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                const float x0 = v[jj][e];
                const float x = ((sn[jj] >> (8 * e)) & 0xffu) ? (x0 >= 0.0f ? x0 * inv_penalty : x0 * penalty) : x0;
                keys[4 * jj + e] = tid + SAMPLE_THREADS * jj < n4 ? order_key(x) : 0u;
            }
    } else {
        float v[KPT];
        unsigned char sn[KPT];
#pragma unroll
        for (int j = 0; j < KPT; ++j) {
            const int i = min(tid + SAMPLE_THREADS * j, vocab - 1);      // clamped, masked below
            v[j] = row[i];
            sn[j] = pen ? seen[i] : 0;
        }
#pragma unroll
        for (int j = 0; j < KPT; ++j) {
            const float x = sn[j] ? (v[j] >= 0.0f ? v[j] * inv_penalty : v[j] * penalty) : v[j];
            keys[j] = tid + SAMPLE_THREADS * j < vocab ? order_key(x) : 0u;
        }
    }
    uint32_t my_max = 0u;
#pragma unroll
    for (int j = 0; j < KPT; ++j) my_max = max(my_max, keys[j]);
    // the c-th largest maximum of this wavefront: c times the largest, one lane struck out each time
    const int c = (top_k + SAMPLE_THREADS / CELEG_WAVE - 1) / (SAMPLE_THREADS / CELEG_WAVE);
    uint32_t left = my_max, cth = 0u;
    for (int round = 0; round < c; ++round) {
        uint32_t m = left;
#pragma unroll
        for (int off = CELEG_WAVE / 2; off > 0; off >>= 1)
            m = max(m, static_cast<uint32_t>(__shfl_xor(static_cast<int>(m), off, CELEG_WAVE)));
        cth = m;
        const unsigned long long holders = __ballot(left == m);
        if (lane == __ffsll(static_cast<long long>(holders)) - 1) left = 0u;
    }
    if (lane == 0) wave_bound[wave] = cth;
    if (tid == 0) { sel[0] = 0u; sel[1] = 0u; }
    __syncthreads();
    uint32_t lower = wave_bound[0];
#pragma unroll
    for (int w = 1; w < SAMPLE_THREADS / CELEG_WAVE; ++w) lower = min(lower, wave_bound[w]);
    lower = lower > 8u ? lower - 8u : 0u;
#pragma unroll
    for (int j = 0; j < KPT; ++j)
        if (index_of(j) < vocab && keys[j] >= lower) {
            const unsigned int p = atomicAdd(&sel[1], 1u);
            if (p < SAMPLE_RANK_CAP) gathered[p].y = static_cast<unsigned>(index_of(j));
        }
    __syncthreads();
    const int n = static_cast<int>(sel[1]);
    if (n > SAMPLE_RANK_CAP) return false;       // the same for every thread
    rank_gathered(row, seen, pen, penalty, temperature, top_k, n, gathered, cand_score, cand_id);
    return true;
}

// The last steps of the ranking: the exact scores of the n gathered logits (gathered[e].y: their
// indices), as the reference computes them, and every one's place among them; the first top_k places
// go to cand_score / cand_id.  All threads call it; n is the same for all.
__device__ __forceinline__ void rank_gathered(const float* __restrict__ row, const uint8_t* __restrict__ seen, bool pen,
                                              float penalty, float temperature, int top_k, int n, uint2* gathered,
                                              float* cand_score, int* cand_id) {
    const int tid = threadIdx.x;
    for (int e = tid; e < n; e += SAMPLE_THREADS) {
        const int id = static_cast<int>(gathered[e].y);
        float x = row[id];
        if (pen && seen[id]) x = x >= 0.0f ? x / penalty : x * penalty;
        gathered[e].x = __float_as_uint(x / temperature);
    }
    __syncthreads();
    for (int e = tid; e < n; e += SAMPLE_THREADS) {
        const uint2 mine = gathered[e];
        const float score = __uint_as_float(mine.x);
        const int id = static_cast<int>(mine.y);
        int place = 0;
        for (int u0 = 0; u0 < n; u0 += 16) {            // sixteen reads from LDS under way at a time
            uint2 other[16];
#pragma unroll
            for (int j = 0; j < 16; ++j) other[j] = gathered[min(u0 + j, n - 1)];
#pragma unroll
            for (int j = 0; j < 16; ++j)
                place += (u0 + j < n && better(__uint_as_float(other[j].x), static_cast<int>(other[j].y), score, id)) ? 1 : 0;
        }
        if (place < top_k) { cand_score[place] = score; cand_id[place] = id; }
    }
    __syncthreads();
}

// The same candidates without reading the row: an output head left, beside the logits, the best
// (logit, index) of every `cols` columns (best[p]: part p of this row, packed as packed_logit
// packs them).  A penalised logit is never above the logit itself, so:
//   1. every thread takes up to SAMPLE_PARTS_PER_THREAD parts' maxima; the c-th largest thread maximum
//      of each wavefront, c = ceil(top_k / 16), bounds the top_k-th largest maximum from below as in
//      top_k_ranked; the threads whose maximum reaches it (top_k different logits at least) apply the
//      penalty to theirs, and the smallest of these penalised values, less eight units in the last
//      place, is a bound from below for the top_k-th largest penalised logit;
//   2. only parts whose maximum reaches that bound can hold a logit that does: their columns are read
//      (a few hundred logits instead of the row), and what reaches the bound is gathered and ranked
//      as in top_k_ranked.
// false (nothing written that matters) if the parts are too many for the threads, too few to bound
// anything, or more parts or logits reach the bound than there is room for: the caller then reads the row.
#define SAMPLE_PARTS_PER_THREAD 4
#define SAMPLE_PART_LIST 1024
__device__ __forceinline__ bool top_k_from_parts(
    const float* __restrict__ row, const uint8_t* __restrict__ seen, float penalty, float temperature, int vocab, int top_k,
    const unsigned long long* __restrict__ best, int n_parts, int cols, uint32_t* wave_bound, uint2* gathered,
    unsigned int* sel, unsigned int* part_list, float* cand_score, int* cand_id) {
    const int tid = threadIdx.x;
    const int lane = tid & (CELEG_WAVE - 1), wave = tid / CELEG_WAVE;
    if (n_parts > SAMPLE_THREADS * SAMPLE_PARTS_PER_THREAD || cols <= 0) return false;
    const bool pen = seen && penalty > 1.0f;
    const float inv_penalty = 1.0f / penalty;
    auto stand_in = [&](float x, unsigned seen_byte) { return seen_byte ? (x >= 0.0f ? x * inv_penalty : x * penalty) : x; };
    uint32_t part_key[SAMPLE_PARTS_PER_THREAD];
    unsigned long long my_best = 0ull;
    {
        unsigned long long v[SAMPLE_PARTS_PER_THREAD];
#pragma unroll
        for (int j = 0; j < SAMPLE_PARTS_PER_THREAD; ++j)
            v[j] = best[min(tid + SAMPLE_THREADS * j, n_parts - 1)];     // clamped, masked below
#pragma unroll
        for (int j = 0; j < SAMPLE_PARTS_PER_THREAD; ++j) {
            const bool valid = tid + SAMPLE_THREADS * j < n_parts;
            part_key[j] = valid ? static_cast<uint32_t>(v[j] >> 32) : 0u;
            my_best = valid ? max(my_best, v[j]) : my_best;
        }
    }
    const uint32_t my_max = static_cast<uint32_t>(my_best >> 32);
    const int c = (top_k + SAMPLE_THREADS / CELEG_WAVE - 1) / (SAMPLE_THREADS / CELEG_WAVE);
    uint32_t left = my_max, cth = 0u;
    for (int round = 0; round < c; ++round) {
        uint32_t m = left;
#pragma unroll
        for (int off = CELEG_WAVE / 2; off > 0; off >>= 1)
            m = max(m, static_cast<uint32_t>(__shfl_xor(static_cast<int>(m), off, CELEG_WAVE)));
        cth = m;
        const unsigned long long holders = __ballot(left == m);
        if (lane == __ffsll(static_cast<long long>(holders)) - 1) left = 0u;
    }
    if (lane == 0) wave_bound[wave] = cth;
    if (tid == 0) { sel[0] = 0u; sel[1] = 0u; sel[2] = 0xffffffffu; }
    __syncthreads();
    uint32_t lower_max = wave_bound[0];
#pragma unroll
    for (int w = 1; w < SAMPLE_THREADS / CELEG_WAVE; ++w) lower_max = min(lower_max, wave_bound[w]);
    if (lower_max == 0u) return false;           // (some wavefront has fewer than c parts: nothing is bounded)
    if (my_max >= lower_max) {
        // this thread's best logit is one of top_k different logits at least: its penalised value
        const int index = packed_logit_index(my_best);
        const float x = stand_in(key_score(my_max), pen ? seen[index] : 0u);
        atomicMin(&sel[2], order_key(x));
    }
    __syncthreads();
    const uint32_t lowest = sel[2];
    const uint32_t lower = lowest > 8u ? lowest - 8u : 0u;
#pragma unroll
    for (int j = 0; j < SAMPLE_PARTS_PER_THREAD; ++j)
        if (tid + SAMPLE_THREADS * j < n_parts && part_key[j] >= lower) {
            const unsigned int p = atomicAdd(&sel[0], 1u);
            if (p < SAMPLE_PART_LIST) part_list[p] = static_cast<unsigned>(tid + SAMPLE_THREADS * j);
        }
    __syncthreads();
    const int n_listed = static_cast<int>(sel[0]);
    if (n_listed > SAMPLE_PART_LIST) return false;
    for (int e = tid; e < n_listed * cols; e += SAMPLE_THREADS) {
        const int i = static_cast<int>(part_list[e / cols]) * cols + e % cols;
        if (i < vocab) {
            const float x = stand_in(row[i], pen ? seen[i] : 0u);
            if (order_key(x) >= lower) {
                const unsigned int p = atomicAdd(&sel[1], 1u);
                if (p < SAMPLE_RANK_CAP) gathered[p].y = static_cast<unsigned>(i);
            }
        }
    }
    __syncthreads();
    const int n = static_cast<int>(sel[1]);
    if (n > SAMPLE_RANK_CAP || n < top_k) return false;
    rank_gathered(row, seen, pen, penalty, temperature, top_k, n, gathered, cand_score, cand_id);
    return true;
}

// What one wavefront does with the candidates (cand_score / cand_id [0, SAMPLE_MAX_K) in LDS, the
// places from top_k on holding (-inf, max id)): sorts them by (score desc, id asc) unless they
// came so, then softmax, the top-p prefix and the walk with the draw u.  Returns the token
// (the same value in every lane).
__device__ __forceinline__ int choose_among(float* cand_score, int* cand_id, int top_k, float top_p, float u,
                                            bool sorted, int lane) {
    // ---- bitonic sort of 128 candidates by (score desc, id asc), unless they came in that
    // order: lane l owns the pair whose lower member is the l-th position with the stride's bit clear
    for (int size = sorted ? 2 * SAMPLE_MAX_K : 2; size <= SAMPLE_MAX_K; size <<= 1) {
        for (int stride = size >> 1; stride > 0; stride >>= 1) {
            const int a = ((lane & ~(stride - 1)) << 1) | (lane & (stride - 1));
            const int partner = a | stride;
            const bool ascending_block = (a & size) == 0;  // "best first" blocks
            const float sa = cand_score[a], sb = cand_score[partner];
            const int ia = cand_id[a], ib = cand_id[partner];
            const bool a_first = better(sa, ia, sb, ib);
            if (ascending_block ? !a_first : a_first) {
                cand_score[a] = sb; cand_id[a] = ib;
                cand_score[partner] = sa; cand_id[partner] = ia;
            }
            __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
            __builtin_amdgcn_wave_barrier();
            __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
        }
    }

    // ---- softmax, top-p prefix and the walk.  The sums run over the candidates one after
    // the other, in the reference's order: every lane runs the same loops over the values in
    // LDS (reads of one address by all lanes, asked for ahead of the additions that need them;
    // a value handed from lane to lane for every addition cost ten times the addition).
    const float maximum = cand_score[0];
    const int id0 = cand_id[lane], id1 = cand_id[lane + 64];
    const float e0 = expf(cand_score[lane] - maximum), e1 = expf(cand_score[lane + 64] - maximum);
    auto wave_sync = [] {
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
    };
    wave_sync();                       // every lane has read the scores it needs
    float* const prob = cand_score;    // from here on the array holds exp(score - max), then the probabilities
    prob[lane] = e0;
    prob[lane + 64] = e1;
    wave_sync();
    float total = 0.f;
    for (int i = 0; i < top_k; ++i) total += prob[i];
    wave_sync();
    prob[lane] = e0 / total;
    prob[lane + 64] = e1 / total;
    wave_sync();
    int active = top_k;
    if (top_p < 1.0f) {
        float cumulative = 0.f;
        active = 0;
        do {
            cumulative += prob[active++];
        } while (active < top_k && cumulative < top_p);
        total = 0.f;
        for (int i = 0; i < active; ++i) total += prob[i];
    } else {
        total = 1.0f;
    }
    float target = u * total;
    int chosen_at = active - 1;
    for (int i = 0; i < active; ++i) {
        target -= prob[i];
        if (target <= 0.0f) { chosen_at = i; break; }
    }
    return __shfl(chosen_at < 64 ? id0 : id1, chosen_at & 63, CELEG_WAVE);
}

// fparams[row] = {temperature, top_p, penalty, u}; iparams[row] = {top_k (or -(token + 1): that
// token is given out, nothing is chosen), seen_row or -1, slot or -1}; the token also goes to last_tokens[slot] (if given and slot >= 0), where the
// next step can take it from without the host in between, and is marked as seen in the row's
// seen_row (if any): the step that feeds it back need not mark it.
__global__ __launch_bounds__(SAMPLE_THREADS) void sample_kernel(
    const float* __restrict__ logits, int ld, int vocab, const float* __restrict__ fparams,
    const int* __restrict__ iparams, uint8_t* __restrict__ seen_all, size_t seen_stride,
    int* __restrict__ out_tokens, int* __restrict__ last_tokens, const unsigned long long* __restrict__ best, int best_ld,
    int best_parts, int best_cols) {
    __shared__ unsigned int part_list[SAMPLE_PART_LIST];
    __shared__ float s_val[SAMPLE_THREADS / CELEG_WAVE];
    __shared__ int s_idx[SAMPLE_THREADS / CELEG_WAVE];
    __shared__ __attribute__((aligned(16))) unsigned int hist[256 * SAMPLE_HIST_COPIES];   // or SAMPLE_RANK_CAP gathered (key, id)
    __shared__ uint32_t maxes[SAMPLE_THREADS / CELEG_WAVE];       // per wavefront: the bound it offers
    __shared__ unsigned int sel[3];       // prefix, remaining, size of the last bin
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

    if (top_k < 0) {
        // ---- a token that the caller forces: -(token + 1) in the place of top_k
        // (src/backend/cuda/model/sampler.cu:44-54: the forced token is copied in and marked as seen)
        if (tid == 0) {
            const int token = min(-(top_k + 1), vocab - 1);
            out_tokens[r] = token;
            if (last_tokens && slot >= 0) last_tokens[slot] = token;
            if (seen_all && seen_row >= 0) seen_all[static_cast<size_t>(seen_row) * seen_stride + token] = 1;
        }
        return;
    }
    if (temperature <= 0.0f || top_k == 1) {
        // ---- penalised argmax, lowest index wins ties
        float best = -INFINITY;
        int best_i = 0x7fffffff;
        for_each_logit(row, seen, penalty, vocab, tid, [&](float v, int i) {
            if (best_i == 0x7fffffff || v > best) { best = v; best_i = i; }
        });
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
            if (seen_all && seen_row >= 0) seen_all[static_cast<size_t>(seen_row) * seen_stride + best_i] = 1;
        }
        return;
    }

    top_k = min(min(top_k, vocab), SAMPLE_MAX_K);
    // the scores of the row are turned into keys once and kept in registers (up to 128 a
    // thread); larger vocabularies walk the row again for every pass
    static_assert(sizeof(hist) >= SAMPLE_RANK_CAP * sizeof(uint2), "the gathered scores share the histograms' room");
    uint2* gathered = reinterpret_cast<uint2*>(hist);
    bool sorted = false;
    if (best) {
        // what the output head left beside the logits: the candidates without reading the row
        sorted = top_k_from_parts(row, seen, penalty, temperature, vocab, top_k, best + static_cast<size_t>(r) * best_ld, best_parts, best_cols, maxes,
                                  gathered, sel, part_list, cand_score, cand_id);
        __syncthreads();        // (before what follows reuses the counters)
    }
    if (sorted) {
    } else if (vocab <= SAMPLE_THREADS * 64)
        sorted = top_k_ranked<64>(row, seen, penalty, temperature, vocab, top_k, maxes, gathered, sel, cand_score, cand_id);
    else if (vocab <= SAMPLE_THREADS * 128)
        sorted = top_k_ranked<128>(row, seen, penalty, temperature, vocab, top_k, maxes, gathered, sel, cand_score, cand_id);
    if (!sorted) {
        if (vocab <= SAMPLE_THREADS * 64)
            top_k_candidates<64>(row, seen, penalty, temperature, vocab, top_k, hist, sel, running, cand_score, cand_id);
        else if (vocab <= SAMPLE_THREADS * 128)
            top_k_candidates<128>(row, seen, penalty, temperature, vocab, top_k, hist, sel, running, cand_score, cand_id);
        else
            top_k_candidates<0>(row, seen, penalty, temperature, vocab, top_k, hist, sel, running, cand_score, cand_id);
    }
    if (tid >= top_k && tid < SAMPLE_MAX_K) { cand_score[tid] = -INFINITY; cand_id[tid] = 0x7fffffff; }
    __syncthreads();
    if (wave != 0) return;         // one wavefront does the rest: no workgroup barriers from here
    const int chosen = choose_among(cand_score, cand_id, top_k, top_p, u, sorted, lane);
    if (lane == 0) {
        out_tokens[r] = chosen;
        if (last_tokens && slot >= 0) last_tokens[slot] = chosen;
        if (seen_all && seen_row >= 0) seen_all[static_cast<size_t>(seen_row) * seen_stride + chosen] = 1;
    }
}

// Penalised argmax of rows that are all greedy, a row cut into parts of ARGMAX_PART logits,
// a workgroup each (one workgroup a row is bound by what one compute unit can pull: 11 us at
// 65,536 logits).  A part's best goes into best[row] by a 64-bit atomic maximum of
// (ordered key of the value, ~index): the largest value wins and, among equal values, the
// lowest index.  The part that arrives last (a counter) reads the winner, writes the token
// and leaves best and arrived at zero for the next launch.  Everything the workgroups tell
// each other goes through these atomics.
#define ARGMAX_PART 4096
#define ARGMAX_THREADS 256
__global__ __launch_bounds__(ARGMAX_THREADS) void argmax_parts_kernel(
    const float* __restrict__ logits, int ld, int vocab, const float* __restrict__ fparams,
    const int* __restrict__ iparams, uint8_t* __restrict__ seen_all, size_t seen_stride,
    int* __restrict__ out_tokens, int* __restrict__ last_tokens, unsigned long long* __restrict__ best,
    unsigned int* __restrict__ arrived) {
    constexpr int PER = ARGMAX_PART / ARGMAX_THREADS;
    __shared__ unsigned long long s_best[ARGMAX_THREADS / CELEG_WAVE];
    const int r = blockIdx.y, tid = threadIdx.x;
    const int lane = tid & (CELEG_WAVE - 1), wave = tid / CELEG_WAVE;
    const float* row = logits + static_cast<size_t>(r) * ld;
    const float penalty = fparams[4 * r + 2];
    const int seen_row = iparams[3 * r + 1], slot = iparams[3 * r + 2];
    const uint8_t* seen = (seen_all && seen_row >= 0 && penalty > 1.0f)
                              ? seen_all + static_cast<size_t>(seen_row) * seen_stride : nullptr;
    const int lo = blockIdx.x * ARGMAX_PART;
    float v[PER];
    unsigned char sn[PER];
#pragma unroll
    for (int j = 0; j < PER; ++j) {
        const int i = min(lo + tid + ARGMAX_THREADS * j, vocab - 1);     // clamped, masked below
        v[j] = row[i];
        sn[j] = seen ? seen[i] : 0;
    }
    unsigned long long mine = 0ull;
#pragma unroll
    for (int j = 0; j < PER; ++j) {
        const int i = lo + tid + ARGMAX_THREADS * j;
        float x = v[j];
        if (sn[j]) x = x >= 0.0f ? x / penalty : x * penalty;
        if (i < vocab) mine = max(mine, packed_logit(x, i));
    }
#pragma unroll
    for (int off = CELEG_WAVE / 2; off > 0; off >>= 1) {
        const unsigned long long other = __shfl_xor(mine, off, CELEG_WAVE);
        mine = max(mine, other);
    }
    if (lane == 0) s_best[wave] = mine;
    __syncthreads();
    if (tid != 0) return;
#pragma unroll
    for (int w = 1; w < ARGMAX_THREADS / CELEG_WAVE; ++w) mine = max(mine, s_best[w]);
    atomicMax(&best[r], mine);
    __threadfence();
    if (atomicAdd(&arrived[r], 1u) != gridDim.x - 1) return;
    __threadfence();
    const unsigned long long winner = atomicExch(&best[r], 0ull);
    atomicExch(&arrived[r], 0u);
    const int token = packed_logit_index(winner);
    out_tokens[r] = token;
    if (last_tokens && slot >= 0) last_tokens[slot] = token;
    if (seen_all && seen_row >= 0) seen_all[static_cast<size_t>(seen_row) * seen_stride + token] = 1;
}

// rows that are all greedy (temperature <= 0 or top_k == 1): best [rows] and arrived [rows]
// must hold zeros when the first launch comes (the kernel leaves them so).  Launches that
// share them must run one after the other.
extern "C" int celeg_argmax_rows(const float* logits, int ld, int rows, int vocab, const float* fparams,
                                 const int* iparams, uint8_t* seen, size_t seen_stride,
                                 int* out_tokens, int* last_tokens, unsigned long long* best,
                                 unsigned int* arrived, hipStream_t stream) {
    if (rows <= 0) return 0;
    if (vocab <= 0) return static_cast<int>(hipErrorInvalidValue);
    hipLaunchKernelGGL(argmax_parts_kernel, dim3((vocab + ARGMAX_PART - 1) / ARGMAX_PART, rows),
                       dim3(ARGMAX_THREADS), 0, stream, logits, ld, vocab, fparams, iparams, seen,
                       seen_stride, out_tokens, last_tokens, best, arrived);
    return CELEG_LAUNCH_RESULT();
}

// The greedy tokens of rows whose output head left the best (logit, index) of every workgroup's
// columns beside the logits (best [rows, ld >= parts], packed as packed_logit packs them): the
// largest of a row's parts is its token.  No repetition penalty: the head
// knows nothing of what a request has seen.  One workgroup a row; the token also goes to
// last_tokens[slot] as with the other kernels.
#define MERGE_THREADS 256
__global__ __launch_bounds__(MERGE_THREADS) void argmax_merge_kernel(
    const unsigned long long* __restrict__ best, int ld, int parts, const int* __restrict__ iparams,
    int* __restrict__ out_tokens, int* __restrict__ last_tokens) {
    __shared__ unsigned long long s_best[MERGE_THREADS / CELEG_WAVE];
    const int r = blockIdx.x, tid = threadIdx.x;
    const int lane = tid & (CELEG_WAVE - 1), wave = tid / CELEG_WAVE;
    const unsigned long long* row = best + static_cast<size_t>(r) * ld;
    unsigned long long mine = 0ull;
    for (int j0 = 0; j0 < parts; j0 += 16 * MERGE_THREADS) {        // sixteen loads of a thread under way at a time:
        unsigned long long v[16];                                   // one trip to memory for 65,536 columns in tiles of 16
#pragma unroll
        for (int j = 0; j < 16; ++j)     // (a part twice changes nothing)
            v[j] = row[min(j0 + tid + MERGE_THREADS * j, parts - 1)];
#pragma unroll
        for (int j = 0; j < 16; ++j) mine = max(mine, v[j]);
    }
#pragma unroll
    for (int off = CELEG_WAVE / 2; off > 0; off >>= 1) mine = max(mine, __shfl_xor(mine, off, CELEG_WAVE));
    if (lane == 0) s_best[wave] = mine;
    __syncthreads();
    if (tid != 0) return;
#pragma unroll
    for (int w = 1; w < MERGE_THREADS / CELEG_WAVE; ++w) mine = max(mine, s_best[w]);
    const int token = packed_logit_index(mine);
    const int slot = iparams[3 * r + 2];
    out_tokens[r] = token;
    if (last_tokens && slot >= 0) last_tokens[slot] = token;
}

extern "C" int celeg_argmax_merge(const unsigned long long* best, int ld, int parts, int rows, const int* iparams,
                                  int* out_tokens, int* last_tokens, hipStream_t stream) {
    if (rows <= 0) return 0;
    if (parts <= 0 || ld < parts) return static_cast<int>(hipErrorInvalidValue);
    hipLaunchKernelGGL(argmax_merge_kernel, dim3(rows), dim3(MERGE_THREADS), 0, stream, best, ld, parts, iparams,
                       out_tokens, last_tokens);
    return CELEG_LAUNCH_RESULT();
}

// best (or null): what an output head left beside these logits, [rows, best_ld >= best_parts], part p of a row
// the best (logit, index) of its columns p * best_cols .. + best_cols - 1 (packed_logit).
extern "C" int celeg_sample(const float* logits, int ld, int rows, int vocab,
                            const float* fparams, const int* iparams, uint8_t* seen,
                            size_t seen_stride, int* out_tokens, int* last_tokens,
                            const unsigned long long* best, int best_ld, int best_parts, int best_cols,
                            hipStream_t stream) {
    if (rows <= 0) return 0;
    if (vocab <= 0) return static_cast<int>(hipErrorInvalidValue);
    if (best && (best_ld < best_parts || best_parts <= 0 || best_cols <= 0 ||
                 static_cast<long long>(best_parts) * best_cols < vocab))
        return static_cast<int>(hipErrorInvalidValue);
    hipLaunchKernelGGL(sample_kernel, dim3(rows), dim3(SAMPLE_THREADS), 0, stream, logits, ld,
                       vocab, fparams, iparams, seen, seen_stride, out_tokens, last_tokens, best, best_ld, best_parts,
                       best_cols);
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
