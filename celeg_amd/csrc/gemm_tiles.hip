// bfloat16 products for many rows on gfx950 (portions of prompts: hundreds to thousands of
// rows), with what surrounds them fused in, under the same contract as the products for
// few rows:
//   out[M,N] = epilogue(scale[m] * (A[M,K] W[N,K]^T) + bias)
// A is bfloat16 with its rows one after the other; behind an RMSNorm it is the bfloat16
// copy of the residual stream, W has the norm's weight folded in and
// scale[m] = rsqrt(mean(x_m^2) + eps) comes from the partial sums of squares that the
// producer of the stream left.  Epilogues: store | add into the 32-bit residual stream,
// refresh its bfloat16 copy and leave partial sums of squares | SwiGLU of a gate and an
// up stream.
//
// Layout.  A workgroup owns a tile of BM rows x BN weight rows (for SwiGLU: BN/2 gate rows
// and the BN/2 up rows of the same columns) over the whole of K.  Blocks of 64 values of k
// of both operands travel from memory straight into LDS (16 bytes a lane,
// global_load_lds), STAGES blocks deep, so that loads of later blocks are in flight while
// the matrix instructions work on the current one; the compiler's barrier would wait for
// every load, so the loop waits for the oldest block by count and uses the bare barrier.
// A row of a block is 128 bytes = 8 chunks of 16; chunk c of row r lies at chunk
// c ^ (r & 7) of its row, which spreads the rows that neighbouring lanes read at the same
// chunk over the banks (measured: as fast as reading 1 KB in a row; rows padded to 144 bytes
// or a swap of neighbouring rows on top were 1.6 times slower).
// The loads place the chunks: a load instruction writes 1 KB = 8 rows, lane l at row l / 8,
// chunk l % 8, so lane l asks memory for the chunk that belongs there.
// WGM x WGN wavefronts share the tile; a wavefront keeps (BN/WGN/16) x (BM/WGM/16) tiles of
// 16x16 sums (v_mfma_f32_16x16x32_bf16 with the weights as the first operand: a lane then
// holds 4 neighbouring columns of one row, which it finishes and writes as one piece).
//
// Reference semantics of the fused parts: RMSNorm src/backend/cpu/kernels/elementwise.cpp:56-76,
// SwiGLU elementwise.cpp:101-119, projections y = x W^T src/model/weight_plan.cpp:82-130;
// the reference fuses the residual addition into its products with beta = 1
// (src/backend/cuda/model/prefill_batched/non_attention.cpp:175-201).
#include "common.h"
#include "tile_params.h"

typedef __bf16 bf16x8_t __attribute__((ext_vector_type(8)));
typedef float floatx4_t __attribute__((ext_vector_type(4)));
typedef __bf16 bf16x4_t __attribute__((ext_vector_type(4)));

enum { T_STORE = 0, T_RESIDUAL = 2, T_SWIGLU = 3, T_QKV = 5 };   // (0, 2, 3: the numbers of the few-rows products)


#define GPTR(p) ((const __attribute__((address_space(1))) void*)(p))
#define LPTR(p) ((__attribute__((address_space(3))) void*)(p))

__device__ __forceinline__ float round_bf16(float x) { return to_float(from_float<bf16>(x)); }

// g / (1 + e^-g) with the hardware's exponential and reciprocal (an ulp each, in 32-bit; the
// result is rounded to bfloat16): the exact division and exponential cost the SwiGLU product
// of 2,048 rows 3 us.
__device__ __forceinline__ float tile_silu(float g) { return g * __frcp_rn(1.0f + __expf(-g)); }

template <int N>
__device__ __forceinline__ void wait_loads() {
    asm volatile("s_waitcnt vmcnt(%0)" ::"n"(N) : "memory");
}

template <int EPI> struct TileStreams { static constexpr int n = EPI == T_SWIGLU ? 2 : 1; };

// The 1/rms of a lane's rows (first, first + 16, ..) from the partial sums of squares that
// the producer of the stream left; 1 without a norm.  The four lanes that share a row (q = 0..3)
// take four partial sums each, as one load where the rows are aligned, and add up over the
// lanes: a few loads a lane, all in flight at once.  (One lane reading all of a row's sums,
// eight at a time, cost a product of 2,048 rows 12 us: 64 loads a lane in two trips, queued
// behind the first blocks of the operands.)
template <int FM>
__device__ __forceinline__ void tile_row_scales(const TileParams& p, const int first, const int q, float (&scale)[FM]) {
#pragma unroll
    for (int tm = 0; tm < FM; ++tm) scale[tm] = 1.f;
    if (!p.stats) return;
    const int nb = p.n_stat_blocks;
    const bool aligned = (p.stats_ld & 3) == 0 && (reinterpret_cast<uintptr_t>(p.stats) & 15) == 0;
    float ssq[FM];
#pragma unroll
    for (int tm = 0; tm < FM; ++tm) ssq[tm] = 0.f;
    for (int c0 = 0; c0 < nb; c0 += 16) {         // (once, up to 16 partial sums a row)
        const int b = c0 + 4 * q;
        floatx4_t part[FM];
#pragma unroll
        for (int tm = 0; tm < FM; ++tm) {
            const float* const srow = p.stats + static_cast<size_t>(min(first + tm * 16, p.M - 1)) * p.stats_ld;
            if (aligned && b + 4 <= nb) {
                part[tm] = *reinterpret_cast<const floatx4_t*>(srow + b);
            } else {
#pragma unroll
                for (int i = 0; i < 4; ++i) part[tm][i] = b + i < nb ? srow[b + i] : 0.f;
            }
        }
#pragma unroll
        for (int tm = 0; tm < FM; ++tm) ssq[tm] += (part[tm][0] + part[tm][1]) + (part[tm][2] + part[tm][3]);
    }
#pragma unroll
    for (int tm = 0; tm < FM; ++tm) {
        float t = ssq[tm];
        t += __shfl_xor(t, 16, 64);
        t += __shfl_xor(t, 32, 64);
        scale[tm] = 1.0f / sqrtf(t / static_cast<float>(p.K) + p.eps);
    }
}

// What becomes of a wavefront's sums (shared by the kernels below).  The wavefront (wm, wn) of
// the tile holds rows m0 + wm*WTM .. of `pieces` (<= FNS) column pieces of 16 from column col0 of
// every stream:  acc[s*FNS + j][tm][i] is row .. + tm*16 + lane%16, column col0 + j*16 + 4*(lane/16) + i.
// ROWS_VIA_LDS (store and SwiGLU): a lane's pieces of 4 columns go to the wavefront's corner of
// LDS first and leave in whole rows of the wavefront's tile, 16 bytes a lane; straight from the
// registers a store instruction would touch 16 rows with 32 bytes each.
template <int BM, int WGM, int WGN, int FNS, int EPI, bool ROWS_VIA_LDS>
__device__ __forceinline__ void tile_epilogue(
    const TileParams& p, floatx4_t (&acc)[TileStreams<EPI>::n * FNS][BM / WGM / 16], const float (&scale)[BM / WGM / 16],
    const int m0, const int col0, const int pieces, const int tile_n, const int wm, const int wn, const int lane,
    char* const lds) {
    constexpr int NW = WGM * WGN;
    constexpr int NS = TileStreams<EPI>::n;
    constexpr int WTM = BM / WGM;
    constexpr int FM = WTM / 16;
    const int M = p.M, N = p.N;
    const int r16 = lane & 15, q = lane >> 4;
    // the residual stream's old values: all asked for at once where the registers hold them
    // beside the sums, else a row of pieces at a time
    constexpr bool RES = EPI == T_RESIDUAL;
    constexpr bool OLD_AT_ONCE = FM * FNS <= 32;
    floatx4_t old_[RES && OLD_AT_ONCE ? FM : 1][RES ? FNS : 1];
    auto fetch_old = [&](int tm, floatx4_t (&to)[RES ? FNS : 1]) {
#pragma unroll
        for (int j = 0; j < (RES ? FNS : 1); ++j) {
            const int m = min(m0 + wm * WTM + tm * 16 + r16, M - 1);
            const int n = min(col0 + j * 16 + 4 * q, N - 4);
            to[j] = *reinterpret_cast<const floatx4_t*>(static_cast<const float*>(p.out) + static_cast<size_t>(m) * p.ldo + n);
        }
    };
    if (RES && OLD_AT_ONCE) {
#pragma unroll
        for (int tm = 0; tm < FM; ++tm) fetch_old(tm, old_[RES && OLD_AT_ONCE ? tm : 0]);
    }
    constexpr int PITCH = FNS * 32 + 16;          // bytes between a wavefront's rows in LDS
    constexpr bool VIA_LDS = ROWS_VIA_LDS && !RES;
    char* const corner = lds + static_cast<size_t>(wm * WGN + wn) * WTM * PITCH;
    if (VIA_LDS) __syncthreads();                 // the stages are no longer read
    float sq[FM];
#pragma unroll
    for (int tm = 0; tm < FM; ++tm) sq[tm] = 0.f;
#pragma unroll
    for (int tm = 0; tm < FM; ++tm) {
        const int m = m0 + wm * WTM + tm * 16 + r16;
        if (RES && !OLD_AT_ONCE) fetch_old(tm, old_[0]);
#pragma unroll
        for (int j = 0; j < FNS; ++j) {
            const int n = col0 + j * 16 + 4 * q;
            if (j >= pieces || m >= M || n >= N) continue;       // N % 4 == 0: a lane's four columns are inside together
            float v[NS][4];
#pragma unroll
            for (int s = 0; s < NS; ++s)
#pragma unroll
                for (int i = 0; i < 4; ++i)
                    v[s][i] = acc[s * FNS + j][tm][i] * scale[tm] +
                              (p.bias ? p.bias[static_cast<size_t>(s) * p.stream_rows + n + i] : 0.f);
            if (EPI == T_RESIDUAL) {
                float* const h = static_cast<float*>(p.out) + static_cast<size_t>(m) * p.ldo + n;
                floatx4_t old = old_[RES && OLD_AT_ONCE ? tm : 0][RES ? j : 0];
                // the product enters the sum rounded to bfloat16, as where it is a tensor of its own
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    old[i] += round_bf16(v[0][i]);
                    sq[tm] += old[i] * old[i];
                }
                *reinterpret_cast<floatx4_t*>(h) = old;
                if (p.out_bf16)     // (the conversion rounds to nearest even, as from_float<bf16>)
                    *reinterpret_cast<bf16x4_t*>(p.out_bf16 + static_cast<size_t>(m) * p.ld_bf16 + n) =
                        bf16x4_t{static_cast<__bf16>(old[0]), static_cast<__bf16>(old[1]),
                                 static_cast<__bf16>(old[2]), static_cast<__bf16>(old[3])};
            } else {
                float o[4];
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    if (EPI == T_SWIGLU) {
                        const float g = round_bf16(v[0][i]), u = round_bf16(v[NS - 1][i]);
                        o[i] = tile_silu(g) * u;
                    } else {
                        o[i] = v[0][i];
                    }
                }
                const bf16x4_t piece = bf16x4_t{static_cast<__bf16>(o[0]), static_cast<__bf16>(o[1]),
                                                static_cast<__bf16>(o[2]), static_cast<__bf16>(o[3])};
                if (VIA_LDS) *reinterpret_cast<bf16x4_t*>(corner + (tm * 16 + r16) * PITCH + (j * 16 + 4 * q) * 2) = piece;
                else *reinterpret_cast<bf16x4_t*>(static_cast<bf16*>(p.out) + static_cast<size_t>(m) * p.ldo + n) = piece;
            }
        }
    }
    if (VIA_LDS) {
        // (the wavefront reads what its own lanes wrote: LDS keeps a wavefront's accesses in order)
        const int cpr = pieces * 2;               // chunks of 8 columns a row
        const bool wide_stores = (p.ldo % 8) == 0 && (reinterpret_cast<uintptr_t>(p.out) & 15) == 0;
        for (int idx = lane; idx < WTM * cpr; idx += 64) {
            const int row = idx / cpr, ch = idx % cpr;
            const int m = m0 + wm * WTM + row, n = col0 + ch * 8;
            if (m >= M || n >= N) continue;
            const char* const from = corner + row * PITCH + ch * 16;
            bf16* const to = static_cast<bf16*>(p.out) + static_cast<size_t>(m) * p.ldo + n;
            if (wide_stores && n + 8 <= N) {
                *reinterpret_cast<bf16x8_t*>(to) = *reinterpret_cast<const bf16x8_t*>(from);
            } else {
                *reinterpret_cast<bf16x4_t*>(to) = *reinterpret_cast<const bf16x4_t*>(from);
                if (n + 8 <= N) *reinterpret_cast<bf16x4_t*>(to + 4) = *reinterpret_cast<const bf16x4_t*>(from + 8);
            }
        }
    }

    if (EPI == T_RESIDUAL && p.stats_out) {
        // a row's squares: over the lane's columns (above), the four lanes that share the
        // row, then the wavefronts that share it, always in the same order
        float* const red = reinterpret_cast<float*>(lds);
        __syncthreads();                          // the stages are no longer read
#pragma unroll
        for (int tm = 0; tm < FM; ++tm) {
            float s = sq[tm];
            s += __shfl_xor(s, 16, 64);
            s += __shfl_xor(s, 32, 64);
            if (q == 0) red[wn * BM + wm * WTM + tm * 16 + r16] = s;
        }
        __syncthreads();
        for (int r = threadIdx.x; r < BM; r += NW * 64) {
            float s = 0.f;
#pragma unroll
            for (int w = 0; w < WGN; ++w) s += red[w * BM + r];
            if (m0 + r < M) p.stats_out[static_cast<size_t>(m0 + r) * p.stats_ld_out + tile_n] = s;
        }
    }
}

// ---- the q/k/v epilogue (heads of 64 columns: a wavefront of a 128x128 tile on 4x2 wavefronts
// holds 32 rows of one head)
#define QKV_HD 64
// What it needs from memory, asked for before the product: the positions of the lane's rows
// and the head's norm weight at the lane's columns; and, lanes 0 .. rows-1 of the wavefront, the
// position and the slot of one row each (whose page is looked up once they have arrived).
template <int FM>
struct QkvEarly {
    int pos[FM];
    floatx4_t weight[4];
    int row_pos, row_slot, row_page;
};

template <int BM, int WGM, int WGN>
__device__ __forceinline__ void qkv_early_rows(const TileParams& p, QkvEarly<BM / WGM / 16>& e, const int m0, const int col0,
                                               const int wm, const int lane) {
    constexpr int WTM = BM / WGM, FM = WTM / 16;
    const int r16 = lane & 15, q = lane >> 4;
    const int head = min(col0, p.N - QKV_HD) / QKV_HD;
    const float* const weight = head < p.q_heads ? p.q_weight : (head < p.q_heads + p.kv_heads ? p.k_weight : nullptr);
#pragma unroll
    for (int tm = 0; tm < FM; ++tm) e.pos[tm] = p.positions[min(m0 + wm * WTM + tm * 16 + r16, p.M - 1)];
#pragma unroll
    for (int j = 0; j < 4; ++j)
        e.weight[j] = weight ? *reinterpret_cast<const floatx4_t*>(weight + j * 16 + 4 * q) : floatx4_t{1.f, 1.f, 1.f, 1.f};
    const int row = min(m0 + wm * WTM + min(lane, WTM - 1), p.M - 1);
    e.row_pos = p.positions[row];
    e.row_slot = p.token_slot[row];
    e.row_page = 0;
}

// (behind the first blocks' loads: the page of the lane's row)
template <int BM, int WGM, int WGN>
__device__ __forceinline__ void qkv_early_pages(const TileParams& p, QkvEarly<BM / WGM / 16>& e, const int col0) {
    const int head = min(col0, p.N - QKV_HD) / QKV_HD;
    if (head >= p.q_heads)
        e.row_page = p.table[static_cast<size_t>(e.row_slot) * p.table_stride + e.row_pos / p.page_tokens];
}

// acc[j][tm][i]: row .. + tm*16 + lane%16, column col0 + j*16 + 4*(lane/16) + i of the head at col0.
// The sums are rounded to bfloat16 first, as where the product is a tensor of its own; norm,
// rotation (split halves: pair (c, c + 32)) as qk_norm_rope_store makes them.  The head's rows
// go to the wavefront's corner of LDS and leave from there: query rows to `out`, key rows to
// their places in the pages, values by groups of four tokens that lie side by side in a page.
template <int BM, int WGM, int WGN>
__device__ __forceinline__ void qkv_epilogue(const TileParams& p, floatx4_t (&acc)[4][BM / WGM / 16],
                                             const float (&scale)[BM / WGM / 16], const QkvEarly<BM / WGM / 16>& e,
                                             const int m0, const int col0, const int wm, const int wn, const int lane,
                                             char* const lds) {
    constexpr int WTM = BM / WGM, FM = WTM / 16;
    constexpr int PITCH = QKV_HD * 2 + 16;            // bytes between a wavefront's rows in LDS
    constexpr int CORNER = WTM * PITCH + WTM * 16;    // the rows, then (position, slot, page, -) of every row
    const int M = p.M;
    const int r16 = lane & 15, q = lane >> 4;
    char* const corner = lds + static_cast<size_t>(wm * WGN + wn) * CORNER;
    int* const rowinfo = reinterpret_cast<int*>(corner + WTM * PITCH);
    const int head = min(col0, p.N - QKV_HD) / QKV_HD;
    const bool is_q = head < p.q_heads, is_k = !is_q && head < p.q_heads + p.kv_heads;
    const int kv_head = is_q ? 0 : (is_k ? head - p.q_heads : head - p.q_heads - p.kv_heads);
    const bool normed = is_q ? p.q_weight != nullptr : (is_k && p.k_weight != nullptr);
    const bool rotate = p.cos_sin && (is_q || is_k);
    // (cos, sin) of the lane's 2 x 4 column pairs for each of its rows: asked for only now (the
    // registers they take would cost the product a wavefront a SIMD), ahead of the barrier
    floatx4_t cs[FM][4];
    if (rotate) {
#pragma unroll
        for (int tm = 0; tm < FM; ++tm) {
            const float* const c = p.cos_sin + static_cast<size_t>(e.pos[tm]) * QKV_HD;     // 32 pairs of two
#pragma unroll
            for (int j = 0; j < 2; ++j) {
                cs[tm][2 * j] = *reinterpret_cast<const floatx4_t*>(c + (j * 16 + 4 * q) * 2);
                cs[tm][2 * j + 1] = *reinterpret_cast<const floatx4_t*>(c + (j * 16 + 4 * q) * 2 + 4);
            }
        }
    }
    __syncthreads();                                  // the stages are no longer read
    if (col0 >= p.N) return;                          // (a tile that hangs over the last head)
#pragma unroll
    for (int tm = 0; tm < FM; ++tm) {
        float x[4][4];
        float ssq = 0.f;
#pragma unroll
        for (int j = 0; j < 4; ++j)
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                x[j][i] = round_bf16(acc[j][tm][i] * scale[tm] + (p.bias ? p.bias[col0 + j * 16 + 4 * q + i] : 0.f));
                ssq += x[j][i] * x[j][i];
            }
        if (normed) {
            ssq += __shfl_xor(ssq, 16, 64);
            ssq += __shfl_xor(ssq, 32, 64);
            const float inv = 1.0f / sqrtf(ssq / static_cast<float>(QKV_HD) + p.qk_eps);
#pragma unroll
            for (int j = 0; j < 4; ++j)
#pragma unroll
                for (int i = 0; i < 4; ++i) x[j][i] = x[j][i] * inv * e.weight[j][i];
        }
        if (rotate) {
#pragma unroll
            for (int j = 0; j < 2; ++j)
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    // (cos, sin) of pair j*16 + 4q + i: four pairs are two loads of four floats
                    const float c = i < 2 ? cs[tm][2 * j][2 * i] : cs[tm][2 * j + 1][2 * (i - 2)];
                    const float s = i < 2 ? cs[tm][2 * j][2 * i + 1] : cs[tm][2 * j + 1][2 * (i - 2) + 1];
                    const float a = x[j][i], b = x[j + 2][i];
                    x[j][i] = a * c - b * s;
                    x[j + 2][i] = b * c + a * s;
                }
        }
#pragma unroll
        for (int j = 0; j < 4; ++j)
            *reinterpret_cast<bf16x4_t*>(corner + (tm * 16 + r16) * PITCH + (j * 16 + 4 * q) * 2) =
                bf16x4_t{static_cast<__bf16>(x[j][0]), static_cast<__bf16>(x[j][1]), static_cast<__bf16>(x[j][2]),
                         static_cast<__bf16>(x[j][3])};
    }
    if (lane < WTM) {
        rowinfo[4 * lane] = e.row_pos;
        rowinfo[4 * lane + 1] = e.row_slot;
        rowinfo[4 * lane + 2] = e.row_page;
    }
    // (the wavefront reads what its own lanes wrote: LDS keeps a wavefront's accesses in order)
    const int page_mask = p.page_tokens - 1;
    const int row_base = m0 + wm * WTM;
    if (is_q || is_k) {
        for (int idx = lane; idx < WTM * 8; idx += 64) {
            const int row = idx >> 3, ch = idx & 7;
            if (row_base + row >= M) continue;
            const bf16x8_t piece = *reinterpret_cast<const bf16x8_t*>(corner + row * PITCH + ch * 16);
            bf16* to;
            if (is_q) {
                to = static_cast<bf16*>(p.out) + static_cast<size_t>(row_base + row) * p.ldo + col0 + ch * 8;
            } else {
                const int pos = rowinfo[4 * row], page = rowinfo[4 * row + 2];
                to = p.k_pool + (((static_cast<size_t>(page) * p.n_layers + p.layer) * p.kv_heads + kv_head) * p.page_tokens +
                                 (pos & page_mask)) * QKV_HD + ch * 8;
            }
            *reinterpret_cast<bf16x8_t*>(to) = piece;
        }
        return;
    }
    // values: [dimension][token] inside a page
    for (int u = lane; u < (WTM / 4) * QKV_HD; u += 64) {
        const int g = u % (WTM / 4), d = u / (WTM / 4);
        const int r0 = 4 * g;
        const int pos0 = rowinfo[4 * r0], slot0 = rowinfo[4 * r0 + 1];
        bool together = row_base + r0 + 3 < M && (pos0 & 3) == 0;
        unsigned short val[4];
#pragma unroll
        for (int k = 0; k < 4; ++k) {
            together = together && rowinfo[4 * (r0 + k)] == pos0 + k && rowinfo[4 * (r0 + k) + 1] == slot0;
            val[k] = *reinterpret_cast<const unsigned short*>(corner + (r0 + k) * PITCH + d * 2);
        }
        if (together) {
            bf16* const to = p.v_pool + ((static_cast<size_t>(rowinfo[4 * r0 + 2]) * p.n_layers + p.layer) * p.kv_heads + kv_head) *
                                            p.page_tokens * QKV_HD + static_cast<size_t>(d) * p.page_tokens + (pos0 & page_mask);
            *reinterpret_cast<uint2*>(to) = uint2{static_cast<unsigned>(val[0]) | (static_cast<unsigned>(val[1]) << 16),
                                                  static_cast<unsigned>(val[2]) | (static_cast<unsigned>(val[3]) << 16)};
        } else {
#pragma unroll
            for (int k = 0; k < 4; ++k) {
                if (row_base + r0 + k >= M) continue;
                const int pos = rowinfo[4 * (r0 + k)], page = rowinfo[4 * (r0 + k) + 2];
                unsigned short* const to = reinterpret_cast<unsigned short*>(
                    p.v_pool + ((static_cast<size_t>(page) * p.n_layers + p.layer) * p.kv_heads + kv_head) * p.page_tokens * QKV_HD +
                    static_cast<size_t>(d) * p.page_tokens + (pos & page_mask));
                *to = val[k];
            }
        }
    }
}

template <int BM, int BN, int WGM, int WGN, int STAGES, int EPI>
__global__ __launch_bounds__(WGM * WGN * 64)
void gemm_tiles_kernel(const TileParams p, const int tiles_m, const int tiles_n, const int dies_m) {
    constexpr int NW = WGM * WGN;
    constexpr int NS = TileStreams<EPI>::n;
    constexpr int WTM = BM / WGM, WTN = BN / WGN;
    constexpr int FM = WTM / 16, FN = WTN / 16;
    constexpr int STAGE_BYTES = (BM + BN) * 128;
    constexpr int GROUPS = (BM + BN) / 8;          // loads of 1 KB a block of k
    constexpr int GPW = (GROUPS + NW - 1) / NW;    // of which a wavefront issues this many (where they do
                                                   // not divide, the last ones ask for the last group again)
    static_assert(FN % NS == 0 && WTM % 16 == 0 && WTN % 16 == 0, "tile shape");
    static_assert(GPW * STAGES < 64, "more loads in flight than the counter holds");
    extern __shared__ __attribute__((aligned(1024))) char lds[];

    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6), lane = threadIdx.x & 63;
    const int wm = wave / WGN, wn = wave % WGN;
    const int M = p.M, N = p.N, K = p.K;

    // Workgroups go to the 8 dies in turn, and every die has an L2 of its own: die x gets the
    // tiles of a rectangle of the tile grid (dies_m x dies_n rectangles), walked down its rows
    // first, so that the tiles that run together on a die share rows of A and of W and each
    // operand crosses the fabric behind the L2s few times.
    const int dies_n = 8 / dies_m;
    const int die = blockIdx.x & 7, local = blockIdx.x >> 3;
    const int di = die / dies_n, dj = die % dies_n;
    const int r0 = di * tiles_m / dies_m, rows = (di + 1) * tiles_m / dies_m - r0;
    const int c0 = dj * tiles_n / dies_n, cols = (dj + 1) * tiles_n / dies_n - c0;
    if (local >= rows * cols) return;
    const int tile_n = c0 + local / rows;
    const int m0 = (r0 + local % rows) * BM;
    const int n0 = tile_n * (BN / NS);

    // ---- what this lane asks memory for: group g = wave + i * NW, rows 8g .. 8g+7 of the stage
    const char* src[GPW];
#pragma unroll
    for (int i = 0; i < GPW; ++i) {
        const int g = min(wave + i * NW, GROUPS - 1);
        const int row = 8 * g + (lane >> 3);               // the row whose chunk lands at this lane's place
        const int chunk = (lane & 7) ^ (row & 7);
        if (g < BM / 8) {
            const int m = min(m0 + row, M - 1);
            src[i] = reinterpret_cast<const char*>(p.a + static_cast<size_t>(m) * p.lda) + chunk * 16;
        } else {
            const int b = row - BM;
            const int s = b / (BN / NS), j = b % (BN / NS);
            const int n = min(n0 + j, N - 1);
            src[i] = reinterpret_cast<const char*>(p.w + (static_cast<size_t>(s) * p.stream_rows + n) * p.ldw) + chunk * 16;
        }
    }
    auto issue = [&](int stage, int kb) {
        char* const base = lds + stage * STAGE_BYTES;
#pragma unroll
        for (int i = 0; i < GPW; ++i)
            __builtin_amdgcn_global_load_lds(GPTR(src[i] + static_cast<size_t>(kb) * 128),
                                             LPTR(base + min(wave + i * NW, GROUPS - 1) * 1024), 16, 0, 0);
    };

    // ---- where this lane's operands lie inside a 16-row piece of a stage (k-step 0 and 1)
    const int r16 = lane & 15, q = lane >> 4;
    int lane_off[2];
#pragma unroll
    for (int ks = 0; ks < 2; ++ks)
        lane_off[ks] = r16 * 128 + (((ks * 4 + q) ^ (r16 & 7)) * 16);

    floatx4_t acc[FN][FM];
#pragma unroll
    for (int tn = 0; tn < FN; ++tn)
#pragma unroll
        for (int tm = 0; tm < FM; ++tm) acc[tn][tm] = floatx4_t{0.f, 0.f, 0.f, 0.f};

    // ---- the rows' 1/rms, asked for ahead of the first blocks
    float scale[FM];
    tile_row_scales<FM>(p, m0 + wm * WTM + r16, q, scale);
    QkvEarly<EPI == T_QKV ? FM : 1> qkv_early;
    if constexpr (EPI == T_QKV) qkv_early_rows<BM, WGM, WGN>(p, qkv_early, m0, n0 + wn * WTN, wm, lane);

    const int nkb = K >> 6;                       // K % 64 == 0 (checked by the host)
#pragma unroll
    for (int s = 0; s < STAGES; ++s)
        if (s < nkb) issue(s, s);
    if constexpr (EPI == T_QKV) qkv_early_pages<BM, WGM, WGN>(p, qkv_early, n0 + wn * WTN);

    // Operands of a k-step (32 values of k) travel from LDS to registers one step ahead of
    // the matrix instructions that use them: a wavefront asks for step 1 of a block, then
    // multiplies step 0; at the barrier in the middle everybody holds the whole block in
    // registers, so its stage is refilled there, and step 0 of the next block is asked for
    // before step 1 is multiplied.
    bf16x8_t af[2][FM], wf[2][FN];
    auto fetch = [&](int stage, int ks, bf16x8_t (&a)[FM], bf16x8_t (&w)[FN]) {
        const char* const sa = lds + stage * STAGE_BYTES + (wm * WTM) * 128 + lane_off[ks];
        const char* const sw = lds + stage * STAGE_BYTES + BM * 128 + lane_off[ks];
#pragma unroll
        for (int tm = 0; tm < FM; ++tm) a[tm] = *reinterpret_cast<const bf16x8_t*>(sa + tm * 2048);
#pragma unroll
        for (int tn = 0; tn < FN; ++tn) {
            const int brow = (tn / (FN / NS)) * (BN / NS) + wn * (WTN / NS) + (tn % (FN / NS)) * 16;
            w[tn] = *reinterpret_cast<const bf16x8_t*>(sw + brow * 128);
        }
    };
    auto multiply = [&](const bf16x8_t (&a)[FM], const bf16x8_t (&w)[FN]) {
#pragma unroll
        for (int tn = 0; tn < FN; ++tn)
#pragma unroll
            for (int tm = 0; tm < FM; ++tm)
                acc[tn][tm] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(w[tn], a[tm], acc[tn][tm], 0, 0, 0);
    };
    // block 0 has arrived when at most the later blocks' loads are out
    if (STAGES - 1 < nkb) wait_loads<GPW * (STAGES - 1)>(); else wait_loads<0>();
    __builtin_amdgcn_s_barrier();
    asm volatile("" ::: "memory");
    fetch(0, 0, af[0], wf[0]);
    int stage = 0;
    for (int kb = 0; kb < nkb; ++kb) {
        fetch(stage, 1, af[1], wf[1]);
        multiply(af[0], wf[0]);
        int next = stage + 1;
        if (next == STAGES) next = 0;
        if (kb + 1 < nkb) {
            if (kb + STAGES - 1 < nkb) wait_loads<GPW * (STAGES - 2)>(); else wait_loads<0>();
            asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
            __builtin_amdgcn_s_barrier();
            asm volatile("" ::: "memory");
            if (kb + STAGES < nkb) issue(stage, kb + STAGES);
            fetch(next, 0, af[0], wf[0]);
        }
        multiply(af[1], wf[1]);
        stage = next;
    }

    if constexpr (EPI == T_QKV) {
        static_assert(EPI != T_QKV || (WTN == QKV_HD && FN == 4), "a wavefront holds one head of 64 columns");
        qkv_epilogue<BM, WGM, WGN>(p, acc, scale, qkv_early, m0, n0 + wn * WTN, wm, wn, lane, lds);
    } else {
        tile_epilogue<BM, WGM, WGN, FN / NS, EPI, false>(p, acc, scale, m0, n0 + wn * (WTN / NS), FN / NS, tile_n, wm, wn, lane, lds);
    }
}

// A read of 16 bytes a lane from LDS at `address` + index * STRIDE, and the waits that go with
// such reads, written as instructions: the compiler does not see the read, so every use of
// `to` has to come behind a wait that names it (the wait takes the registers in and out, which
// keeps the uses behind it), with no branch and no indexing by a variable in between (either
// would let the compiler copy the registers before the data is there).  `left`: how many later
// reads may still be out.
template <int STRIDE>
__device__ __forceinline__ void lds_read(bf16x8_t& to, const unsigned address, const int index) {
    switch (index) {
#define CELEG_LDS_READ_CASE(I) \
    case I: asm volatile("ds_read_b128 %0, %1 offset:%2" : "=v"(to) : "v"(address), "n"(I * STRIDE)); break;
        CELEG_LDS_READ_CASE(0) CELEG_LDS_READ_CASE(1) CELEG_LDS_READ_CASE(2) CELEG_LDS_READ_CASE(3)
        CELEG_LDS_READ_CASE(4) CELEG_LDS_READ_CASE(5) CELEG_LDS_READ_CASE(6) CELEG_LDS_READ_CASE(7)
        CELEG_LDS_READ_CASE(8) CELEG_LDS_READ_CASE(9) CELEG_LDS_READ_CASE(10) CELEG_LDS_READ_CASE(11)
#undef CELEG_LDS_READ_CASE
        default: __builtin_trap();
    }
}
__device__ __forceinline__ void lds_wait(const int left, bf16x8_t& x) {
    switch (left) {
        case 0: asm volatile("s_waitcnt lgkmcnt(0)" : "+v"(x)); break;
        case 1: asm volatile("s_waitcnt lgkmcnt(1)" : "+v"(x)); break;
        case 2: asm volatile("s_waitcnt lgkmcnt(2)" : "+v"(x)); break;
        default: asm volatile("s_waitcnt lgkmcnt(3)" : "+v"(x)); break;
    }
}
template <int FM>
__device__ __forceinline__ void lds_wait_rows(const int left, bf16x8_t& x, bf16x8_t (&rows)[FM]) {
    lds_wait(left, x);
#pragma unroll
    for (int tm = 0; tm < FM; ++tm) asm volatile("" : "+v"(rows[tm]));     // (behind the wait above: volatile statements keep their order)
}

// SwiGLU of a wide tile whose wavefronts each hold columns of one stream only: gate and up
// (rounded to bfloat16, as where they are tensors of their own) meet in LDS, [stream][row], and
// leave as whole rows, 16 bytes a lane.
template <int BM, int BN, int WGM, int WGN>
__device__ __forceinline__ void wide_swiglu_epilogue(
    const TileParams& p, floatx4_t (&acc)[BN / 16 / WGN][BM / WGM / 16], const float (&scale)[BM / WGM / 16],
    const int m0, const int n0, const int wm, const int wn, const int lane, char* const lds) {
    constexpr int NW = WGM * WGN, WTM = BM / WGM, FM = WTM / 16, FN = BN / 16 / WGN;
    constexpr int PS = BN / 32;                   // column pieces of a stream
    constexpr int OC = BN / 2, PITCH = OC * 2 + 16;
    const int M = p.M, N = p.N;
    const int r16 = lane & 15, q = lane >> 4;
    const int s = (wn * FN) / PS, j0 = (wn * FN) % PS;
    __syncthreads();                              // the stages are no longer read
    char* const mine = lds + static_cast<size_t>(s) * BM * PITCH;
    floatx4_t bias[FN];                           // of the lane's columns
#pragma unroll
    for (int j = 0; j < FN; ++j) {
        const int n = n0 + (j0 + j) * 16 + 4 * q;
        bias[j] = floatx4_t{0.f, 0.f, 0.f, 0.f};
        if (p.bias && n < N) bias[j] = *reinterpret_cast<const floatx4_t*>(p.bias + static_cast<size_t>(s) * p.stream_rows + n);
    }
#pragma unroll
    for (int tm = 0; tm < FM; ++tm)
#pragma unroll
        for (int j = 0; j < FN; ++j) {
            const floatx4_t v = acc[j][tm] * scale[tm] + bias[j];
            *reinterpret_cast<bf16x4_t*>(mine + (wm * WTM + tm * 16 + r16) * PITCH + ((j0 + j) * 16 + 4 * q) * 2) =
                bf16x4_t{static_cast<__bf16>(v[0]), static_cast<__bf16>(v[1]), static_cast<__bf16>(v[2]), static_cast<__bf16>(v[3])};
        }
    __syncthreads();
    constexpr int CPR = OC / 8;                   // chunks of 8 columns a row
    const bool wide_stores = (p.ldo % 8) == 0 && (reinterpret_cast<uintptr_t>(p.out) & 15) == 0;
    for (int idx = threadIdx.x; idx < BM * CPR; idx += NW * 64) {
        const int row = idx / CPR, ch = idx % CPR;
        const int m = m0 + row, n = n0 + ch * 8;
        if (m >= M || n >= N) continue;
        const bf16x8_t g = *reinterpret_cast<const bf16x8_t*>(lds + row * PITCH + ch * 16);
        const bf16x8_t u = *reinterpret_cast<const bf16x8_t*>(lds + static_cast<size_t>(BM) * PITCH + row * PITCH + ch * 16);
        bf16x8_t o;
#pragma unroll
        for (int i = 0; i < 8; ++i) o[i] = static_cast<__bf16>(tile_silu(static_cast<float>(g[i])) * static_cast<float>(u[i]));
        bf16* const to = static_cast<bf16*>(p.out) + static_cast<size_t>(m) * p.ldo + n;
        if (wide_stores && n + 8 <= N) {
            *reinterpret_cast<bf16x8_t*>(to) = o;
        } else {
            *reinterpret_cast<bf16x4_t*>(to) = bf16x4_t{o[0], o[1], o[2], o[3]};
            if (n + 8 <= N) *reinterpret_cast<bf16x4_t*>(to + 4) = bf16x4_t{o[4], o[5], o[6], o[7]};
        }
    }
}

// The same product with wide tiles (256 rows x up to 288 weight rows a workgroup), for the
// products whose operands would otherwise cross from the L2 caches to the compute units many
// times over.  A wavefront's tile is too large to hold a block's operands in registers beside
// its sums, so the weights' operands stream from LDS a piece (16 weight rows) at a time, two
// pieces ahead of the matrix instructions that use them, and the rows' operands of the next
// step of 32 values of k come in between; the order is pinned (sched_barrier) and the reads and
// their waits are written as instructions, because left alone the compiler reads two pieces
// into the same registers, waits for them, multiplies, and reads again.  Blocks are KB = 32 or 64 values of k (rows of 64 or 128 bytes in LDS, a load
// instruction fills 16 or 8 rows), STAGES of them, with one barrier a block: behind it
// everybody's loads of this block have landed and nobody reads the block before any more,
// whose stage the loads of block + STAGES - 1 then fill.  Chunk c (16 bytes) of row r lies at
// chunk c ^ ((r / 4) % 4) (rows of 64 bytes) or c ^ (r % 8) (128), so that the 16 rows that
// lanes read at one chunk fall on all banks.  Rows of 64 bytes ask memory for half a cache
// line at a time, and the vector cache fetches the whole line for each half (measured: the
// loads alone then take a third longer).
// The tile's BN / 16 column pieces (gate pieces, then up pieces) are dealt evenly to the WGN
// wavefronts of a row of wavefronts, each within one stream.
template <int BM, int BN, int WGM, int WGN, int STAGES, int KB, int EPI>
__global__ __launch_bounds__(WGM * WGN * 64)
void gemm_tiles_wide_kernel(const TileParams p, const int tiles_m, const int tiles_n, const int dies_m) {
    constexpr int NW = WGM * WGN;
    constexpr int NS = TileStreams<EPI>::n;
    constexpr int WTM = BM / WGM;
    constexpr int FM = WTM / 16;
    constexpr int FN = BN / 16 / WGN;              // column pieces of a wavefront
    constexpr int PS = BN / 16 / NS;               // column pieces of a stream in the tile
    constexpr int KS = KB / 32;                    // steps of 32 values of k a block
    constexpr int ROW_BYTES = KB * 2, CPR = ROW_BYTES / 16, RPL = 1024 / ROW_BYTES;   // chunks a row, rows a load
    constexpr int STAGE_BYTES = (BM + BN) * ROW_BYTES;
    constexpr int GROUPS = (BM + BN) / RPL;        // loads of 1 KB a block of k
    constexpr int GPW = (GROUPS + NW - 1) / NW;
    static_assert(BN % (16 * WGN) == 0 && BN % (16 * NS) == 0 && PS % FN == 0 && WTM % 16 == 0 &&
                  (BM + BN) % 16 == 0 && STAGES >= 2 && FN >= 2 && FN <= 12 && FM <= 12 && (KB == 32 || KB == 64), "tile shape");
    static_assert(GPW * STAGES < 64, "more loads in flight than the counter holds");
    extern __shared__ __attribute__((aligned(1024))) char lds[];

    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6), lane = threadIdx.x & 63;
    const int wm = wave / WGN, wn = wave % WGN;
    const int M = p.M, N = p.N, K = p.K;

    // (the dies' rectangles: as in gemm_tiles_kernel)
    const int dies_n = 8 / dies_m;
    const int die = blockIdx.x & 7, local = blockIdx.x >> 3;
    const int di = die / dies_n, dj = die % dies_n;
    const int r0 = di * tiles_m / dies_m, rows = (di + 1) * tiles_m / dies_m - r0;
    const int c0 = dj * tiles_n / dies_n, cols = (dj + 1) * tiles_n / dies_n - c0;
    if (local >= rows * cols) return;
    const int tile_n = c0 + local / rows;
    const int m0 = (r0 + local % rows) * BM;
    const int n0 = tile_n * (BN / NS);

    // ---- what this lane asks memory for: group g, rows RPL*g .. of the stage
    const char* src[GPW];
#pragma unroll
    for (int i = 0; i < GPW; ++i) {
        const int g = min(wave + i * NW, GROUPS - 1);
        const int row = RPL * g + lane / CPR;
        const int chunk = (lane % CPR) ^ (KB == 32 ? (row >> 2) & 3 : row & 7);
        if (row < BM) {
            const int m = min(m0 + row, M - 1);
            src[i] = reinterpret_cast<const char*>(p.a + static_cast<size_t>(m) * p.lda) + chunk * 16;
        } else {
            const int b = row - BM;
            const int s = b / (BN / NS), j = b % (BN / NS);
            const int n = min(n0 + j, N - 1);
            src[i] = reinterpret_cast<const char*>(p.w + (static_cast<size_t>(s) * p.stream_rows + n) * p.ldw) + chunk * 16;
        }
    }
    auto issue = [&](int stage, int kb) {
        char* const base = lds + stage * STAGE_BYTES;
#pragma unroll
        for (int i = 0; i < GPW; ++i)
            __builtin_amdgcn_global_load_lds(GPTR(src[i] + static_cast<size_t>(kb) * ROW_BYTES),
                                             LPTR(base + min(wave + i * NW, GROUPS - 1) * 1024), 16, 0, 0);
    };

    const int r16 = lane & 15, q = lane >> 4;
    int lane_off[KS];                             // per step of 32 values of k
#pragma unroll
    for (int ks = 0; ks < KS; ++ks)
        lane_off[ks] = r16 * ROW_BYTES + (((ks * 4 + q) ^ (KB == 32 ? (r16 >> 2) & 3 : r16 & 7)) * 16);

    floatx4_t acc[FN][FM];
#pragma unroll
    for (int tn = 0; tn < FN; ++tn)
#pragma unroll
        for (int tm = 0; tm < FM; ++tm) acc[tn][tm] = floatx4_t{0.f, 0.f, 0.f, 0.f};

    float scale[FM];                              // (asked for ahead of the first blocks)
    tile_row_scales<FM>(p, m0 + wm * WTM + r16, q, scale);

    const int nkb = K / KB;                       // K % 64 == 0 (checked by the host)
#pragma unroll
    for (int s = 0; s < STAGES - 1; ++s)
        if (s < nkb) issue(s, s);

    const unsigned lds_base = static_cast<unsigned>(reinterpret_cast<uintptr_t>(LPTR(lds)));
    int stage = 0;
    for (int kb = 0; kb < nkb; ++kb) {
        // this wavefront's loads of block kb have landed when at most the later blocks' are out
        if (kb + STAGES - 2 < nkb) wait_loads<GPW * (STAGES - 2)>(); else wait_loads<0>();
        __builtin_amdgcn_s_barrier();
        asm volatile("" ::: "memory");
        int refill = stage - 1;
        if (refill < 0) refill = STAGES - 1;
        if (kb + STAGES - 1 < nkb) issue(refill, kb + STAGES - 1);
        __builtin_amdgcn_sched_barrier(0);
        // LDS addresses of this lane's operands per step of 32 values of k; pieces are 16 rows apart
        unsigned at_a[KS], at_w[KS];
#pragma unroll
        for (int ks = 0; ks < KS; ++ks) {
            at_a[ks] = lds_base + stage * STAGE_BYTES + (wm * WTM) * ROW_BYTES + lane_off[ks];
            at_w[ks] = lds_base + stage * STAGE_BYTES + (BM + wn * FN * 16) * ROW_BYTES + lane_off[ks];
        }
        // The reads and the waits for them are written out (the compiler, left to count, waits for
        // every read in flight before each second piece).  Piece t = ks * FN + j of the block: step
        // ks, column piece j.  In the order of issue: the rows' operands of step 0, weights 0 and 1;
        // then behind the first matrix instruction of piece t weights t + 2 and, for the first FM
        // pieces of a step, one of the rows' operands of the next step.  LDS answers in order, so
        // piece t may start when no more reads are out than were issued behind weights t.
        bf16x8_t a[2][FM], w[3];
#pragma unroll
        for (int tm = 0; tm < FM; ++tm) lds_read<16 * ROW_BYTES>(a[0][tm], at_a[0], tm);
        lds_read<16 * ROW_BYTES>(w[0], at_w[0], 0);
        lds_read<16 * ROW_BYTES>(w[1], at_w[1 / FN < KS ? 1 / FN : 0], 1 % FN);
#pragma unroll
        for (int t = 0; t < KS * FN; ++t) {
            const int ks = t / FN, j = t % FN;
            // reads issued behind weights t: weights t + 1 (if any) and the rows' operands that went
            // with weights t and t + 1 (issued in pieces t - 2 and t - 1)
            constexpr auto rows_with = [](int piece) {      // does piece `piece` issue one of the next step's rows' operands?
                return piece >= 0 && piece / FN + 1 < KS && piece % FN < FM ? 1 : 0;
            };
            const int behind = (t + 1 < KS * FN ? 1 : 0) + (t >= 2 ? rows_with(t - 2) : 0) + (t >= 1 ? rows_with(t - 1) : 0);
            if (j == 0) lds_wait_rows(behind, w[t % 3], a[ks & 1]);
            else lds_wait(behind, w[t % 3]);
            acc[j][0] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(w[t % 3], a[ks & 1][0], acc[j][0], 0, 0, 0);
            if (t + 2 < KS * FN) lds_read<16 * ROW_BYTES>(w[(t + 2) % 3], at_w[(t + 2) / FN < KS ? (t + 2) / FN : 0], (t + 2) % FN);
            if (rows_with(t)) lds_read<16 * ROW_BYTES>(a[(ks + 1) & 1][j < FM ? j : 0], at_a[ks + 1 < KS ? ks + 1 : 0], j);
#pragma unroll
            for (int tm = 1; tm < FM; ++tm)
                acc[j][tm] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(w[t % 3], a[ks & 1][tm], acc[j][tm], 0, 0, 0);
            __builtin_amdgcn_sched_barrier(0);
        }
        if (++stage == STAGES) stage = 0;
    }
    if constexpr (EPI == T_SWIGLU) {
        wide_swiglu_epilogue<BM, BN, WGM, WGN>(p, acc, scale, m0, n0, wm, wn, lane, lds);
    } else {
        // (rows leave through LDS where the stages have room for the whole tile's output)
        constexpr bool ROWS_FIT = NW * WTM * (FN * 32 + 16) <= STAGES * STAGE_BYTES;
        tile_epilogue<BM, WGM, WGN, FN, EPI, ROWS_FIT>(p, acc, scale, m0, n0 + wn * FN * 16, FN, tile_n, wm, wn, lane, lds);
    }
}

// ---- the shape of the work for given sizes
struct TileShape {
    int id;         // index into the table below
    int bm, bn;     // bn counts weight rows of all streams
};

// For tests and tuning: a shape that overrides the choice below (-1: none).
static int g_force_shape = -1, g_force_dies_m = 0;
extern "C" void celeg_gemm_tiles_force(int shape) { g_force_shape = shape; }
extern "C" void celeg_gemm_tiles_force_dies(int dies_m) { g_force_dies_m = dies_m; }

// id, rows, weight rows, wavefronts along rows and along weight rows, stages, values of k a block of
// the wide kernel (0: the kernel with tiles up to 256x128)
#define TILE_SHAPES(X) \
    X(0, 128, 128, 2, 2, 3, 0) \
    X(1, 256, 128, 2, 2, 3, 0) \
    X(2, 128, 64, 2, 2, 3, 0)  \
    X(3, 64, 128, 2, 2, 3, 0)  \
    X(4, 128, 128, 2, 2, 2, 0) \
    X(5, 256, 128, 4, 2, 3, 0) \
    X(6, 128, 128, 2, 2, 4, 0) \
    X(7, 64, 64, 2, 2, 4, 0)   \
    X(8, 64, 64, 2, 2, 2, 0)   \
    X(9, 128, 64, 2, 2, 2, 0)  \
    X(10, 128, 128, 4, 2, 2, 0) \
    X(11, 256, 288, 4, 2, 2, 64) \
    X(12, 256, 160, 4, 2, 3, 64) \
    X(13, 256, 192, 4, 2, 2, 64) \
    X(14, 128, 192, 2, 2, 3, 64) \
    X(15, 256, 128, 4, 2, 3, 64) \
    X(16, 128, 64, 4, 2, 4, 0) \
    X(17, 64, 128, 2, 4, 4, 0) \
    X(18, 128, 192, 4, 2, 3, 0)

static const int k_shape_bm[] = {128, 256, 128, 64, 128, 256, 128, 64, 64, 128, 128, 256, 256, 256, 128, 256, 128, 64, 128};
static const int k_shape_bn[] = {128, 128, 64, 128, 128, 128, 128, 64, 64, 64, 128, 288, 160, 192, 192, 128, 64, 128, 192};
#define N_TILE_SHAPES 19

static TileShape tile_shape(int M, int N, int K, int streams) {
    int id = 0;
    if (g_force_shape >= 0 && g_force_shape < N_TILE_SHAPES) id = g_force_shape;
    else {
        // Measured at 2,048 rows (1,024 to 9,216 weight rows, 1,024 and 4,608 values of k):
        // tiles of 128x128 with two workgroups of 8 wavefronts a compute unit where they give
        // every unit one and a half or more (8 wavefronts: a tenth faster than 4), else
        // smaller tiles, which fill the chip.
        // Tiles of 256x288, one workgroup a compute unit, where a round of them (2.2 times as long
        // as a round of 128x128 tiles, measured at 1,024 and 2,048 values of k) covers the product
        // in less time: 2,048 rows by 9,216 weight rows are exactly one round, 44 us with the
        // SwiGLU against 63 us.
        const long long wide = static_cast<long long>((M + 127) / 128) * ((static_cast<long long>(N) * streams + 127) / 128);
        const long long tiles288 = static_cast<long long>((M + 255) / 256) * ((static_cast<long long>(N) * streams + 287) / 288);
        const long long rounds288 = (tiles288 + 255) / 256, rounds128 = (wide + 511) / 512;
        // Few weight rows (w2, out_proj: 1,024 of them by 2,048 rows): what a compute unit pulls
        // from L2 bounds the product, so tiles of 128x64 or 64x128 on 8 wavefronts, one a compute
        // unit and 4 blocks of k in flight, beat 64x64 where they still give nearly every unit
        // one (w2 at K = 4,608: 34.8 us as 128x64, 36.0 as 64x128, 40.3 as 64x64; out_proj at
        // K = 1,024: 14.1, 13.6, 14.5).
        const long long tall = static_cast<long long>((M + 127) / 128) * ((static_cast<long long>(N) * streams + 63) / 64);
        const long long flat = static_cast<long long>((M + 63) / 64) * ((static_cast<long long>(N) * streams + 127) / 128);
        // Tiles of 128x192 where they are just one a compute unit (in_proj, 2,048 rows by 3,072
        // weight rows: 256 of them, 20.9 us against 22.2 on 384 tiles of 128x128).
        const long long tiles192 = static_cast<long long>((M + 127) / 128) * ((static_cast<long long>(N) * streams + 191) / 192);
        id = wide >= 384   ? (rounds288 * 22 < rounds128 * 10 ? 11 : (tiles192 > 192 && tiles192 <= 256 ? 18 : 10))
             : wide >= 256 ? 10
             : wide >= 192 ? 3
             : tall >= 224 && K >= 2048 ? 16
             : flat >= 224 ? 17
                           : 7;
    }
    return TileShape{id, k_shape_bm[id], k_shape_bn[id]};
}

template <int BM, int BN, int WGM, int WGN, int STAGES, int KB, int EPI>
static int launch_tiles(const TileParams& p, hipStream_t stream) {
    constexpr int NS = TileStreams<EPI>::n;
    constexpr size_t stages_lds = static_cast<size_t>(STAGES) * (BM + BN) * (KB == 32 ? 64 : 128);
    // (the wide kernel's SwiGLU lays the tile's gate and up values out in LDS)
    constexpr size_t swiglu_lds = KB != 0 && EPI == T_SWIGLU ? static_cast<size_t>(2) * BM * (BN + 16) : 0;
    constexpr size_t lds = stages_lds > swiglu_lds ? stages_lds : swiglu_lds;
    void (*kernel)(const TileParams, const int, const int, const int);
    if constexpr (KB != 0) kernel = &gemm_tiles_wide_kernel<BM, BN, WGM, WGN, STAGES, KB, EPI>;
    else kernel = &gemm_tiles_kernel<BM, BN, WGM, WGN, STAGES, EPI>;
    static_assert(lds <= 160 * 1024, "more LDS than a compute unit has");
    static bool raised = false;              // once per instantiation: more LDS than the default limit
    if (lds > 48 * 1024 && !raised) {
        hipError_t err = hipFuncSetAttribute(reinterpret_cast<const void*>(kernel),
                                             hipFuncAttributeMaxDynamicSharedMemorySize, static_cast<int>(lds));
        if (err != hipSuccess) return static_cast<int>(err);
        raised = true;
    }
    const int tiles_m = (p.M + BM - 1) / BM, tiles_n = (p.N * NS + BN - 1) / BN;
    // how the dies share the grid: every row of tiles of A is read by dies_n dies, every
    // column of tiles of W by dies_m; the split with the fewest bytes read
    int dies_m = 1;
    double best = -1.;
    for (int dm = 1; dm <= 8; dm *= 2) {
        const int dn = 8 / dm;
        if (dm > tiles_m || dn > tiles_n) continue;       // a die without a tile
        const double cost = static_cast<double>(dn) * p.M + static_cast<double>(dm) * p.N * NS;
        if (best < 0. || cost < best) { best = cost; dies_m = dm; }
    }
    if (g_force_dies_m > 0) dies_m = g_force_dies_m;
    const int dies_n = 8 / dies_m;
    const int per_die = ((tiles_m + dies_m - 1) / dies_m) * ((tiles_n + dies_n - 1) / dies_n);
    dim3 grid(per_die * 8), block(WGM * WGN * 64);
    hipLaunchKernelGGL(kernel, grid, block, lds, stream, p, tiles_m, tiles_n, dies_m);
    return CELEG_LAUNCH_RESULT();
}

template <int EPI>
static int launch_epilogue(const TileParams& p, hipStream_t stream) {
    const TileShape s = tile_shape(p.M, p.N, p.K, TileStreams<EPI>::n);
#define TILE_CASE(ID, BM, BN, WGM, WGN, STAGES, KB) \
    if (s.id == ID) return launch_tiles<BM, BN, WGM, WGN, STAGES, KB, EPI>(p, stream);
    TILE_SHAPES(TILE_CASE)
#undef TILE_CASE
    return static_cast<int>(hipErrorInvalidValue);
}

// Number of partial sums of squares a row gets from the "residual" epilogue for these
// sizes (one per tile column): the caller sizes stats_out [>= M, >= blocks].
extern "C" int celeg_gemm_tiles_blocks(int M, int N, int K) {
    const TileShape s = tile_shape(M, N, K, 1);
    return (N + s.bn - 1) / s.bn;
}

extern "C" int celeg_gemm_tiles_params_size() { return static_cast<int>(sizeof(TileParams)); }

// K % 64 == 0, N % 4 == 0, lda, ldw % 8 == 0, outputs with rows aligned to their vector
// stores (ldo % 4 == 0).  Any M >= 1.
extern "C" int celeg_gemm_tiles(const TileParams* params, int epi, hipStream_t stream) {
    const TileParams& p = *params;
    if (p.M <= 0 || p.N <= 0) return 0;
    if (p.K <= 0 || (p.K % 64) || (p.N % 4) || (p.lda % 8) || (p.ldw % 8) || (p.ldo % 4) ||
        p.lda < p.K || p.ldw < p.K || p.ldo < p.N)
        return static_cast<int>(hipErrorInvalidValue);
    if (p.stats && p.n_stat_blocks < 1) return static_cast<int>(hipErrorInvalidValue);
    if (reinterpret_cast<uintptr_t>(p.bias) & 15) return static_cast<int>(hipErrorInvalidValue);
    if (p.out_bf16 && ((p.ld_bf16 % 4) || p.ld_bf16 < p.N)) return static_cast<int>(hipErrorInvalidValue);
    if (epi == T_SWIGLU && p.stream_rows < p.N) return static_cast<int>(hipErrorInvalidValue);
    switch (epi) {
        case T_STORE: return launch_epilogue<T_STORE>(p, stream);
        case T_RESIDUAL: return launch_epilogue<T_RESIDUAL>(p, stream);
        case T_SWIGLU: return launch_epilogue<T_SWIGLU>(p, stream);
        case T_QKV: {
            const auto misaligned = [](const void* ptr) { return (reinterpret_cast<uintptr_t>(ptr) & 15) != 0; };
            const long long heads = static_cast<long long>(p.q_heads) + 2LL * p.kv_heads;
            if (p.q_heads <= 0 || p.kv_heads <= 0 || p.N != heads * QKV_HD || p.ldo % 8 || misaligned(p.out) ||
                !p.positions || !p.token_slot || !p.table || p.table_stride <= 0 || !p.k_pool || !p.v_pool ||
                misaligned(p.k_pool) || misaligned(p.v_pool) || p.page_tokens < 4 || (p.page_tokens & (p.page_tokens - 1)) ||
                p.n_layers <= 0 || p.layer < 0 || p.layer >= p.n_layers || misaligned(p.q_weight) || misaligned(p.k_weight) ||
                misaligned(p.cos_sin))
                return static_cast<int>(hipErrorInvalidValue);
            // a wavefront of the 128x128 tile on 4x2 wavefronts holds 32 rows of one head
            return launch_tiles<128, 128, 4, 2, 2, 0, T_QKV>(p, stream);
        }
        default: return static_cast<int>(hipErrorInvalidValue);
    }
}
