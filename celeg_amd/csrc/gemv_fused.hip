// Skinny bfloat16 matrix products for decode (1..64 rows) on gfx950, with what surrounds
// them fused in: out[M,N] = A[M,K] W[N,K]^T, weights streamed once from HBM through the
// matrix cores, the few rows of A re-read from cache.
//
// A decode step is bound by the number of dependent kernels as much as by bytes, so each
// product takes its neighbours along:
//   A side   plain bfloat16 rows, or rows of the 32-bit residual stream normalised on the
//            fly (RMSNorm: x * rsqrt(mean(x^2) + eps) * w), the row sums of squares taken
//            from the partial sums the producer of the stream left, or recomputed;
//   epilogue store | 32-bit store (logits) | add into the residual stream and leave partial
//            sums of squares | SwiGLU of a gate and an up stream | the double-gated short
//            convolution of a B, a C and an x stream for one new token per request, with
//            its state update.
// Layout of the work: a workgroup owns 16 output columns (of every weight stream); its
// wavefronts split K in chunks of 64 and their partial tiles are added in LDS in wavefront
// order, so the result does not depend on timing.  MFMA 16x16x16: A operand lane l holds
// row l%16, k = 4*(l/16)..+3; B operand lane l holds column l%16, same k; the result lane
// l holds column l%16, rows 4*(l/16)..+3.  Within a chunk, lane group q = l/16 takes the
// 16 consecutive k values q*16.. (both operands alike), so every lane reads 32 contiguous
// bytes of its weight row per chunk.
//
// Reference semantics of the fused parts: RMSNorm src/backend/cpu/kernels/elementwise.cpp:56-76,
// SwiGLU elementwise.cpp:101-119, short convolution src/backend/cpu/kernels/convolution.cpp:7-28,
// projections y = x W^T src/model/weight_plan.cpp:82-130; the reference fuses the residual
// addition into its products with beta = 1 (src/backend/cuda/model/prefill_batched/non_attention.cpp:175-201).
#include "common.h"
#include "gemv_params.h"

typedef short bf16x4_t __attribute__((ext_vector_type(4)));
typedef float floatx4_t __attribute__((ext_vector_type(4)));
typedef __bf16 nbf16x4_t __attribute__((ext_vector_type(4)));
struct __attribute__((aligned(16))) Frag2 {   // 16 bytes = 8 bfloat16 = two MFMA operands
    bf16x4_t lo, hi;
};

enum { A_BF16 = 0, A_NORM = 1 };
enum { E_STORE = 0, E_STORE_F32 = 1, E_RESIDUAL = 2, E_SWIGLU = 3, E_CONV = 4 };


__device__ __forceinline__ short to_bits(float x) { return static_cast<short>(from_float<bf16>(x).bits); }
__device__ __forceinline__ float round_bf16(float x) { return to_float(from_float<bf16>(x)); }

template <int EPI> struct Streams { static constexpr int n = 1; };
template <> struct Streams<E_SWIGLU> { static constexpr int n = 2; };
template <> struct Streams<E_CONV> { static constexpr int n = 3; };

// What the epilogue reads besides the product, asked for before the product is computed:
// the old value of the residual stream, or the convolution's state, taps and bias.
#define CONV_PREFETCH_TAPS 8
template <int MT, int EPI>
struct EpiloguePrefetch {
    float old[EPI == E_RESIDUAL ? MT : 1][4];
    float state[EPI == E_CONV ? MT : 1][4][EPI == E_CONV ? CONV_PREFETCH_TAPS - 1 : 1];
    float taps[EPI == E_CONV ? CONV_PREFETCH_TAPS : 1];
    int slot_row[EPI == E_CONV ? MT : 1][4];
};

template <int MT, int EPI>
__device__ __forceinline__ void gemv_prefetch(const GemvParams& p, EpiloguePrefetch<MT, EPI>& pre,
                                              int tile, int lane) {
    const int c16 = lane & 15, q = lane >> 4;
    const int n = min(tile * 16 + c16, p.N - 1);
    if (EPI == E_RESIDUAL) {
#pragma unroll
        for (int mt = 0; mt < MT; ++mt)
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                const int m = min(mt * 16 + 4 * q + r, p.M - 1);
                pre.old[mt][r] = static_cast<const float*>(p.out)[static_cast<size_t>(m) * p.ldo + n];
            }
    }
    if (EPI == E_CONV) {
#pragma unroll
        for (int t = 0; t < CONV_PREFETCH_TAPS; ++t)
            pre.taps[t] = t < p.taps ? p.conv_w[static_cast<size_t>(n) * p.taps + t] : 0.f;
#pragma unroll
        for (int mt = 0; mt < MT; ++mt)
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                const int m = min(mt * 16 + 4 * q + r, p.M - 1);
                const float* st = p.state + static_cast<size_t>(p.seq_slot[m]) * p.state_slot_stride + n;
#pragma unroll
                for (int t = 0; t < CONV_PREFETCH_TAPS - 1; ++t)
                    pre.state[mt][r][t] = t + 1 < p.taps ? st[static_cast<size_t>(t + 1) * p.N] : 0.f;
            }
    }
}

// ---- epilogue of one 16-column tile: this lane holds column n0 + lane%16 of rows
// 4*(lane/16)..+3 of every row tile
template <int MT, int NS, int EPI>
__device__ __forceinline__ void gemv_epilogue(const GemvParams& p, floatx4_t (&acc)[MT][NS],
                                              const EpiloguePrefetch<MT, EPI>& pre,
                                              int tile, int lane) {
    const int c16 = lane & 15, q = lane >> 4;
    const int M = p.M;
    const int n = tile * 16 + c16;
    const bool col_ok = n < p.N;
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) {
        float sq[4] = {0.f, 0.f, 0.f, 0.f};
        unsigned long long best[4] = {0ull, 0ull, 0ull, 0ull};
#pragma unroll
        for (int r = 0; r < 4; ++r) {
            const int m = mt * 16 + 4 * q + r;
            const bool ok = col_ok && m < M;
            if (EPI == E_STORE || EPI == E_STORE_F32) {
                const float v = acc[mt][0][r] + (p.bias && ok ? p.bias[n] : 0.f);
                if (EPI == E_STORE_F32 && p.row_best) best[r] = group_best_logit<16>(v, ok, tile * 16);
                if (ok) {
                    if (EPI == E_STORE) static_cast<bf16*>(p.out)[static_cast<size_t>(m) * p.ldo + n] = from_float<bf16>(v);
                    else static_cast<float*>(p.out)[static_cast<size_t>(m) * p.ldo + n] = v;
                }
            } else if (EPI == E_RESIDUAL) {
                if (ok) {
                    float* hp = static_cast<float*>(p.out) + static_cast<size_t>(m) * p.ldo + n;
                    // the product enters the sum rounded to bfloat16, as when it is stored first
                    const float v = pre.old[mt][r] + round_bf16(acc[mt][0][r] + (p.bias ? p.bias[n] : 0.f));
                    *hp = v;
                    sq[r] = v * v;
                }
            } else if (EPI == E_SWIGLU) {
                if (ok) {
                    const float g = round_bf16(acc[mt][0][r]), u = round_bf16(acc[mt][1][r]);
                    static_cast<bf16*>(p.out)[static_cast<size_t>(m) * p.ldo + n] =
                        from_float<bf16>((g / (1.0f + expf(-g))) * u);
                }
            } else if (EPI == E_CONV) {
                if (ok) {
                    const float bb = round_bf16(acc[mt][0][r] + (p.bias ? p.bias[n] : 0.f));
                    const float cc = round_bf16(acc[mt][1][r] + (p.bias ? p.bias[p.stream_rows + n] : 0.f));
                    const float xx = round_bf16(acc[mt][2][r] + (p.bias ? p.bias[2 * p.stream_rows + n] : 0.f));
                    const float bx = bb * xx;
                    float* st = p.state + static_cast<size_t>(p.seq_slot[m]) * p.state_slot_stride + n;
                    float conv = 0.f;
#pragma unroll
                    for (int tap = 0; tap < CONV_PREFETCH_TAPS - 1; ++tap) {
                        if (tap + 1 < p.taps) {
                            const float old = pre.state[mt][r][tap];
                            conv = fmaf(pre.taps[tap], old, conv);
                            st[static_cast<size_t>(tap) * p.N] = old;     // shift by one position
                        }
                    }
                    float last_tap = 0.f;
#pragma unroll
                    for (int tap = 0; tap < CONV_PREFETCH_TAPS; ++tap)
                        if (tap == p.taps - 1) last_tap = pre.taps[tap];
                    conv = fmaf(last_tap, bx, conv);
                    st[static_cast<size_t>(p.taps - 1) * p.N] = bx;
                    if (p.conv_b) conv += p.conv_b[n];
                    static_cast<bf16*>(p.out)[static_cast<size_t>(m) * p.ldo + n] = from_float<bf16>(cc * conv);
                }
            }
        }
        if (EPI == E_STORE_F32 && p.row_best) {
            // the best of the tile's 16 columns, row by row: one part of the row
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                const int m = mt * 16 + 4 * q + r;
                if (c16 == 0 && m < M) p.row_best[static_cast<size_t>(m) * p.row_best_ld + tile] = best[r];
            }
        }
        if (EPI == E_RESIDUAL && p.stats_out) {
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                float s = sq[r];
                s += __shfl_xor(s, 1, 64);
                s += __shfl_xor(s, 2, 64);
                s += __shfl_xor(s, 4, 64);
                s += __shfl_xor(s, 8, 64);
                const int m = mt * 16 + 4 * q + r;
                if (c16 == 0 && m < M)
                    p.stats_out[static_cast<size_t>(m) * p.stats_ld_out + tile] = s;
            }
        }
    }
}

// A workgroup of TW*KW wavefronts: wavefront (tw, kw) works on column tile
// blockIdx.x*TW + tw and on the kw-th share of K.  ALDS: the rows of A (normalised, if
// asked) are put into LDS once per workgroup as bfloat16 and every wavefront reads its
// operands from there; otherwise every wavefront reads (and normalises) them itself.
// Dynamic LDS: [partial tiles (KW > 1)] [1/rms of the rows] [rows of A (ALDS)].
template <int MT, int TW, int KW, int AMODE, int EPI, int ALDS>
__global__ __launch_bounds__(TW * KW * 64) void gemv_fused_kernel(const GemvParams p) {
    constexpr int NS = Streams<EPI>::n;
    constexpr int NW = TW * KW;
    constexpr int RED = KW > 1 ? NW * MT * NS * 64 : 0;   // floatx4 entries
    extern __shared__ __attribute__((aligned(16))) unsigned char lds_raw[];
    floatx4_t* red = reinterpret_cast<floatx4_t*>(lds_raw);
    float* inv_rms = reinterpret_cast<float*>(lds_raw + static_cast<size_t>(RED) * 16);
    bf16* xs = reinterpret_cast<bf16*>(lds_raw + static_cast<size_t>(RED) * 16 + 64 * sizeof(float));
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
    const int c16 = lane & 15, q = lane >> 4;
    const int tw = wave / KW, kw = wave % KW;
    const int K = p.K, M = p.M;
    const int ldx = K + 8;          // row stride in LDS: 16 bytes more than a row
    const int tile = blockIdx.x * TW + tw;
    const bool tile_ok = tile * 16 < p.N;

    floatx4_t acc[MT][NS];
#pragma unroll
    for (int mt = 0; mt < MT; ++mt)
#pragma unroll
        for (int s = 0; s < NS; ++s) acc[mt][s] = floatx4_t{0.f, 0.f, 0.f, 0.f};

    // element (n, k) of w lies at n * w_row_stride + (k / 32) * w_kb_stride + k % 32: rows one after
    // the other (K, 32), or [K/32, rows, 32] (32, rows * 32), where the 16 weight rows of a tile are
    // a kilobyte in a row for every block of 32 values of k: an output head of 65,536 rows then
    // reads whole kilobytes instead of 64 bytes of each of 16 rows that lie kilobytes apart (rows
    // of 2,048 values, 8 rows of A: 54.6 against 62.4 us; rows of 1,024 values: no difference)
    const size_t w_row_stride = static_cast<size_t>(p.w_row_stride), w_kb_stride = static_cast<size_t>(p.w_kb_stride);
    const bf16* wrow[NS];
#pragma unroll
    for (int s = 0; s < NS; ++s)
        wrow[s] = p.w + (static_cast<size_t>(s) * p.stream_rows + min(tile * 16 + c16, p.N - 1)) * w_row_stride;

    // K is cut in chunks of 64 which are dealt to the KW wavefronts of a tile.  Inside a
    // chunk, lane group q holds the k values {q*8..q*8+7} and {32+q*8..32+q*8+7}: each of
    // the two 16-byte loads of a lane is side by side with its neighbours' in the row.
    // U chunks of weights are loaded before any is multiplied, and the first U are asked
    // for before the rows of A are prepared, so that memory latency and that work overlap.
    constexpr int U = ALDS ? (MT * NS <= 2 ? 8 : (MT * NS <= 4 ? 4 : 2))
                           : (MT == 1 ? 4 : (MT == 2 ? 2 : 1));
    const int chunks = (K + 63) >> 6;
    const int c_begin = tile_ok ? kw * chunks / KW : 0, c_end = tile_ok ? (kw + 1) * chunks / KW : 0;
    EpiloguePrefetch<MT, EPI> pre;
    if (kw == 0 && tile_ok) gemv_prefetch<MT, EPI>(p, pre, tile, lane);
    Frag2 wv[U][NS][2];
    auto load_weights = [&](int c0) {
#pragma unroll
        for (int u = 0; u < U; ++u)
#pragma unroll
            for (int v = 0; v < 2; ++v) {
                const int k = (c0 + u) * 64 + v * 32 + q * 8;   // 8 values from here
                const bool in = c0 + u < c_end && k + 8 <= K;    // K % 8 == 0
#pragma unroll
                for (int s = 0; s < NS; ++s)
                    // (8 values from k on never leave a block of 32)
                    wv[u][s][v] = in ? *reinterpret_cast<const Frag2*>(wrow[s] + static_cast<size_t>(k >> 5) * w_kb_stride + (k & 31)) : Frag2{};
            }
    };
    // ---- rows of A: 1/rms (A_NORM), and the rows themselves into LDS (ALDS); one wavefront
    // per row.  Loads come back in the order they were asked for, so the (cached) rows of A
    // are asked for first and the weights right after: preparing the rows then overlaps
    // with the weights' way from memory instead of waiting behind it.
    if (AMODE == A_NORM || ALDS) {
        constexpr int RV = AMODE == A_NORM ? 4 : 8;   // 16-byte loads of a row kept in flight
        floatx4_t hv4[AMODE == A_NORM ? 4 : 1], nw4[AMODE == A_NORM ? 4 : 1];
        Frag2 rv[AMODE == A_NORM ? 1 : RV];
        float s = 0.f;
        bool weights_asked = false;
        for (int m = wave; m < M || !weights_asked; m += NW) {
            const bool row_ok = m < M;
            const size_t src = row_ok ? static_cast<size_t>(p.rows ? p.rows[m] : m) : 0;
            if (AMODE == A_NORM) {
                const float* row = static_cast<const float*>(p.a) + src * p.lda;
                s = 0.f;
                if (p.stats && row_ok) {
                    for (int j = lane; j < p.n_stat_blocks; j += 64)
                        s += p.stats[src * p.stats_ld + j];
                }
                float inv = 0.f;
                for (int k0 = 0; k0 < K; k0 += 1024) {
#pragma unroll
                    for (int i = 0; i < 4; ++i) {
                        const int k = k0 + i * 256 + lane * 4;
                        const bool in = row_ok && k < K;
                        hv4[i] = in ? *reinterpret_cast<const floatx4_t*>(row + k) : floatx4_t{};
                        if (ALDS) nw4[i] = in ? *reinterpret_cast<const floatx4_t*>(p.norm_w + k) : floatx4_t{};
                    }
                    if (!weights_asked) { load_weights(c_begin); weights_asked = true; }
                    if (!row_ok) break;
                    if (k0 == 0) {
                        if (!p.stats) {   // no partial sums were left: walk the row
                            if (K <= 1024) {
#pragma unroll
                                for (int i = 0; i < 4; ++i)
                                    s += hv4[i][0] * hv4[i][0] + hv4[i][1] * hv4[i][1] +
                                         hv4[i][2] * hv4[i][2] + hv4[i][3] * hv4[i][3];
                            } else {
                                for (int k = lane * 4; k < K; k += 256) {
                                    const floatx4_t v = *reinterpret_cast<const floatx4_t*>(row + k);
                                    s += v[0] * v[0] + v[1] * v[1] + v[2] * v[2] + v[3] * v[3];
                                }
                            }
                        }
                        s = wave_sum(s);
                        inv = 1.0f / sqrtf(s / static_cast<float>(K) + p.eps);
                        if (lane == 0) inv_rms[m] = inv;
                        if (!ALDS) break;
                    }
#pragma unroll
                    for (int i = 0; i < 4; ++i) {
                        const int k = k0 + i * 256 + lane * 4;
                        if (k < K)
                            *reinterpret_cast<bf16x4_t*>(xs + static_cast<size_t>(m) * ldx + k) =
                                __builtin_bit_cast(bf16x4_t, __builtin_convertvector(hv4[i] * inv * nw4[i], nbf16x4_t));
                    }
                }
            } else {
                const bf16* row = static_cast<const bf16*>(p.a) + src * p.lda;
                for (int k0 = 0; k0 < K; k0 += 512 * RV) {
#pragma unroll
                    for (int i = 0; i < RV; ++i) {
                        const int k = k0 + i * 512 + lane * 8;
                        rv[i] = (row_ok && k < K) ? *reinterpret_cast<const Frag2*>(row + k) : Frag2{};
                    }
                    if (!weights_asked) { load_weights(c_begin); weights_asked = true; }
                    if (!row_ok) break;
#pragma unroll
                    for (int i = 0; i < RV; ++i) {
                        const int k = k0 + i * 512 + lane * 8;
                        if (k < K) *reinterpret_cast<Frag2*>(xs + static_cast<size_t>(m) * ldx + k) = rv[i];
                    }
                }
            }
        }
        __syncthreads();
    } else {
        load_weights(c_begin);
    }

    // the row of A this lane feeds in every row tile (rows beyond M repeat the last one;
    // their results are dropped)
    size_t a_off[MT];
    float a_inv[MT];
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) {
        const int m = min(mt * 16 + c16, M - 1);
        a_off[mt] = ALDS ? static_cast<size_t>(m) * ldx
                         : static_cast<size_t>(p.rows ? p.rows[m] : m) * p.lda;
        a_inv[mt] = (AMODE == A_NORM && !ALDS) ? inv_rms[m] : 1.f;
    }

    for (int c0 = c_begin; c0 < c_end;) {
        Frag2 av[ALDS ? 1 : U][MT][2];            // rows read from memory: bfloat16
        floatx4_t hv[ALDS ? 1 : U][MT][4];        //   or 32-bit, to be normalised
        floatx4_t nv[ALDS ? 1 : U][4];
        if (!ALDS) {
#pragma unroll
            for (int u = 0; u < U; ++u)
#pragma unroll
                for (int v = 0; v < 2; ++v) {
                    const int k = (c0 + u) * 64 + v * 32 + q * 8;
                    const bool in = c0 + u < c_end && k + 8 <= K;
#pragma unroll
                    for (int mt = 0; mt < MT; ++mt) {
                        if (AMODE == A_BF16) {
                            av[u][mt][v] = in ? *reinterpret_cast<const Frag2*>(
                                                    static_cast<const bf16*>(p.a) + a_off[mt] + k)
                                              : Frag2{};
                        } else {
                            const float* hr = static_cast<const float*>(p.a) + a_off[mt] + k;
                            hv[u][mt][2 * v] = in ? *reinterpret_cast<const floatx4_t*>(hr) : floatx4_t{};
                            hv[u][mt][2 * v + 1] = in ? *reinterpret_cast<const floatx4_t*>(hr + 4) : floatx4_t{};
                        }
                    }
                    if (AMODE == A_NORM) {
                        nv[u][2 * v] = in ? *reinterpret_cast<const floatx4_t*>(p.norm_w + k) : floatx4_t{};
                        nv[u][2 * v + 1] = in ? *reinterpret_cast<const floatx4_t*>(p.norm_w + k + 4) : floatx4_t{};
                    }
                }
        }
#pragma unroll
        for (int u = 0; u < U; ++u) {
            bf16x4_t af[MT][4];
#pragma unroll
            for (int mt = 0; mt < MT; ++mt) {
                if (ALDS) {
#pragma unroll
                    for (int v = 0; v < 2; ++v) {
                        const int k = min((c0 + u) * 64 + v * 32 + q * 8, K - 8);   // stay inside the row
                        const Frag2 f = *reinterpret_cast<const Frag2*>(xs + a_off[mt] + k);
                        af[mt][2 * v] = f.lo;
                        af[mt][2 * v + 1] = f.hi;
                    }
                } else if (AMODE == A_BF16) {
                    af[mt][0] = av[u][mt][0].lo; af[mt][1] = av[u][mt][0].hi;
                    af[mt][2] = av[u][mt][1].lo; af[mt][3] = av[u][mt][1].hi;
                } else {
#pragma unroll
                    for (int s4 = 0; s4 < 4; ++s4)
                        af[mt][s4] = __builtin_bit_cast(
                            bf16x4_t, __builtin_convertvector(hv[u][mt][s4] * a_inv[mt] * nv[u][s4], nbf16x4_t));
                }
            }
#pragma unroll
            for (int s = 0; s < NS; ++s) {
                const bf16x4_t bfr[4] = {wv[u][s][0].lo, wv[u][s][0].hi, wv[u][s][1].lo, wv[u][s][1].hi};
#pragma unroll
                for (int s4 = 0; s4 < 4; ++s4)
#pragma unroll
                    for (int mt = 0; mt < MT; ++mt)
                        acc[mt][s] = __builtin_amdgcn_mfma_f32_16x16x16bf16_1k(af[mt][s4], bfr[s4], acc[mt][s], 0, 0, 0);
            }
        }
        c0 += U;
        if (c0 < c_end) load_weights(c0);
    }

    // ---- add the partial tiles of the KW wavefronts of a tile, in their order
    if (KW > 1) {
#pragma unroll
        for (int mt = 0; mt < MT; ++mt)
#pragma unroll
            for (int s = 0; s < NS; ++s) red[(wave * MT * NS + mt * NS + s) * 64 + lane] = acc[mt][s];
        __syncthreads();
        if (kw != 0) return;
#pragma unroll
        for (int mt = 0; mt < MT; ++mt)
#pragma unroll
            for (int s = 0; s < NS; ++s) {
                floatx4_t t = red[(wave * MT * NS + mt * NS + s) * 64 + lane];
                for (int w = 1; w < KW; ++w) t += red[((wave + w) * MT * NS + mt * NS + s) * 64 + lane];
                acc[mt][s] = t;
            }
    }
    if (!tile_ok) return;
    gemv_epilogue<MT, NS, EPI>(p, acc, pre, tile, lane);
}

static size_t gemv_lds_bytes(int mt, int tw, int kw, int streams, int alds, int m, int k) {
    size_t bytes = 64 * sizeof(float);
    if (kw > 1) bytes += static_cast<size_t>(tw) * kw * mt * streams * 64 * 16;
    if (alds) bytes += static_cast<size_t>(m) * (k + 8) * 2;
    return bytes;
}

template <int MT, int TW, int KW, int ALDS>
static int launch_shape(const GemvParams& p, int amode, int epi, hipStream_t stream) {
    const int tiles = (p.N + 15) / 16;
    dim3 grid((tiles + TW - 1) / TW), block(TW * KW * 64);
    const int streams = epi == E_SWIGLU ? 2 : (epi == E_CONV ? 3 : 1);
    const size_t lds = gemv_lds_bytes(MT, TW, KW, streams, ALDS, p.M, p.K);
#define CELEG_GEMV(AM, EP)                                                                       \
    do {                                                                                         \
        auto kernel = gemv_fused_kernel<MT, TW, KW, AM, EP, ALDS>;                               \
        if (lds > 48 * 1024) {                                                                   \
            hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(kernel),            \
                                               hipFuncAttributeMaxDynamicSharedMemorySize,       \
                                               static_cast<int>(lds));                           \
            if (e != hipSuccess) return static_cast<int>(e);                                     \
        }                                                                                        \
        hipLaunchKernelGGL(kernel, grid, block, lds, stream, p);                                 \
    } while (0)
    if (amode == A_BF16) {
        switch (epi) {
            case E_STORE: CELEG_GEMV(A_BF16, E_STORE); break;
            case E_STORE_F32: CELEG_GEMV(A_BF16, E_STORE_F32); break;
            case E_RESIDUAL: CELEG_GEMV(A_BF16, E_RESIDUAL); break;
            default: return static_cast<int>(hipErrorInvalidValue);
        }
    } else {
        switch (epi) {
            case E_STORE: CELEG_GEMV(A_NORM, E_STORE); break;
            case E_STORE_F32: CELEG_GEMV(A_NORM, E_STORE_F32); break;
            case E_SWIGLU: CELEG_GEMV(A_NORM, E_SWIGLU); break;
            case E_CONV: CELEG_GEMV(A_NORM, E_CONV); break;
            default: return static_cast<int>(hipErrorInvalidValue);
        }
    }
#undef CELEG_GEMV
    return CELEG_LAUNCH_RESULT();
}

// The shape of the workgroup follows the number of column tiles: many tiles, one
// wavefront a tile over all of K (8 tiles a workgroup); few tiles, 8 (or 4) wavefronts
// share a tile's K.  The rows of A go through LDS when they fit (up to 144 KiB).
// shape: 0 lets the tile count decide; 1..4 force (TW, KW) = (8,1), (2,4), (1,8), (1,4) (for
// up to 16 rows; a tuning aid).
extern "C" int celeg_gemv_fused(const GemvParams* params, int amode, int epi, int shape,
                                hipStream_t stream) {
    const GemvParams& p = *params;
    if (p.M <= 0 || p.N <= 0) return 0;
    if (p.M > 64 || p.K <= 0 || (p.K % 8) || (p.lda % 8)) return static_cast<int>(hipErrorInvalidValue);
    if (epi == E_CONV && (p.taps < 1 || p.taps > CONV_PREFETCH_TAPS || p.stream_rows != p.N))
        return static_cast<int>(hipErrorInvalidValue);
    // (the weights' layout: rows one after the other, or blocks of 32 values of k with the rows side by side)
    if (p.w_row_stride <= 0 || p.w_kb_stride <= 0 || (p.w_row_stride % 8) || (p.w_kb_stride % 8) ||
        (p.w_kb_stride != 32 && (p.K % 32)))
        return static_cast<int>(hipErrorInvalidValue);
    const int tiles = (p.N + 15) / 16, chunks = (p.K + 63) / 64;
    if (p.row_best && (epi != E_STORE_F32 || p.row_best_rows < p.M || p.row_best_ld < tiles)) return static_cast<int>(hipErrorInvalidValue);
    const int streams = epi == E_SWIGLU ? 2 : (epi == E_CONV ? 3 : 1);
    const int mt = p.M <= 16 ? 1 : (p.M <= 32 ? 2 : 4);
    const size_t limit = 144 * 1024;
#define CELEG_SHAPE(MT_, TW_, KW_)                                                               \
    (gemv_lds_bytes(MT_, TW_, KW_, streams, 1, p.M, p.K) <= limit                                \
         ? launch_shape<MT_, TW_, KW_, 1>(p, amode, epi, stream)                                 \
         : launch_shape<MT_, 1, 4, 0>(p, amode, epi, stream))
    if (mt == 1) {
        if (shape == 1) return CELEG_SHAPE(1, 8, 1);
        if (shape == 2) return CELEG_SHAPE(1, 2, 4);
        if (shape == 3) return CELEG_SHAPE(1, 1, 8);
        if (shape == 4) return CELEG_SHAPE(1, 1, 4);
        if (tiles >= 2048) return CELEG_SHAPE(1, 8, 1);
        // two tiles a workgroup (they share the prepared rows) once there are enough tiles
        // and K is short enough that four wavefronts a tile keep their loads in one batch
        if (tiles >= 512 || (tiles >= 128 && chunks <= 32)) return CELEG_SHAPE(1, 2, 4);
        if (chunks >= 8) return CELEG_SHAPE(1, 1, 8);
        return CELEG_SHAPE(1, 1, 4);
    }
    if (mt == 2) {
        if (tiles >= 2048) return CELEG_SHAPE(2, 8, 1);
        if (tiles >= 512 || (tiles >= 128 && chunks <= 32)) return CELEG_SHAPE(2, 2, 4);
        return CELEG_SHAPE(2, 1, 4);
    }
    if (tiles >= 2048) return CELEG_SHAPE(4, 8, 1);
    return CELEG_SHAPE(4, 1, 4);
#undef CELEG_SHAPE
}

// Embedding gather that also leaves the sum of squares of every row, for the first norm:
// out[row, :] = table[ids[row], :] (32-bit), stats[row * stats_ld] = sum(out[row, :]^2).
__global__ void embed_stats_kernel(const bf16* __restrict__ table, const int* __restrict__ ids,
                                   float* __restrict__ out, float* __restrict__ stats, int stats_ld,
                                   int width, int vocab) {
    __shared__ float scratch[16];
    const int row = blockIdx.x;
    const int id = ids[row];
    float* dst = out + static_cast<size_t>(row) * width;
    float s = 0.f;
    if (id >= 0 && id < vocab) {
        const bf16* src = table + static_cast<size_t>(id) * width;
        for (int i = threadIdx.x; i < width; i += blockDim.x) {
            const float v = to_float(src[i]);
            dst[i] = v;
            s += v * v;
        }
    } else {
        for (int i = threadIdx.x; i < width; i += blockDim.x) dst[i] = 0.f;
    }
    s = block_sum(s, scratch);
    if (threadIdx.x == 0) stats[static_cast<size_t>(row) * stats_ld] = s;
}

extern "C" int celeg_embed_stats(const void* table, const int* ids, float* out, float* stats, int stats_ld,
                                 int rows, int width, int vocab, hipStream_t stream) {
    if (rows <= 0) return 0;
    hipLaunchKernelGGL(embed_stats_kernel, dim3(rows), dim3(256), 0, stream,
                       static_cast<const bf16*>(table), ids, out, stats, stats_ld, width, vocab);
    return CELEG_LAUNCH_RESULT();
}
