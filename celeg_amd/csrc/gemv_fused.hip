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

typedef short bf16x4_t __attribute__((ext_vector_type(4)));
typedef float floatx4_t __attribute__((ext_vector_type(4)));
typedef __bf16 nbf16x4_t __attribute__((ext_vector_type(4)));
struct __attribute__((aligned(16))) Frag2 {   // 16 bytes = 8 bfloat16 = two MFMA operands
    bf16x4_t lo, hi;
};

enum { A_BF16 = 0, A_NORM = 1 };
enum { E_STORE = 0, E_STORE_F32 = 1, E_RESIDUAL = 2, E_SWIGLU = 3, E_CONV = 4 };

struct GemvParams {
    // A side
    const void* a;          // bf16 [M, lda] or float [*, lda]
    int lda;
    const int* rows;        // optional: A row of output row m is rows[m]
    const float* norm_w;    // A_NORM: [K]
    float eps;
    const float* stats;     // A_NORM: [n_stat_blocks, stats_ld] partial sums of squares, or null
    int n_stat_blocks, stats_ld;
    // weights: stream s starts at row s * stream_rows
    const bf16* w;
    int stream_rows;
    const float* bias;      // optional [streams * stream_rows]
    int M, N, K;
    // outputs
    void* out;              // bf16 or float [M, ldo]; E_RESIDUAL: the residual stream itself
    int ldo;
    float* stats_out;       // E_RESIDUAL: [gridDim.x, stats_ld_out] or null
    int stats_ld_out;
    // E_CONV
    const float* conv_w;    // [N, taps]
    const float* conv_b;    // optional [N]
    float* state;           // [slots, taps, N]
    size_t state_slot_stride;
    const int* seq_slot;    // [M]
    int taps;
};

__device__ __forceinline__ short to_bits(float x) { return static_cast<short>(from_float<bf16>(x).bits); }
__device__ __forceinline__ float round_bf16(float x) { return to_float(from_float<bf16>(x)); }

template <int EPI> struct Streams { static constexpr int n = 1; };
template <> struct Streams<E_SWIGLU> { static constexpr int n = 2; };
template <> struct Streams<E_CONV> { static constexpr int n = 3; };

template <int MT, int NW, int AMODE, int EPI>
__global__ __launch_bounds__(NW * 64) void gemv_fused_kernel(const GemvParams p) {
    constexpr int NS = Streams<EPI>::n;
    __shared__ floatx4_t red[NW][MT * NS][64];
    __shared__ float inv_rms[MT * 16];
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
    const int c16 = lane & 15, q = lane >> 4;
    const int n0 = blockIdx.x * 16;
    const int K = p.K, M = p.M;

    // ---- A_NORM: 1/rms of every row
    if (AMODE == A_NORM) {
        const float* h = static_cast<const float*>(p.a);
        if (p.stats) {
            // one wavefront per row; its lanes read the partial sums side by side
            for (int m = wave; m < MT * 16; m += NW) {
                float s = 0.f;
                if (m < M) {
                    const int src = p.rows ? p.rows[m] : m;
                    for (int j = lane; j < p.n_stat_blocks; j += 64)
                        s += p.stats[static_cast<size_t>(j) * p.stats_ld + src];
                }
                s = wave_sum(s);
                if (lane == 0) inv_rms[m] = 1.0f / sqrtf(s / static_cast<float>(K) + p.eps);
            }
        } else {
            // one wavefront per row, rows dealt round robin
            for (int m = wave; m < MT * 16; m += NW) {
                float s = 0.f;
                if (m < M) {
                    const float* row = h + static_cast<size_t>(p.rows ? p.rows[m] : m) * p.lda;
                    for (int k = lane; k < K; k += 64) s += row[k] * row[k];
                }
                s = wave_sum(s);
                if (lane == 0) inv_rms[m] = 1.0f / sqrtf(s / static_cast<float>(K) + p.eps);
            }
        }
        __syncthreads();
    }

    floatx4_t acc[MT][NS];
#pragma unroll
    for (int mt = 0; mt < MT; ++mt)
#pragma unroll
        for (int s = 0; s < NS; ++s) acc[mt][s] = floatx4_t{0.f, 0.f, 0.f, 0.f};

    // rows of A this lane feeds (one per row tile) and their 1/rms
    size_t a_off[MT];
    float a_inv[MT];
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) {
        const int m = min(mt * 16 + c16, M - 1);
        a_off[mt] = static_cast<size_t>(p.rows ? p.rows[m] : m) * p.lda;
        a_inv[mt] = AMODE == A_NORM ? inv_rms[mt * 16 + c16 < M ? mt * 16 + c16 : M - 1] : 1.f;
    }
    const bf16* wrow[NS];
#pragma unroll
    for (int s = 0; s < NS; ++s)
        wrow[s] = p.w + (static_cast<size_t>(s) * p.stream_rows + min(n0 + c16, p.N - 1)) * K;

    // K is cut in chunks of 64 which are dealt to the wavefronts.  Inside a chunk, lane
    // group q holds the k values {q*8..q*8+7} and {32+q*8..32+q*8+7}: each of the two
    // 16-byte loads of a lane is then side by side with its neighbours' in the row.  U chunks
    // are loaded before any is multiplied, so that several loads are in flight.
    constexpr int U = MT == 1 ? 4 : (MT == 2 ? 2 : 1);
    const int chunks = (K + 63) >> 6;
    const int c_begin = wave * chunks / NW, c_end = (wave + 1) * chunks / NW;
    for (int c0 = c_begin; c0 < c_end; c0 += U) {
        Frag2 wv[U][NS][2];
        Frag2 av[U][MT][2];          // A_BF16
        floatx4_t hv[U][MT][4];      // A_NORM
        floatx4_t nv[U][4];
#pragma unroll
        for (int u = 0; u < U; ++u) {
            const bool live = c0 + u < c_end;
#pragma unroll
            for (int v = 0; v < 2; ++v) {
                const int k = (c0 + u) * 64 + v * 32 + q * 8;   // 8 values from here
                const bool in = live && k + 8 <= K;              // K % 8 == 0
#pragma unroll
                for (int s = 0; s < NS; ++s)
                    wv[u][s][v] = in ? *reinterpret_cast<const Frag2*>(wrow[s] + k) : Frag2{};
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
                if (AMODE == A_BF16) {
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
    }

    // ---- add the wavefronts' partial tiles, in wavefront order
#pragma unroll
    for (int mt = 0; mt < MT; ++mt)
#pragma unroll
        for (int s = 0; s < NS; ++s) red[wave][mt * NS + s][lane] = acc[mt][s];
    __syncthreads();
    if (wave != 0) return;
#pragma unroll
    for (int mt = 0; mt < MT; ++mt)
#pragma unroll
        for (int s = 0; s < NS; ++s) {
            floatx4_t t = red[0][mt * NS + s][lane];
            for (int w = 1; w < NW; ++w) t += red[w][mt * NS + s][lane];
            acc[mt][s] = t;
        }

    // ---- epilogue: this lane holds column n of rows 4q..4q+3 of every row tile
    const int n = n0 + c16;
    const bool col_ok = n < p.N;
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) {
        float sq[4] = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int r = 0; r < 4; ++r) {
            const int m = mt * 16 + 4 * q + r;
            const bool ok = col_ok && m < M;
            if (EPI == E_STORE || EPI == E_STORE_F32) {
                const float v = acc[mt][0][r] + (p.bias && ok ? p.bias[n] : 0.f);
                if (ok) {
                    if (EPI == E_STORE) static_cast<bf16*>(p.out)[static_cast<size_t>(m) * p.ldo + n] = from_float<bf16>(v);
                    else static_cast<float*>(p.out)[static_cast<size_t>(m) * p.ldo + n] = v;
                }
            } else if (EPI == E_RESIDUAL) {
                if (ok) {
                    float* hp = static_cast<float*>(p.out) + static_cast<size_t>(m) * p.ldo + n;
                    // the product enters the sum rounded to bfloat16, as when it is stored first
                    const float v = *hp + round_bf16(acc[mt][0][r] + (p.bias ? p.bias[n] : 0.f));
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
                    const float* cw = p.conv_w + static_cast<size_t>(n) * p.taps;
                    float conv = 0.f;
                    for (int tap = 0; tap + 1 < p.taps; ++tap) {
                        const float old = st[static_cast<size_t>(tap + 1) * p.N];
                        conv = fmaf(cw[tap], old, conv);
                        st[static_cast<size_t>(tap) * p.N] = old;     // shift by one position
                    }
                    conv = fmaf(cw[p.taps - 1], bx, conv);
                    st[static_cast<size_t>(p.taps - 1) * p.N] = bx;
                    if (p.conv_b) conv += p.conv_b[n];
                    static_cast<bf16*>(p.out)[static_cast<size_t>(m) * p.ldo + n] = from_float<bf16>(cc * conv);
                }
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
                    p.stats_out[static_cast<size_t>(blockIdx.x) * p.stats_ld_out + m] = s;
            }
        }
    }
}

template <int MT, int NW>
static int launch_mt_nw(const GemvParams& p, int amode, int epi, hipStream_t stream) {
    dim3 grid((p.N + 15) / 16), block(NW * 64);
#define CELEG_GEMV(AM, EP)                                                                      \
    hipLaunchKernelGGL((gemv_fused_kernel<MT, NW, AM, EP>), grid, block, 0, stream, p)
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

template <int MT>
static int launch_mt(const GemvParams& p, int amode, int epi, int waves, hipStream_t stream) {
    if (waves == 8 && MT <= 2) return launch_mt_nw<(MT <= 2 ? MT : 1), 8>(p, amode, epi, stream);
    if (waves == 4 || waves == 8) return launch_mt_nw<MT, 4>(p, amode, epi, stream);
    return static_cast<int>(hipErrorInvalidValue);
}

// waves: wavefronts per workgroup that split K: 4, or 8 (which is honoured up to 32 rows).
extern "C" int celeg_gemv_fused(const GemvParams* params, int amode, int epi, int waves,
                                hipStream_t stream) {
    const GemvParams& p = *params;
    if (p.M <= 0 || p.N <= 0) return 0;
    if (p.M > 64 || p.K <= 0 || (p.K % 8) || (p.lda % 8)) return static_cast<int>(hipErrorInvalidValue);
    if (epi == E_CONV && (p.taps < 1 || p.stream_rows != p.N)) return static_cast<int>(hipErrorInvalidValue);
    const int mt = (p.M + 15) / 16;
    switch (mt) {
        case 1: return launch_mt<1>(p, amode, epi, waves, stream);
        case 2: return launch_mt<2>(p, amode, epi, waves, stream);
        case 3: return launch_mt<3>(p, amode, epi, waves, stream);
        default: return launch_mt<4>(p, amode, epi, waves, stream);
    }
}

// Embedding gather that also leaves the sum of squares of every row, for the first norm:
// out[row, :] = table[ids[row], :] (32-bit), stats[row] = sum(out[row, :]^2).
__global__ void embed_stats_kernel(const bf16* __restrict__ table, const int* __restrict__ ids,
                                   float* __restrict__ out, float* __restrict__ stats, int width,
                                   int vocab) {
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
    if (threadIdx.x == 0) stats[row] = s;
}

extern "C" int celeg_embed_stats(const void* table, const int* ids, float* out, float* stats,
                                 int rows, int width, int vocab, hipStream_t stream) {
    if (rows <= 0) return 0;
    hipLaunchKernelGGL(embed_stats_kernel, dim3(rows), dim3(256), 0, stream,
                       static_cast<const bf16*>(table), ids, out, stats, width, vocab);
    return CELEG_LAUNCH_RESULT();
}
