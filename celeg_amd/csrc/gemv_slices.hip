// Skinny bfloat16 products for up to 16 rows on gfx950 (decode steps), with what
// surrounds them fused in:
//   out[M,N] = epilogue(scale[m] * (A[M,K] W[N,K]^T) + bias)
// A is bfloat16.  For a product behind an RMSNorm, A is the bfloat16 copy of the residual
// stream, W has the norm's weight folded into its columns by the caller, and scale[m] =
// rsqrt(mean(x_m^2) + eps) is taken from the partial sums of squares that the producer of
// the stream left; the scaling is applied to the 32-bit sums at the end.
// Epilogues: store | 32-bit store | add into the 32-bit residual stream, refresh its
// bfloat16 copy and leave partial sums of squares | SwiGLU of a gate and an up stream |
// the double-gated short convolution of a B, a C and an x stream for one new token per
// request, with its state update.
//
// Layout.  These products have few rows and are bound by memory latency and by how much
// of the chip takes part, so the 16x16 tile of the MFMA is cut in G x G blocks of MP x MP
// (MP = 16 / G >= M): the instruction's row index is (k-slice g, row m) and its column
// index (k-slice g', column j); A rows of slice g hold A[m, g*K/G + k] and B columns of
// slice g' hold W[n0 + j, g'*K/G + k], so the diagonal blocks g == g' are G partial
// products over G parts of K for the same MP x MP outputs, and the others are dropped.  A
// workgroup then owns only MP columns (of every weight stream) - G times as many
// workgroups -, every lane's loads are useful when M == MP, and the rows of A are read
// from cache straight into the instruction's operand layout (no staging, no barrier
// before the products).  KW wavefronts split each slice's K; their tiles meet in LDS and
// MP x MP threads finish one output each, always adding in the same order.
//
// Reference semantics of the fused parts: RMSNorm src/backend/cpu/kernels/elementwise.cpp:56-76,
// SwiGLU elementwise.cpp:101-119, short convolution src/backend/cpu/kernels/convolution.cpp:7-28,
// projections y = x W^T src/model/weight_plan.cpp:82-130; the reference fuses the residual
// addition into its products with beta = 1 (src/backend/cuda/model/prefill_batched/non_attention.cpp:175-201).
#include "common.h"
#include "gemv_params.h"

typedef short bf16x4_t __attribute__((ext_vector_type(4)));
typedef float floatx4_t __attribute__((ext_vector_type(4)));
struct __attribute__((aligned(16))) Frag2 {   // 16 bytes = 8 bfloat16 = two MFMA operands
    bf16x4_t lo, hi;
};

enum { E_STORE = 0, E_STORE_F32 = 1, E_RESIDUAL = 2, E_SWIGLU = 3, E_CONV = 4 };
#define SLICES_MAX_TAPS 8
#define SLICES_MAX_STAT_BLOCKS 512   // partial sums of squares a row may come with

__device__ __forceinline__ float round_bf16(float x) { return to_float(from_float<bf16>(x)); }

template <int EPI> struct Streams { static constexpr int n = 1; };
template <> struct Streams<E_SWIGLU> { static constexpr int n = 2; };
template <> struct Streams<E_CONV> { static constexpr int n = 3; };

// U: chunks of 64 along K that a wavefront keeps in flight at a time.
// Wavefronts 0 .. KW-1 multiply: nothing stands in front of their weight loads.  The
// wavefronts behind them (FW of them: MP*MP threads, one output each) first fetch what
// the end needs - the old value of the stream, or the convolution's state through the
// request's slot, and the partial sums of squares for the rows' 1/rms - while the
// products are under way, wait at the barrier, and finish.
// CT: tiles of MP columns a workgroup takes one after the other with the same rows of A in its
// registers (wide products, where MP columns a workgroup would be thousands of workgroups that the
// compute units cannot share out evenly: 4,608 columns of two streams at 8 rows are 576 workgroups of
// 8 columns, 2 on some compute units and 3 on others, but 256 of 18 in three tiles).
template <int G, int KW, int U, int CT, int EPI>
__global__ __launch_bounds__((KW + ((16 / G) * (16 / G) * CT + 63) / 64) * 64)
void gemv_slices_kernel(const void* const a_, const bf16* const w_, const int* const rows_, const int M, const int N, const int K,
                        const int cols, const int lda_, const int stream_rows_, const int w_row_stride_, const int w_kb_stride_,
                        const GemvParams p) {
    // (What the first loads need comes as arguments of its own, ahead of the struct that holds it too:
    // the first 14 words of a kernel's arguments arrive in registers with the launch, the rest is
    // fetched by the wavefronts.)
    constexpr int MP = 16 / G;
    constexpr int NS = Streams<EPI>::n;
    // rows a finishing wavefront holds the sums of squares of: its own share of the rows where one tile
    // fills several wavefronts (MP = 16), else all MP rows
    constexpr int ROWS_FW = MP * MP > 64 ? 64 / MP : MP;
    constexpr bool ROWS_BY_WAVE = MP * MP > 64;
    static_assert(CT == 1 || !ROWS_BY_WAVE, "several tiles of columns go with tiles of up to 64 outputs");
    __shared__ floatx4_t red[NS][CT][KW][64];
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
    const int n0 = blockIdx.x * cols;       // the workgroup owns `cols` <= CT * MP columns

    if (wave < KW) {
        // ---- the products
        const int c16 = lane & 15, q = lane >> 4;
        const int idx = c16 & (MP - 1), slice = c16 / MP;
        const int Ks = K / G;                   // K % (8 G) == 0 (checked by the host)
        const size_t a_row = static_cast<size_t>(rows_ ? rows_[min(idx, M - 1)] : min(idx, M - 1));
        const bf16* arow = static_cast<const bf16*>(a_) + a_row * lda_ + slice * Ks;
        const bf16* wrow[NS][CT];
#pragma unroll
        for (int s = 0; s < NS; ++s)
#pragma unroll
            for (int ct = 0; ct < CT; ++ct) {
                // (a lane whose column is not the workgroup's repeats its first column: no memory traffic of its own)
                const int j = ct * MP + idx;
                wrow[s][ct] = w_ + (static_cast<size_t>(s) * stream_rows_ + (j < cols && n0 + j < N ? n0 + j : n0)) * w_row_stride_;
            }
        const int k_slice = slice * Ks;
        const int chunks = (Ks + 63) >> 6;
        const int c_begin = wave * chunks / KW, c_end = (wave + 1) * chunks / KW;
        floatx4_t acc[NS][CT];
#pragma unroll
        for (int s = 0; s < NS; ++s)
#pragma unroll
            for (int ct = 0; ct < CT; ++ct) acc[s][ct] = floatx4_t{0.f, 0.f, 0.f, 0.f};
        for (int c0 = c_begin; c0 < c_end; c0 += U) {
            Frag2 wv[U][NS][CT][2], av[U][2];
#pragma unroll
            for (int u = 0; u < U; ++u)
#pragma unroll
                for (int v = 0; v < 2; ++v) {
                    const int k = (c0 + u) * 64 + v * 32 + q * 8;
                    const bool in = c0 + u < c_end && k + 8 <= Ks;
                    const int kw_ = k_slice + k;      // 8 values from here never leave a block of 32
                    const size_t w_off = static_cast<size_t>(kw_ >> 5) * w_kb_stride_ + (kw_ & 31);
                    av[u][v] = in ? *reinterpret_cast<const Frag2*>(arow + k) : Frag2{};
#pragma unroll
                    for (int s = 0; s < NS; ++s)
#pragma unroll
                        for (int ct = 0; ct < CT; ++ct)
                            wv[u][s][ct][v] = in ? *reinterpret_cast<const Frag2*>(wrow[s][ct] + w_off) : Frag2{};
                }
#pragma unroll
            for (int u = 0; u < U; ++u)
#pragma unroll
                for (int v = 0; v < 2; ++v)
#pragma unroll
                    for (int s = 0; s < NS; ++s)
#pragma unroll
                        for (int ct = 0; ct < CT; ++ct) {
                            acc[s][ct] = __builtin_amdgcn_mfma_f32_16x16x16bf16_1k(av[u][v].lo, wv[u][s][ct][v].lo, acc[s][ct], 0, 0, 0);
                            acc[s][ct] = __builtin_amdgcn_mfma_f32_16x16x16bf16_1k(av[u][v].hi, wv[u][s][ct][v].hi, acc[s][ct], 0, 0, 0);
                        }
        }
        // acc: lane l holds column l%16 of rows 4*(l/16)..+3 of the 16x16 tile
#pragma unroll
        for (int s = 0; s < NS; ++s)
#pragma unroll
            for (int ct = 0; ct < CT; ++ct) red[s][ct][wave][lane] = acc[s][ct];
        __syncthreads();
        return;
    }

    // ---- the finishing wavefronts: thread t finishes row em, column n0 + ej of tile tile_ct
    const int fw = wave - KW;
    const int t = fw * 64 + lane;
    const int tile_ct = CT == 1 ? 0 : min(t / (MP * MP), CT - 1);
    const int em = (t / MP) & (MP - 1), ej = (CT == 1 ? 0 : tile_ct * MP) + t % MP;
    const bool e_ok = t < MP * MP * CT && em < M && ej < cols && n0 + ej < N;
    const int en = min(n0 + ej, N - 1), emc = min(em, M - 1);
    float old = 0.f, taps[EPI == E_CONV ? SLICES_MAX_TAPS : 1], state[EPI == E_CONV ? SLICES_MAX_TAPS - 1 : 1];
    float bias[NS];
    float* state_ptr = nullptr;
    int slot = 0;
    if (EPI == E_CONV) slot = p.seq_slot[emc];
    // partial sums of squares of the ROWS_FW rows this wavefront holds: LPR lanes share a
    // row, every lane takes each LPR-th partial sum; all are asked for at once.  (Loads are
    // made without conditions, from clamped places, and masked afterwards: a load under a
    // condition of its own is waited for before the next one is asked for.)
    constexpr int LPR = 64 / ROWS_FW;
    constexpr int NFIRST = 16;
    float ssq = 0.f;
    if (p.stats) {
        const int nb = p.n_stat_blocks;
        const int sm = min((ROWS_BY_WAVE ? fw * ROWS_FW : 0) + lane / LPR, M - 1), sj = lane % LPR;
        const float* srow = p.stats + static_cast<size_t>(rows_ ? rows_[sm] : sm) * p.stats_ld;
        float part[NFIRST];
#pragma unroll
        for (int i = 0; i < NFIRST; ++i) part[i] = srow[min(sj + LPR * i, nb - 1)];
        for (int i0 = NFIRST; i0 * LPR < nb; i0 += 8) {   // the same for every lane; rare
            float rest[8];
#pragma unroll
            for (int i = 0; i < 8; ++i) rest[i] = srow[min(sj + LPR * (i0 + i), nb - 1)];
#pragma unroll
            for (int i = 0; i < 8; ++i) ssq += sj + LPR * (i0 + i) < nb ? rest[i] : 0.f;
        }
#pragma unroll
        for (int i = 0; i < NFIRST; ++i) ssq += sj + LPR * i < nb ? part[i] : 0.f;
    }
    if (EPI == E_RESIDUAL)
        old = static_cast<const float*>(p.out)[static_cast<size_t>(emc) * p.ldo + en];
#pragma unroll
    for (int s = 0; s < NS; ++s) bias[s] = p.bias ? p.bias[static_cast<size_t>(s) * stream_rows_ + en] : 0.f;
    if (EPI == E_CONV) {
#pragma unroll
        for (int i = 0; i < SLICES_MAX_TAPS; ++i) taps[i] = p.conv_w[static_cast<size_t>(en) * p.taps + min(i, p.taps - 1)];
        state_ptr = p.state + static_cast<size_t>(slot) * p.state_slot_stride + en;
#pragma unroll
        for (int i = 0; i < SLICES_MAX_TAPS - 1; ++i) state[i] = state_ptr[static_cast<size_t>(min(i + 1, p.taps - 1)) * N];
    }
    float scale = 1.f;
    if (p.stats) {
#pragma unroll
        for (int off = LPR / 2; off > 0; off >>= 1) ssq += __shfl_xor(ssq, off, 64);
        // the lanes of row em - fw * ROWS_FW hold its sum
        const float total = __shfl(ssq, ((em - (ROWS_BY_WAVE ? fw * ROWS_FW : 0)) & (ROWS_FW - 1)) * LPR, 64);
        scale = 1.0f / sqrtf(total / static_cast<float>(K) + p.eps);
    }
    __syncthreads();
    float sum[NS];
#pragma unroll
    for (int s = 0; s < NS; ++s) {
        sum[s] = 0.f;
#pragma unroll
        for (int g = 0; g < G; ++g) {
            const int r = g * MP + em, c = g * MP + t % MP;
            const int src = c + 16 * (r >> 2), reg = r & 3;
#pragma unroll
            for (int w = 0; w < KW; ++w) sum[s] += red[s][tile_ct][w][src][reg];
        }
        sum[s] = sum[s] * scale + bias[s];
    }
    const size_t o = static_cast<size_t>(emc) * p.ldo + en;
    if (EPI == E_STORE) {
        if (e_ok) static_cast<bf16*>(p.out)[o] = from_float<bf16>(sum[0]);
    } else if (EPI == E_STORE_F32) {
        if (e_ok) static_cast<float*>(p.out)[o] = sum[0];
        if (p.row_best) {
            // an output head: the best (logit, index) of the tile's columns, row by row (they sit in MP
            // neighbouring lanes): one part of the row
            const unsigned long long b = group_best_logit<MP>(sum[0], e_ok, n0 + tile_ct * MP);
            if (t % MP == 0 && em < M && t < MP * MP * CT)
                p.row_best[static_cast<size_t>(em) * p.row_best_ld + blockIdx.x * CT + tile_ct] = b;
        }
    } else if (EPI == E_RESIDUAL) {
        // the product enters the sum rounded to bfloat16, as where it is a tensor of its own
        const float v = e_ok ? old + round_bf16(sum[0]) : 0.f;
        if (e_ok) {
            static_cast<float*>(p.out)[o] = v;
            if (p.out_bf16) static_cast<bf16*>(p.out_bf16)[static_cast<size_t>(em) * p.ld_bf16 + en] = from_float<bf16>(v);
        }
        if (p.stats_out) {
            float sq = v * v;                   // the MP columns of a row and tile sit in MP neighbouring lanes
#pragma unroll
            for (int off = MP / 2; off > 0; off >>= 1) sq += __shfl_xor(sq, off, 64);
            // (one partial sum a tile: CT of them a workgroup)
            if (t % MP == 0 && em < M && t < MP * MP * CT)
                p.stats_out[static_cast<size_t>(em) * p.stats_ld_out + blockIdx.x * CT + tile_ct] = sq;
        }
    } else if (EPI == E_SWIGLU) {
        if (e_ok) {
            const float g = round_bf16(sum[0]), u = round_bf16(sum[1]);
            static_cast<bf16*>(p.out)[o] = from_float<bf16>((g / (1.0f + expf(-g))) * u);
        }
    } else if (EPI == E_CONV) {
        if (e_ok) {
            const float bb = round_bf16(sum[0]), cc = round_bf16(sum[1]), xx = round_bf16(sum[2]);
            const float bx = bb * xx;
            float conv = 0.f, last_tap = 0.f;
#pragma unroll
            for (int tap = 0; tap < SLICES_MAX_TAPS - 1; ++tap)
                if (tap + 1 < p.taps) {
                    conv = fmaf(taps[tap], state[tap], conv);
                    state_ptr[static_cast<size_t>(tap) * N] = state[tap];     // shift by one position
                }
#pragma unroll
            for (int tap = 0; tap < SLICES_MAX_TAPS; ++tap)
                if (tap == p.taps - 1) last_tap = taps[tap];
            conv = fmaf(last_tap, bx, conv);
            state_ptr[static_cast<size_t>(p.taps - 1) * N] = bx;
            if (p.conv_b) conv += p.conv_b[en];
            static_cast<bf16*>(p.out)[o] = from_float<bf16>(cc * conv);
        }
    }
}

template <int G, int KW, int CT, int EPI>
static int launch_slices(const GemvParams& params, int chunks_per_wave, int cols, hipStream_t stream) {
    constexpr int MP = 16 / G;
    GemvParams p = params;
    p.cols = cols;
    dim3 grid((p.N + cols - 1) / cols), block((KW + (MP * MP * CT + 63) / 64) * 64);
    constexpr int NS = Streams<EPI>::n;
    if (CT > 1 || chunks_per_wave <= 2 || (NS == 3 && KW == 8 && G == 1))   // (or the weights in flight fill the registers)
        hipLaunchKernelGGL((gemv_slices_kernel<G, KW, 2, CT, EPI>), grid, block, 0, stream, p.a, p.w, p.rows, p.M, p.N, p.K, cols, p.lda, p.stream_rows,
                           static_cast<int>(p.w_row_stride), static_cast<int>(p.w_kb_stride), p);
    else if (chunks_per_wave <= 4 || NS > 1)
        hipLaunchKernelGGL((gemv_slices_kernel<G, KW, 4, 1, EPI>), grid, block, 0, stream, p.a, p.w, p.rows, p.M, p.N, p.K, cols, p.lda, p.stream_rows,
                           static_cast<int>(p.w_row_stride), static_cast<int>(p.w_kb_stride), p);
    else if (NS == 1 && chunks_per_wave > 6 && chunks_per_wave <= 8)
        // (a long K, 7,168 or 8,192 values over two halves and eight wavefronts: all of a wavefront's
        // chunks in one trip to memory instead of six and then one or two)
        hipLaunchKernelGGL((gemv_slices_kernel<G, KW, (NS > 1 ? 4 : 8), 1, EPI>), grid, block, 0, stream, p.a, p.w, p.rows, p.M, p.N, p.K, cols, p.lda, p.stream_rows,
                           static_cast<int>(p.w_row_stride), static_cast<int>(p.w_kb_stride), p);
    else
        hipLaunchKernelGGL((gemv_slices_kernel<G, KW, (NS > 1 ? 4 : 6), 1, EPI>), grid, block, 0, stream, p.a, p.w, p.rows, p.M, p.N, p.K, cols, p.lda, p.stream_rows,
                           static_cast<int>(p.w_row_stride), static_cast<int>(p.w_kb_stride), p);
    return CELEG_LAUNCH_RESULT();
}

// The shape of the work: how many k-slices share the matrix instruction's tile (g: 4 for up to 4
// rows, 2 for up to 8, else 1; a tile then holds 16 / g columns), how many columns a workgroup owns and
// in how many tiles.  What these products wait for is what a compute unit pulls through its vector
// cache (its share of the weights and, every workgroup anew, the rows of A), so a product lasts as long
// as the compute unit with the most workgroups.  Few columns: a workgroup owns fewer than its tile holds
// (the lanes of the others load nothing), so that every compute unit has one.  The widest product (w1
// with w3) at 5 to 8 rows: the columns are shared out so that the workgroups are as many as the compute
// units, each with up to three tiles that share the rows of A in its registers (4,608 columns: 6.5 us
// instead of 6.9).  Measured and left: several tiles for the other epilogues and for 4 k-slices (the
// same or slower).
struct SlicesShape {
    int g, cols, ct;
};
static int g_force_slices = 0;     // tuning aids: 1, 2 or 4 k-slices; the columns a workgroup owns (where they fit)
static int g_force_cols = 0;
extern "C" void celeg_gemv_slices_force(int g) { g_force_slices = g; }
extern "C" void celeg_gemv_slices_force_cols(int cols) { g_force_cols = cols; }
#define SLICES_COMPUTE_UNITS 256
#define SLICES_MAX_TILES 3

static SlicesShape slices_shape(int M, int N, int K, int epi) {
    SlicesShape s;
    s.g = M <= 4 ? 4 : (M <= 8 ? 2 : 1);
    if (g_force_slices > 0 && g_force_slices <= s.g) s.g = g_force_slices;
    while (s.g > 1 && K % (8 * s.g)) s.g >>= 1;
    // more than about a thousand workgroups gain nothing (measured on 4,608 columns)
    while (s.g > 1 && g_force_slices == 0 && N / (16 / s.g) > 1024) s.g >>= 1;
    const int mp = 16 / s.g;
    const int max_tiles = s.g == 2 && epi == E_SWIGLU ? SLICES_MAX_TILES : 1;
    s.cols = mp, s.ct = 1;
    if ((N + mp - 1) / mp < SLICES_COMPUTE_UNITS) {
        while (s.cols > 4 && (N + s.cols - 1) / s.cols < SLICES_COMPUTE_UNITS) s.cols >>= 1;
    } else if (max_tiles > 1 && M > 4) {
        for (int k = 1; k <= 16; ++k) {
            const int cols = (N + SLICES_COMPUTE_UNITS * k - 1) / (SLICES_COMPUTE_UNITS * k);
            if (cols > mp * max_tiles) continue;
            if (cols > mp) s.cols = cols;
            break;
        }
    }
    if (g_force_cols > 0 && g_force_cols <= mp * max_tiles) s.cols = g_force_cols;
    s.ct = (s.cols + mp - 1) / mp;
    return s;
}

template <int G, int KW, int EPI>
static int launch_tiles(const GemvParams& p, int cpw, const SlicesShape& s, hipStream_t stream) {
    if constexpr (G == 2 && EPI == E_SWIGLU) {
        if (s.ct == 2) return launch_slices<G, KW, 2, EPI>(p, cpw, s.cols, stream);
        if (s.ct == 3) return launch_slices<G, KW, 3, EPI>(p, cpw, s.cols, stream);
    }
    if (s.ct != 1) return static_cast<int>(hipErrorInvalidValue);
    return launch_slices<G, KW, 1, EPI>(p, cpw, s.cols, stream);
}

template <int EPI>
static int launch_epilogue(const GemvParams& p, hipStream_t stream) {
    const SlicesShape s = slices_shape(p.M, p.N, p.K, EPI);
    const int chunks = (p.K / s.g + 63) / 64;
    const int kw = chunks >= 24 ? 8 : 4;
    const int cpw = (chunks + kw - 1) / kw;
    if (s.g == 4) return kw == 8 ? launch_tiles<4, 8, EPI>(p, cpw, s, stream) : launch_tiles<4, 4, EPI>(p, cpw, s, stream);
    if (s.g == 2) return kw == 8 ? launch_tiles<2, 8, EPI>(p, cpw, s, stream) : launch_tiles<2, 4, EPI>(p, cpw, s, stream);
    return kw == 8 ? launch_tiles<1, 8, EPI>(p, cpw, s, stream) : launch_tiles<1, 4, EPI>(p, cpw, s, stream);
}

extern "C" int celeg_gemv_params_size() { return static_cast<int>(sizeof(GemvParams)); }

// Number of workgroups for these sizes, which is also the number of partial sums of
// squares a row gets from the "residual" epilogue: the caller sizes stats_out [>= M, >= blocks].
extern "C" int celeg_gemv_slices_cols(int M, int N, int K) { return slices_shape(M, N, K, E_RESIDUAL).cols; }
extern "C" int celeg_gemv_slices_blocks(int M, int N, int K) {
    const SlicesShape s = slices_shape(M, N, K, E_RESIDUAL);
    return (N + s.cols - 1) / s.cols * s.ct;
}

// M <= 16, K % 8 == 0, bfloat16 a and w (w in either layout that w_row_stride and
// w_kb_stride describe).  Fields of GemvParams that are read: a, lda, rows,
// stats/n_stat_blocks/stats_ld/eps (scale by 1/rms if stats is set), w, stream_rows, bias,
// M, N, K, out, ldo, and per epilogue out_bf16/ld_bf16/stats_out/stats_ld_out (residual) or
// conv_w/conv_b/state/state_slot_stride/seq_slot/taps (conv).
extern "C" int celeg_gemv_slices(const GemvParams* params, int epi, hipStream_t stream) {
    const GemvParams& p = *params;
    if (p.M <= 0 || p.N <= 0) return 0;
    if (p.M > 16 || p.K <= 0 || (p.K % 8) || (p.lda % 8)) return static_cast<int>(hipErrorInvalidValue);
    if ((p.w_row_stride % 8) || (p.w_kb_stride % 8) || p.w_row_stride <= 0 || p.w_kb_stride <= 0 ||
        p.w_row_stride > 0x7fffffffLL || p.w_kb_stride > 0x7fffffffLL)
        return static_cast<int>(hipErrorInvalidValue);
    if (p.stats && (p.n_stat_blocks < 1 || p.n_stat_blocks > SLICES_MAX_STAT_BLOCKS))
        return static_cast<int>(hipErrorInvalidValue);
    if (epi == E_CONV && (p.taps < 1 || p.taps > SLICES_MAX_TAPS || p.stream_rows != p.N))
        return static_cast<int>(hipErrorInvalidValue);
    if (p.row_best && (epi != E_STORE_F32 || p.row_best_rows < p.M || p.row_best_ld < celeg_gemv_slices_blocks(p.M, p.N, p.K)))
        return static_cast<int>(hipErrorInvalidValue);
    switch (epi) {
        case E_STORE: return launch_epilogue<E_STORE>(p, stream);
        case E_STORE_F32: return launch_epilogue<E_STORE_F32>(p, stream);
        case E_RESIDUAL: return launch_epilogue<E_RESIDUAL>(p, stream);
        case E_SWIGLU: return launch_epilogue<E_SWIGLU>(p, stream);
        case E_CONV: return launch_epilogue<E_CONV>(p, stream);
        default: return static_cast<int>(hipErrorInvalidValue);
    }
}

// Prepares a 32-bit stream for products behind a norm: its bfloat16 copy and every row's
// sum of squares (one partial sum a row: stats[row * stats_ld]).  Used where the stream was written by
// something that leaves neither.
// (xb: element (row, i) at row * ldx + (i / 8) * xb_k8 + i % 8; rows one after the other: xb_k8 = 8)
__global__ void stream_prepare_kernel(const float* __restrict__ h, int ldh, bf16* __restrict__ xb,
                                      int ldx, long long xb_k8, float* __restrict__ stats, int stats_ld,
                                      int width) {
    __shared__ float scratch[16];
    const int row = blockIdx.x;
    const float* src = h + static_cast<size_t>(row) * ldh;
    float s = 0.f;
    for (int i = threadIdx.x; i < width; i += blockDim.x) {
        const float v = src[i];
        xb[static_cast<size_t>(row) * ldx + static_cast<size_t>(i >> 3) * xb_k8 + (i & 7)] = from_float<bf16>(v);
        s += v * v;
    }
    s = block_sum(s, scratch);
    if (threadIdx.x == 0) stats[static_cast<size_t>(row) * stats_ld] = s;
}

extern "C" int celeg_stream_prepare(const float* h, int ldh, void* xb, int ldx, long long xb_k8,
                                    float* stats, int stats_ld, int rows, int width, hipStream_t stream) {
    if (rows <= 0) return 0;
    hipLaunchKernelGGL(stream_prepare_kernel, dim3(rows), dim3(256), 0, stream, h, ldh,
                       static_cast<bf16*>(xb), ldx, xb_k8, stats, stats_ld, width);
    return CELEG_LAUNCH_RESULT();
}

// Embedding gather into the 32-bit stream, its bfloat16 copy and the rows' sums of squares:
// out[row, :] = table[ids[row], :], stats[row * stats_ld] = sum(out[row, :]^2).
__global__ void embed_stream_kernel(const bf16* __restrict__ table, const int* __restrict__ ids,
                                    float* __restrict__ out, bf16* __restrict__ xb, int ldx,
                                    long long xb_k8, float* __restrict__ stats, int stats_ld,
                                    int width, int vocab) {
    __shared__ float scratch[16];
    const int row = blockIdx.x;
    const int id = ids[row];
    const bool ok = id >= 0 && id < vocab;
    const bf16* src = table + static_cast<size_t>(ok ? id : 0) * width;
    float s = 0.f;
    for (int i = threadIdx.x; i < width; i += blockDim.x) {
        const bf16 raw = ok ? src[i] : bf16{0};
        const float v = to_float(raw);
        out[static_cast<size_t>(row) * width + i] = v;
        xb[static_cast<size_t>(row) * ldx + static_cast<size_t>(i >> 3) * xb_k8 + (i & 7)] = raw;
        s += v * v;
    }
    s = block_sum(s, scratch);
    if (threadIdx.x == 0) stats[static_cast<size_t>(row) * stats_ld] = s;
}

// The same with what a step begins with taken along (one kernel fewer in a step that is bound by
// its number of kernels): a row whose token id is negative takes the token its request sampled
// last and leaves it in ids, and the blocks behind the rows' write the step's block-table
// updates (count, then (slot, logical page, page) triples).
__global__ void embed_stream_prologue_kernel(const bf16* __restrict__ table, int* __restrict__ ids,
                                             float* __restrict__ out, bf16* __restrict__ xb, int ldx,
                                             long long xb_k8, float* __restrict__ stats, int stats_ld,
                                             int width, int vocab, int rows,
                                             int* __restrict__ block_table, int stride, int n_slots,
                                             const int* __restrict__ updates, int capacity,
                                             const int* __restrict__ token_slot,
                                             const int* __restrict__ last_tokens) {
    __shared__ float scratch[16];
    if (static_cast<int>(blockIdx.x) >= rows) {
        const int i = (static_cast<int>(blockIdx.x) - rows) * blockDim.x + threadIdx.x;
        if (i < min(updates[0], capacity)) {
            const int slot = updates[1 + 3 * i], logical = updates[2 + 3 * i], page = updates[3 + 3 * i];
            if (slot >= 0 && slot < n_slots && logical >= 0 && logical < stride)
                block_table[static_cast<size_t>(slot) * stride + logical] = page;
        }
        return;
    }
    const int row = blockIdx.x;
    int id = ids[row];
    if (id < 0 && last_tokens) {
        // (a thread that reads ids[row] after thread 0 has written it finds the same token there)
        id = last_tokens[token_slot[row]];
        if (threadIdx.x == 0) ids[row] = id;
    }
    const bool ok = id >= 0 && id < vocab;
    const bf16* src = table + static_cast<size_t>(ok ? id : 0) * width;
    float s = 0.f;
    for (int i = threadIdx.x; i < width; i += blockDim.x) {
        const bf16 raw = ok ? src[i] : bf16{0};
        const float v = to_float(raw);
        out[static_cast<size_t>(row) * width + i] = v;
        xb[static_cast<size_t>(row) * ldx + static_cast<size_t>(i >> 3) * xb_k8 + (i & 7)] = raw;
        s += v * v;
    }
    s = block_sum(s, scratch);
    if (threadIdx.x == 0) stats[static_cast<size_t>(row) * stats_ld] = s;
}

extern "C" int celeg_embed_stream_prologue(const void* table, int* ids, float* out, void* xb, int ldx,
                                           long long xb_k8, float* stats, int stats_ld, int rows, int width,
                                           int vocab, int* block_table, int stride, int n_slots,
                                           const int* updates, int capacity, const int* token_slot,
                                           const int* last_tokens, hipStream_t stream) {
    if (rows <= 0 || capacity <= 0 || !updates || !block_table) return static_cast<int>(hipErrorInvalidValue);
    hipLaunchKernelGGL(embed_stream_prologue_kernel, dim3(rows + (capacity + 255) / 256), dim3(256), 0, stream,
                       static_cast<const bf16*>(table), ids, out, static_cast<bf16*>(xb), ldx, xb_k8,
                       stats, stats_ld, width, vocab, rows, block_table, stride, n_slots, updates, capacity,
                       token_slot, last_tokens);
    return CELEG_LAUNCH_RESULT();
}

extern "C" int celeg_embed_stream(const void* table, const int* ids, float* out, void* xb, int ldx,
                                  long long xb_k8, float* stats, int stats_ld, int rows, int width,
                                  int vocab, hipStream_t stream) {
    if (rows <= 0) return 0;
    hipLaunchKernelGGL(embed_stream_kernel, dim3(rows), dim3(256), 0, stream,
                       static_cast<const bf16*>(table), ids, out, static_cast<bf16*>(xb), ldx, xb_k8,
                       stats, stats_ld, width, vocab);
    return CELEG_LAUNCH_RESULT();
}
