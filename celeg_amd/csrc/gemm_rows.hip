// bfloat16 products for 9 to 64 rows on gfx950 (decode steps of many requests, short
// portions of prompts), with what surrounds them fused in, as for the products of fewer
// rows:
//   out[M,N] = epilogue(scale[m] * (A[M,K] W[N,K]^T) + bias)
// A is bfloat16; behind an RMSNorm it is the bfloat16 copy of the residual stream, W has
// the norm's weight folded in and scale[m] = rsqrt(mean(x_m^2) + eps) comes from the
// partial sums of squares that the producer of the stream left.
// Epilogues: store | 32-bit store | add into the 32-bit residual stream, refresh its
// bfloat16 copy and leave partial sums of squares | SwiGLU of a gate and an up stream |
// the double-gated short convolution of a B, a C and an x stream for one new token per
// request, with its state update.
//
// Layout.  At these sizes the weights are read once from memory and the rows of A come
// from cache.  A workgroup owns CT tiles of 16 columns (of every weight stream), for MT tiles
// of 16 rows (all rows, or a part of them where the columns alone give fewer workgroups
// than the chip has compute units: the weights are then read once per part, from L2), over the
// WHOLE of K, which its wavefronts split between them; a wavefront keeps
// MT x (streams x CT) tiles of 16x16 sums, reads 16 bytes of weights per lane and tile for
// 32 values of k and the rows of A straight into the instruction's operand layout (whole
// runs of memory where A lies with its rows side by side inside every group of 8 values:
// rows that lie one after the other cost a cache line per lane), and holds the loads of
// the next 32 values in flight while it multiplies.  The wavefronts' tiles meet in LDS;
// every thread then finishes outputs of one row, always adding in the same order, so a
// result does not depend on what else is in the batch.  No workgroup needs another one's
// sums.  The columns a workgroup owns need not fill its tiles: where whole tiles would give a
// number of workgroups that the compute units do not share out evenly (4,608 columns are 288
// tiles of 16 for 256 compute units: 32 of them get twice the work, and the product lasts as
// long as they do), a workgroup owns fewer columns than its tiles hold (18 of 32) and the lanes
// of the others repeat an address that is loaded anyway.  What these products wait for is what a
// compute unit pulls through its vector cache, rows of A and weights alike (about 45 GB/s a compute
// unit when the weights come from memory), so they last as long as the compute unit with the most
// workgroups.  (Cutting K across workgroups, with a second kernel that adds the slices, was
// measured and gained nothing: narrow tiles and many wavefronts a workgroup were as fast
// or faster at every size tried, 1024 to 14336 columns and 1024 to 7168 values of k.)
//
// Reference semantics of the fused parts: RMSNorm src/backend/cpu/kernels/elementwise.cpp:56-76,
// SwiGLU elementwise.cpp:101-119, short convolution src/backend/cpu/kernels/convolution.cpp:7-28,
// projections y = x W^T src/model/weight_plan.cpp:82-130; the reference fuses the residual
// addition into its products with beta = 1 (src/backend/cuda/model/prefill_batched/non_attention.cpp:175-201).
#include <algorithm>

#include "common.h"
#include "gemv_params.h"

typedef __bf16 bf16x8_t __attribute__((ext_vector_type(8)));
typedef float floatx4_t __attribute__((ext_vector_type(4)));

enum { E_STORE = 0, E_STORE_F32 = 1, E_RESIDUAL = 2, E_SWIGLU = 3, E_CONV = 4 };
#define ROWS_MAX_TAPS 8
#define ROWS_MAX_STAT_BLOCKS 512
#define ROWS_MAX_LDS (128 * 1024)
#define ROWS_COMPUTE_UNITS 256

__device__ __forceinline__ float round_bf16(float x) { return to_float(from_float<bf16>(x)); }

template <int EPI> struct Streams { static constexpr int n = 1; };
template <> struct Streams<E_SWIGLU> { static constexpr int n = 2; };
template <> struct Streams<E_CONV> { static constexpr int n = 3; };

// Most wavefronts of a workgroup: what LDS holds of their tiles (a power of two, up to 16).
constexpr int rows_max_waves(int mt, int sc) {
    int w = 16;
    while (w > 1 && w * mt * sc * 1024 + 256 > ROWS_MAX_LDS) w >>= 1;
    return w;
}

// What the end of an output (row r, column n, both inside the sizes) needs from memory:
// asked for before the products, so that it has long arrived when they are done.
template <int EPI>
struct Early {
    float bias[Streams<EPI>::n];
    float old;                                           // E_RESIDUAL: the stream's value
    float taps[EPI == E_CONV ? ROWS_MAX_TAPS : 1];       // E_CONV
    float state[EPI == E_CONV ? ROWS_MAX_TAPS - 1 : 1];
    float conv_b;
    float* state_ptr;
};

template <int EPI>
__device__ __forceinline__ Early<EPI> early_fetch(const GemvParams& p, int r, int n) {
    Early<EPI> e;
#pragma unroll
    for (int s = 0; s < Streams<EPI>::n; ++s)
        e.bias[s] = p.bias ? p.bias[static_cast<size_t>(s) * p.stream_rows + n] : 0.f;
    e.old = 0.f; e.conv_b = 0.f; e.state_ptr = nullptr;
    if (EPI == E_RESIDUAL) e.old = static_cast<const float*>(p.out)[static_cast<size_t>(r) * p.ldo + n];
    if (EPI == E_CONV) {
        e.state_ptr = p.state + static_cast<size_t>(p.seq_slot[r]) * p.state_slot_stride + n;
#pragma unroll
        for (int i = 0; i < ROWS_MAX_TAPS; ++i) e.taps[i] = p.conv_w[static_cast<size_t>(n) * p.taps + min(i, p.taps - 1)];
#pragma unroll
        for (int i = 0; i < ROWS_MAX_TAPS - 1; ++i) e.state[i] = e.state_ptr[static_cast<size_t>(min(i + 1, p.taps - 1)) * p.N];
        if (p.conv_b) e.conv_b = p.conv_b[n];
    }
    return e;
}

// Finishes one output from the scaled sums of its weight streams.  Returns the new value of
// the residual stream (E_RESIDUAL) or the value stored (E_STORE_F32).
template <int EPI>
__device__ __forceinline__ float finish_output(const GemvParams& p, int r, int n, const float* scaled,
                                               const Early<EPI>& early) {
    float sum[Streams<EPI>::n];
#pragma unroll
    for (int s = 0; s < Streams<EPI>::n; ++s) sum[s] = scaled[s] + early.bias[s];
    const size_t o = static_cast<size_t>(r) * p.ldo + n;      // 32-bit outputs: rows one after the other
    const size_t ob = static_cast<size_t>(r) * p.ldo + static_cast<size_t>(n >> 3) * p.out_k8_stride + (n & 7);
    if (EPI == E_STORE) {
        static_cast<bf16*>(p.out)[ob] = from_float<bf16>(sum[0]);
    } else if (EPI == E_STORE_F32) {
        static_cast<float*>(p.out)[o] = sum[0];
        return sum[0];
    } else if (EPI == E_RESIDUAL) {
        // the product enters the sum rounded to bfloat16, as where it is a tensor of its own
        const float v = early.old + round_bf16(sum[0]);
        static_cast<float*>(p.out)[o] = v;
        if (p.out_bf16)
            static_cast<bf16*>(p.out_bf16)[static_cast<size_t>(r) * p.ld_bf16 + static_cast<size_t>(n >> 3) * p.bf16_k8_stride + (n & 7)] = from_float<bf16>(v);
        return v;
    } else if (EPI == E_SWIGLU) {
        const float g = round_bf16(sum[0]), u = round_bf16(sum[1]);
        static_cast<bf16*>(p.out)[ob] = from_float<bf16>((g / (1.0f + expf(-g))) * u);
    } else if (EPI == E_CONV) {
        const float bb = round_bf16(sum[0]), cc = round_bf16(sum[1]), xx = round_bf16(sum[2]);
        const float bx = bb * xx;
        float conv = 0.f, last_tap = 0.f;
#pragma unroll
        for (int tap = 0; tap < ROWS_MAX_TAPS - 1; ++tap)
            if (tap + 1 < p.taps) {
                conv = fmaf(early.taps[tap], early.state[tap], conv);
                early.state_ptr[static_cast<size_t>(tap) * p.N] = early.state[tap];     // shift by one position
            }
#pragma unroll
        for (int tap = 0; tap < ROWS_MAX_TAPS; ++tap)
            if (tap == p.taps - 1) last_tap = early.taps[tap];
        conv = fmaf(last_tap, bx, conv);
        early.state_ptr[static_cast<size_t>(p.taps - 1) * p.N] = bx;
        static_cast<bf16*>(p.out)[ob] = from_float<bf16>(cc * (conv + early.conv_b));
    }
    return 0.f;
}

// MT: tiles of 16 rows; CT: tiles of 16 columns per weight stream; blockDim.x / 64
// wavefronts split K.  LDS: [waves][MT][streams * CT][4][64] floats, then MT*16 scales.
template <int MT, int CT, int EPI>
__global__ __launch_bounds__(64 * rows_max_waves(MT, Streams<EPI>::n * CT))
void gemm_rows_kernel(const void* const a_, const bf16* const w_, const int* const rows_, const int N, const int K, const int M,
                      const int shape_, const int stream_rows_, const int w_row_stride_, const int w_kb_stride_,
                      const int a_strides_, const GemvParams p) {
    // (What the first loads need comes as arguments of its own, ahead of the struct that holds it too:
    // the first 14 words of a kernel's arguments arrive in registers with the launch, the rest is
    // fetched by the wavefronts.  shape_: the columns the workgroup owns, its wavefronts << 8,
    // w_q_stride << 16; a_strides_: lda, a_k8_stride << 20.)
    const int cols = shape_ & 0xff;
    const int w_q_stride_ = shape_ >> 16, lda_ = a_strides_ & 0xfffff, a_k8_stride_ = a_strides_ >> 20;
    constexpr int NS = Streams<EPI>::n;
    constexpr int SC = NS * CT;
    constexpr int COLS = CT * 16;          // columns the tiles hold; the workgroup owns the first `cols` of them
    constexpr int ROWS = MT * 16;
    extern __shared__ float smem[];
    const int n_waves = (shape_ >> 8) & 0xff;
    float* const red = smem;
    float* const s_scale = smem + static_cast<size_t>(n_waves) * MT * SC * 256;
    // (E_STORE_F32 with row_best: the best logit of every 16 columns of a row, [ROWS][CT])
    unsigned long long* const s_best = reinterpret_cast<unsigned long long*>(s_scale + ROWS);
    // the wavefront's number as a scalar: the branches on its range of k are then uniform
    // ones (the matrix instructions do not honour a lane mask)
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6), lane = threadIdx.x & 63;
    const int n0 = blockIdx.x * cols;
    const int row0 = blockIdx.y * ROWS;        // the workgroup's first row
    const int c16 = lane & 15, q = lane >> 4;

    // ---- operands: A rows t*16 + c16, W columns n0 + ct*16 + c16 of every stream
    const bf16* arow[MT];
#pragma unroll
    for (int t = 0; t < MT; ++t) {
        const int m = min(row0 + t * 16 + c16, M - 1);
        arow[t] = static_cast<const bf16*>(a_) + static_cast<size_t>(rows_ ? rows_[m] : m) * lda_ + q * a_k8_stride_;
    }
    const bf16* wcol[SC];
#pragma unroll
    for (int s = 0; s < NS; ++s)
#pragma unroll
        for (int ct = 0; ct < CT; ++ct) {
            // a lane whose column is not the workgroup's repeats the first column's address (no memory traffic of its own)
            const int jn = ct * 16 + c16;
            const int n = jn < cols && n0 + jn < N ? n0 + jn : n0;
            wcol[s * CT + ct] = w_ + (static_cast<size_t>(s) * stream_rows_ + n) * w_row_stride_ + q * w_q_stride_;
        }
    const int nkb = K >> 5;                    // K % 32 == 0 (checked by the host)
    const int kb_begin = wave * nkb / n_waves, kb_end = (wave + 1) * nkb / n_waves;

    floatx4_t acc[MT][SC];
#pragma unroll
    for (int t = 0; t < MT; ++t)
#pragma unroll
        for (int s = 0; s < SC; ++s) acc[t][s] = floatx4_t{0.f, 0.f, 0.f, 0.f};

    // D blocks of 32 values of k in flight (four where the registers hold them were no faster)
    constexpr int D = 2;
    bf16x8_t av_[D][MT], wv_[D][SC];
    auto fetch = [&](int kb, bf16x8_t (&av)[MT], bf16x8_t (&wv)[SC]) {
#pragma unroll
        for (int s = 0; s < SC; ++s)
            wv[s] = *reinterpret_cast<const bf16x8_t*>(wcol[s] + static_cast<size_t>(kb) * w_kb_stride_);
#pragma unroll
        for (int t = 0; t < MT; ++t)
            av[t] = *reinterpret_cast<const bf16x8_t*>(arow[t] + static_cast<size_t>(kb) * 4 * a_k8_stride_);
    };
    auto multiply = [&](const bf16x8_t (&av)[MT], const bf16x8_t (&wv)[SC]) {
#pragma unroll
        for (int t = 0; t < MT; ++t)
#pragma unroll
            for (int s = 0; s < SC; ++s)
                acc[t][s] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(av[t], wv[s], acc[t][s], 0, 0, 0);
    };
#pragma unroll
    for (int d = 0; d < D; ++d)
        if (kb_begin + d < kb_end) fetch(kb_begin + d, av_[d], wv_[d]);

    // ---- what the end of this thread's first output needs (asked for behind the first weights)
    const int e0 = min(static_cast<int>(threadIdx.x), ROWS * COLS - 1);
    const Early<EPI> early0 = early_fetch<EPI>(p, min(row0 + e0 / COLS, M - 1), min(n0 + e0 % COLS, N - 1));

    // ---- the rows' 1/rms from the partial sums of squares (likewise): LPR neighbouring
    // threads share a row
    if (p.stats) {
        const int lpr = n_waves * 64 / ROWS;         // a power of two, 1 .. 32
        const int r = threadIdx.x / lpr, sub = threadIdx.x % lpr;
        const int nb = p.n_stat_blocks;
        const int m = min(row0 + r, M - 1);
        const float* srow = p.stats + static_cast<size_t>(rows_ ? rows_[m] : m) * p.stats_ld;
        float ssq = 0.f;
        for (int b0 = 0; b0 < nb; b0 += 8 * lpr) {   // the same trips for every thread
            float part[8];
#pragma unroll
            for (int i = 0; i < 8; ++i) part[i] = srow[min(b0 + sub + lpr * i, nb - 1)];
#pragma unroll
            for (int i = 0; i < 8; ++i) ssq += b0 + sub + lpr * i < nb ? part[i] : 0.f;
        }
        for (int off = lpr >> 1; off > 0; off >>= 1) ssq += __shfl_xor(ssq, off, 64);
        if (sub == 0) s_scale[r] = 1.0f / sqrtf(ssq / static_cast<float>(K) + p.eps);
    }

    for (int kb = kb_begin; kb < kb_end; kb += D) {
#pragma unroll
        for (int d = 0; d < D; ++d) {
            if (kb + d < kb_end) multiply(av_[d], wv_[d]);
            if (kb + d + D < kb_end) fetch(kb + d + D, av_[d], wv_[d]);
        }
    }

    // acc[t][s]: lane l holds column l%16 of rows 4*(l/16)..+3 of the tile
#pragma unroll
    for (int t = 0; t < MT; ++t)
#pragma unroll
        for (int s = 0; s < SC; ++s)
#pragma unroll
            for (int i = 0; i < 4; ++i)
                red[(((static_cast<size_t>(wave) * MT + t) * SC + s) * 4 + i) * 64 + lane] = acc[t][s][i];
    __syncthreads();

    // ---- thread e takes row e / COLS, column e % COLS of the workgroup's tile
    const int n_threads = n_waves * 64;
    for (int e = threadIdx.x; e < ROWS * COLS; e += n_threads) {
        const int rl = e / COLS, j = e % COLS;      // row inside the workgroup's rows
        const int t = rl >> 4, rr = rl & 15, ct = j >> 4, jj = j & 15;
        const int src = jj + 16 * (rr >> 2), reg = rr & 3;
        const int r = row0 + rl, n = n0 + j;
        const bool ok = r < M && n < N && j < cols;
        const int rc = min(r, M - 1), nc = min(n, N - 1);
        float sum[NS];
#pragma unroll
        for (int s = 0; s < NS; ++s) {
            float v = 0.f;
            for (int w = 0; w < n_waves; ++w)
                v += red[(((static_cast<size_t>(w) * MT + t) * SC + s * CT + ct) * 4 + reg) * 64 + src];
            sum[s] = v;
        }
        const float scale = p.stats ? s_scale[rl] : 1.f;
#pragma unroll
        for (int s = 0; s < NS; ++s) sum[s] *= scale;
        float v = 0.f;
        if (e == static_cast<int>(threadIdx.x)) {
            if (ok) v = finish_output<EPI>(p, rc, nc, sum, early0);
        } else if (ok) {
            v = finish_output<EPI>(p, rc, nc, sum, early_fetch<EPI>(p, rc, nc));
        }
        if (EPI == E_RESIDUAL && p.stats_out) {
            float sq = v * v;               // the COLS columns of a row sit in COLS neighbouring lanes
#pragma unroll
            for (int off = COLS / 2; off > 0; off >>= 1) sq += __shfl_xor(sq, off, 64);
            if (j == 0 && r < M) p.stats_out[static_cast<size_t>(r) * p.stats_ld_out + blockIdx.x] = sq;
        }
        if (EPI == E_STORE_F32 && p.row_best) {
            // the best (logit, index) of the tile's 16 columns of this row (no trip through LDS, which
            // this loop's reads of the partial sums would wait behind); the tiles meet below
            const unsigned long long b = group_best_logit<16>(v, ok, n0 + (j & ~15));
            if (jj == 0) s_best[rl * CT + ct] = b;
        }
    }
    if (EPI == E_STORE_F32 && p.row_best) {
        // one part a row and workgroup: the best of its tiles
        __syncthreads();
        const int rl = threadIdx.x;
        if (rl < ROWS && row0 + rl < M) {
            unsigned long long b = 0ull;
#pragma unroll
            for (int ct = 0; ct < CT; ++ct) b = max(b, s_best[rl * CT + ct]);
            p.row_best[static_cast<size_t>(row0 + rl) * p.row_best_ld + blockIdx.x] = b;
        }
    }
}

// The shape of the work for these sizes: narrow tiles, so that there are many workgroups
// (wide ones only where even they give thousands, as for an output head), and as many
// wavefronts as LDS holds tiles of and as still have two blocks of 32 each.  Then the columns a
// workgroup owns: all its tiles hold, or fewer (a) where that leaves compute units without a
// workgroup (1,024 columns of a product of 16 rows are 64 tiles: 4 columns a workgroup give 256
// workgroups, 6.9 against 8.4 us for K = 4,608) and (b) where the last round of workgroups would
// be far from full (4,608 columns of two streams are 288 tiles, a round of 256 and one of 32 that
// takes as long: tiles twice as wide of which a workgroup owns 18 columns are two full rounds,
// 10.7 against 12.2 us at 64 rows, 9.0 against 9.4 at 32, 7.5 against 7.8 at 16).
struct RowsShape {
    int mt, ct, waves, cols;
};

// For tests and tuning: a share of columns (ct: 1, 2 or 4 tiles of 16, owned whole), a number of
// wavefronts and a share of rows (mt: 1, 2 or 4 tiles of 16) that override the choice below
// where they fit; 0 leaves a choice alone.  celeg_gemm_rows_force_cols: the columns a workgroup owns.
static int g_force_ct = 0, g_force_waves = 0, g_force_mt = 0, g_force_cols = 0;
extern "C" void celeg_gemm_rows_force(int ct, int waves, int mt) { g_force_ct = ct; g_force_waves = waves; g_force_mt = mt; }
extern "C" void celeg_gemm_rows_force_cols(int cols) { g_force_cols = cols; }

static RowsShape rows_shape(int M, int N, int K, int streams) {
    RowsShape s;
    const int max_mt = M <= 16 ? 1 : (M <= 32 ? 2 : 4);
    s.mt = max_mt;
    const int max_ct = streams == 1 ? 4 : (streams == 2 ? 2 : 1);
    s.ct = 1;
    while (s.ct < max_ct && (N + 32 * s.ct - 1) / (32 * s.ct) >= 1024) s.ct *= 2;
    if (g_force_ct > 0 && g_force_ct <= max_ct) s.ct = g_force_ct;
    // few columns: the rows are shared out too, until there is a workgroup per compute unit
    while (s.mt > 1 && ((N + 16 * s.ct - 1) / (16 * s.ct)) * ((M + 16 * s.mt - 1) / (16 * s.mt)) < ROWS_COMPUTE_UNITS)
        s.mt >>= 1;
    if ((g_force_mt == 1 || g_force_mt == 2 || g_force_mt == 4) && g_force_mt <= max_mt) s.mt = g_force_mt;
    s.cols = 16 * s.ct;
    const bool forced = g_force_ct > 0 || g_force_mt > 0 || g_force_cols > 0;
    if (!forced) {
        const auto row_groups = [&](int mt) { return (M + 16 * mt - 1) / (16 * mt); };
        // (a) compute units without a workgroup: half the columns a workgroup, and half again, while
        // that still leaves no compute unit with a second one (36 to 48 rows by 1,024 columns are 3
        // groups of rows and 192 workgroups of 16 columns: 8 columns would be 384, a round and a half,
        // w2 8.4 to 9.2 us against 7.2 to 7.7; shares that are no power of two, 13 columns for 237
        // workgroups, were slower too: 8.0 to 8.4)
        if (s.ct == 1)
            while (s.cols > 4 && row_groups(s.mt) * ((N + s.cols / 2 - 1) / (s.cols / 2)) <= ROWS_COMPUTE_UNITS) s.cols >>= 1;
        // (b) a last round of workgroups that is less than three quarters full
        const long long groups = static_cast<long long>(row_groups(s.mt)) * ((N + s.cols - 1) / s.cols);
        const long long rounds = (groups + ROWS_COMPUTE_UNITS - 1) / ROWS_COMPUTE_UNITS;
        if (s.cols == 16 * s.ct && groups > ROWS_COMPUTE_UNITS && rounds * ROWS_COMPUTE_UNITS - groups > ROWS_COMPUTE_UNITS / 4 &&
            2 * s.ct <= max_ct) {
            const int mt = std::min(s.mt, 2), wide = 32 * s.ct;
            for (int k = 1; k <= 8; ++k) {
                const long long want = static_cast<long long>(ROWS_COMPUTE_UNITS) * k;      // workgroups: whole rounds
                const int cols = static_cast<int>((static_cast<long long>(N) * row_groups(mt) + want - 1) / want);
                if (cols > wide) continue;
                if (cols > 16 * s.ct) s.mt = mt, s.ct *= 2, s.cols = cols;
                break;
            }
        }
    }
    if (g_force_cols >= 1 && g_force_cols <= 16 * max_ct) {
        s.cols = g_force_cols;
        s.ct = s.cols <= 16 ? 1 : (s.cols <= 32 ? 2 : 4);
    }
    const int nkb = K / 32;
    s.waves = rows_max_waves(s.mt, streams * s.ct);
    if (K <= 2048 && s.waves > 8) s.waves = 8;     // a short K: two workgroups of 8 a compute unit were the faster
    // tiles of 64 columns (an output head): 2 wavefronts, so that a compute unit holds four such
    // workgroups and their ends overlap (65,536 columns by 1,024: 36.6 against 42.3 us with 4 wavefronts at
    // 64 rows, 29.5 against 30.7 at 32, 26.8 against 31.0 at 16; by 2,048: 60.3 against 64.0 at 64 rows;
    // one wavefront and eight are slower)
    if (s.ct == 4 && s.waves > 2) s.waves = 2;
    while (s.waves > 1 && s.waves * 2 > nkb) s.waves >>= 1;
    if (g_force_waves > 0 && g_force_waves <= rows_max_waves(s.mt, streams * s.ct)) s.waves = g_force_waves;
    return s;
}

template <int MT, int CT, int EPI>
static int launch_rows(const GemvParams& params, int waves, int cols, hipStream_t stream) {
    constexpr int NS = Streams<EPI>::n;
    GemvParams p = params;
    p.cols = cols;
    const size_t lds = static_cast<size_t>(waves) * MT * NS * CT * 1024 + MT * 16 * sizeof(float) +
                       (p.row_best ? static_cast<size_t>(MT) * 16 * CT * sizeof(unsigned long long) : 0);
    static bool raised = false;              // once per instantiation: more LDS than the default limit
    if (lds > 48 * 1024 && !raised) {
        hipError_t err = hipFuncSetAttribute(reinterpret_cast<const void*>(&gemm_rows_kernel<MT, CT, EPI>),
                                             hipFuncAttributeMaxDynamicSharedMemorySize, ROWS_MAX_LDS);
        if (err != hipSuccess) return static_cast<int>(err);
        raised = true;
    }
    dim3 grid((p.N + cols - 1) / cols, (p.M + MT * 16 - 1) / (MT * 16)), block(waves * 64);
    hipLaunchKernelGGL((gemm_rows_kernel<MT, CT, EPI>), grid, block, lds, stream, p.a, p.w, p.rows, p.N, p.K, p.M,
                       cols | (waves << 8) | (static_cast<int>(p.w_q_stride) << 16), p.stream_rows,
                       static_cast<int>(p.w_row_stride), static_cast<int>(p.w_kb_stride),
                       p.lda | (static_cast<int>(p.a_k8_stride) << 20), p);
    return CELEG_LAUNCH_RESULT();
}

template <int EPI>
static int launch_epilogue(const GemvParams& p, hipStream_t stream) {
    constexpr int NS = Streams<EPI>::n;
    const RowsShape s = rows_shape(p.M, p.N, p.K, NS);
#define ROWS_CASE(MT_, CT_) \
    if (s.mt == MT_ && s.ct == CT_) return launch_rows<MT_, CT_, EPI>(p, s.waves, s.cols, stream);
    ROWS_CASE(1, 1) ROWS_CASE(2, 1) ROWS_CASE(4, 1)
    if constexpr (NS <= 2) { ROWS_CASE(1, 2) ROWS_CASE(2, 2) ROWS_CASE(4, 2) }
    if constexpr (NS == 1) { ROWS_CASE(1, 4) ROWS_CASE(2, 4) ROWS_CASE(4, 4) }
#undef ROWS_CASE
    return static_cast<int>(hipErrorInvalidValue);
}

static int streams_of(int epi) { return epi == E_SWIGLU ? 2 : (epi == E_CONV ? 3 : 1); }

// Number of workgroups for these sizes, which is also the number of partial sums of
// squares a row gets from the "residual" epilogue: the caller sizes stats_out [>= M, >= blocks].
extern "C" int celeg_gemm_rows_cols(int M, int N, int K, int epi) { return rows_shape(M, N, K, streams_of(epi)).cols; }
extern "C" int celeg_gemm_rows_blocks(int M, int N, int K, int epi) {
    const RowsShape s = rows_shape(M, N, K, streams_of(epi));
    return (N + s.cols - 1) / s.cols;
}
// All workgroups of the launch: those shares of columns times the groups of rows.
extern "C" int celeg_gemm_rows_workgroups(int M, int N, int K, int epi) {
    const RowsShape s = rows_shape(M, N, K, streams_of(epi));
    return ((N + s.cols - 1) / s.cols) * ((M + s.mt * 16 - 1) / (s.mt * 16));
}

// M <= 64 (made for 17 and more; fewer rows work too), K % 32 == 0, bfloat16 a and
// w (in the layouts that the strides describe).  The fields of GemvParams that are read are
// those of the products for up to 16 rows and the strides of the operands' groups of 8.
extern "C" int celeg_gemm_rows(const GemvParams* params, int epi, hipStream_t stream) {
    const GemvParams& p = *params;
    if (p.M <= 0 || p.N <= 0) return 0;
    if (p.M > 64 || p.K <= 0 || (p.K % 32) || (p.lda % 8)) return static_cast<int>(hipErrorInvalidValue);
    if ((p.w_row_stride % 8) || (p.w_kb_stride % 8) || (p.w_q_stride % 8) || p.w_row_stride <= 0 ||
        p.w_kb_stride <= 0 || p.w_q_stride <= 0 || p.w_row_stride > 0x7fffffffLL || p.w_kb_stride > 0x7fffffffLL ||
        p.w_q_stride > 0x7fffLL || p.a_k8_stride > 0x7ffLL || p.lda > 0xfffff)      // (they travel in packed words)
        return static_cast<int>(hipErrorInvalidValue);
    if ((p.a_k8_stride % 8) || p.a_k8_stride <= 0 || (p.out_k8_stride % 8) || p.out_k8_stride <= 0 ||
        (p.out_bf16 && ((p.bf16_k8_stride % 8) || p.bf16_k8_stride <= 0)))
        return static_cast<int>(hipErrorInvalidValue);
    if (p.stats && (p.n_stat_blocks < 1 || p.n_stat_blocks > ROWS_MAX_STAT_BLOCKS))
        return static_cast<int>(hipErrorInvalidValue);
    if (epi == E_CONV && (p.taps < 1 || p.taps > ROWS_MAX_TAPS || p.stream_rows != p.N))
        return static_cast<int>(hipErrorInvalidValue);
    if (p.row_best && (epi != E_STORE_F32 || p.row_best_rows < p.M || p.row_best_ld < celeg_gemm_rows_blocks(p.M, p.N, p.K, epi)))
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
