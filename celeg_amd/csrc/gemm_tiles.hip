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

enum { T_STORE = 0, T_RESIDUAL = 2, T_SWIGLU = 3 };   // the numbers of the few-rows products


#define GPTR(p) ((const __attribute__((address_space(1))) void*)(p))
#define LPTR(p) ((__attribute__((address_space(3))) void*)(p))

__device__ __forceinline__ float round_bf16(float x) { return to_float(from_float<bf16>(x)); }

template <int N>
__device__ __forceinline__ void wait_loads() {
    asm volatile("s_waitcnt vmcnt(%0)" ::"n"(N) : "memory");
}

template <int EPI> struct TileStreams { static constexpr int n = EPI == T_SWIGLU ? 2 : 1; };

template <int BM, int BN, int WGM, int WGN, int STAGES, int EPI>
__global__ __launch_bounds__(WGM * WGN * 64)
void gemm_tiles_kernel(const TileParams p, const int tiles_m, const int tiles_n, const int dies_m) {
    constexpr int NW = WGM * WGN;
    constexpr int NS = TileStreams<EPI>::n;
    constexpr int WTM = BM / WGM, WTN = BN / WGN;
    constexpr int FM = WTM / 16, FN = WTN / 16;
    constexpr int STAGE_BYTES = (BM + BN) * 128;
    constexpr int GROUPS = (BM + BN) / 8;          // loads of 1 KB a block of k
    constexpr int GPW = GROUPS / NW;               // of which a wavefront issues this many
    static_assert(GROUPS % NW == 0 && FN % NS == 0 && WTM % 16 == 0 && WTN % 16 == 0, "tile shape");
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
        const int g = wave + i * NW;
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
                                             LPTR(base + (wave + i * NW) * 1024), 16, 0, 0);
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

    const int nkb = K >> 6;                       // K % 64 == 0 (checked by the host)
#pragma unroll
    for (int s = 0; s < STAGES; ++s)
        if (s < nkb) issue(s, s);

    // ---- the rows' 1/rms, asked for behind the first blocks
    float scale[FM];
#pragma unroll
    for (int tm = 0; tm < FM; ++tm) scale[tm] = 1.f;
    if (p.stats) {
        // eight partial sums of every row in flight at once (a chain of single loads would
        // cost a trip to memory each)
        const float* srow[FM];
        float ssq[FM];
#pragma unroll
        for (int tm = 0; tm < FM; ++tm) {
            srow[tm] = p.stats + static_cast<size_t>(min(m0 + wm * WTM + tm * 16 + r16, M - 1)) * p.stats_ld;
            ssq[tm] = 0.f;
        }
        const int nb = p.n_stat_blocks;
        for (int b0 = 0; b0 < nb; b0 += 8) {
            float part[FM][8];
#pragma unroll
            for (int tm = 0; tm < FM; ++tm)
#pragma unroll
                for (int i = 0; i < 8; ++i) part[tm][i] = srow[tm][min(b0 + i, nb - 1)];
#pragma unroll
            for (int tm = 0; tm < FM; ++tm)
#pragma unroll
                for (int i = 0; i < 8; ++i) ssq[tm] += b0 + i < nb ? part[tm][i] : 0.f;
        }
#pragma unroll
        for (int tm = 0; tm < FM; ++tm) scale[tm] = 1.0f / sqrtf(ssq[tm] / static_cast<float>(K) + p.eps);
    }

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

    // ---- acc[tn][tm][i]: row m0 + wm*WTM + tm*16 + lane%16, column (of the stream) ... + 4*(lane/16) + i
    constexpr int FNS = FN / NS;                  // column pieces of 16 per stream
    // the residual stream's old values, all asked for at once
    floatx4_t old_[EPI == T_RESIDUAL ? FM : 1][EPI == T_RESIDUAL ? FNS : 1];
    if (EPI == T_RESIDUAL) {
#pragma unroll
        for (int tm = 0; tm < FM; ++tm)
#pragma unroll
            for (int j = 0; j < FNS; ++j) {
                const int m = min(m0 + wm * WTM + tm * 16 + r16, M - 1);
                const int n = min(n0 + wn * (WTN / NS) + j * 16 + 4 * q, N - 4);
                old_[EPI == T_RESIDUAL ? tm : 0][EPI == T_RESIDUAL ? j : 0] =
                    *reinterpret_cast<const floatx4_t*>(static_cast<const float*>(p.out) + static_cast<size_t>(m) * p.ldo + n);
            }
    }
    float sq[FM];
#pragma unroll
    for (int tm = 0; tm < FM; ++tm) sq[tm] = 0.f;
#pragma unroll
    for (int tm = 0; tm < FM; ++tm) {
        const int m = m0 + wm * WTM + tm * 16 + r16;
#pragma unroll
        for (int j = 0; j < FNS; ++j) {
            const int n = n0 + wn * (WTN / NS) + j * 16 + 4 * q;
            if (m >= M || n >= N) continue;       // N % 4 == 0: a lane's four columns are inside together
            float v[NS][4];
#pragma unroll
            for (int s = 0; s < NS; ++s)
#pragma unroll
                for (int i = 0; i < 4; ++i)
                    v[s][i] = acc[s * FNS + j][tm][i] * scale[tm] +
                              (p.bias ? p.bias[static_cast<size_t>(s) * p.stream_rows + n + i] : 0.f);
            if (EPI == T_RESIDUAL) {
                float* const h = static_cast<float*>(p.out) + static_cast<size_t>(m) * p.ldo + n;
                floatx4_t old = old_[EPI == T_RESIDUAL ? tm : 0][EPI == T_RESIDUAL ? j : 0];
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
                        o[i] = (g / (1.0f + expf(-g))) * u;
                    } else {
                        o[i] = v[0][i];
                    }
                }
                *reinterpret_cast<bf16x4_t*>(static_cast<bf16*>(p.out) + static_cast<size_t>(m) * p.ldo + n) =
                    bf16x4_t{static_cast<__bf16>(o[0]), static_cast<__bf16>(o[1]),
                             static_cast<__bf16>(o[2]), static_cast<__bf16>(o[3])};
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

// ---- the shape of the work for given sizes
struct TileShape {
    int id;         // index into the table below
    int bm, bn;     // bn counts weight rows of all streams
};

// For tests and tuning: a shape that overrides the choice below (-1: none).
static int g_force_shape = -1, g_force_dies_m = 0;
extern "C" void celeg_gemm_tiles_force(int shape) { g_force_shape = shape; }
extern "C" void celeg_gemm_tiles_force_dies(int dies_m) { g_force_dies_m = dies_m; }

#define TILE_SHAPES(X) \
    X(0, 128, 128, 2, 2, 3) \
    X(1, 256, 128, 2, 2, 3) \
    X(2, 128, 64, 2, 2, 3)  \
    X(3, 64, 128, 2, 2, 3)  \
    X(4, 128, 128, 2, 2, 2) \
    X(5, 256, 128, 4, 2, 3) \
    X(6, 128, 128, 2, 2, 4) \
    X(7, 64, 64, 2, 2, 4)   \
    X(8, 64, 64, 2, 2, 2)   \
    X(9, 128, 64, 2, 2, 2)  \
    X(10, 128, 128, 4, 2, 2)

static const int k_shape_bm[] = {128, 256, 128, 64, 128, 256, 128, 64, 64, 128, 128};
static const int k_shape_bn[] = {128, 128, 64, 128, 128, 128, 128, 64, 64, 64, 128};
#define N_TILE_SHAPES 11

static TileShape tile_shape(int M, int N, int streams) {
    int id = 0;
    if (g_force_shape >= 0 && g_force_shape < N_TILE_SHAPES) id = g_force_shape;
    else {
        // Measured at 2,048 rows (1,024 to 9,216 weight rows, 1,024 and 4,608 values of k):
        // tiles of 128x128 with two workgroups of 8 wavefronts a compute unit where they give
        // every unit one and a half or more (8 wavefronts: a tenth faster than 4), else
        // smaller tiles, which fill the chip.
        const long long wide = static_cast<long long>((M + 127) / 128) * ((static_cast<long long>(N) * streams + 127) / 128);
        id = wide >= 384 ? 10 : (wide >= 192 ? 3 : 7);
    }
    return TileShape{id, k_shape_bm[id], k_shape_bn[id]};
}

template <int BM, int BN, int WGM, int WGN, int STAGES, int EPI>
static int launch_tiles(const TileParams& p, hipStream_t stream) {
    constexpr int NS = TileStreams<EPI>::n;
    constexpr size_t lds = static_cast<size_t>(STAGES) * (BM + BN) * 128;
    static_assert(lds <= 160 * 1024, "more LDS than a compute unit has");
    static bool raised = false;              // once per instantiation: more LDS than the default limit
    if (lds > 48 * 1024 && !raised) {
        hipError_t err = hipFuncSetAttribute(reinterpret_cast<const void*>(&gemm_tiles_kernel<BM, BN, WGM, WGN, STAGES, EPI>),
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
    hipLaunchKernelGGL((gemm_tiles_kernel<BM, BN, WGM, WGN, STAGES, EPI>), grid, block, lds, stream, p, tiles_m, tiles_n, dies_m);
    return CELEG_LAUNCH_RESULT();
}

template <int EPI>
static int launch_epilogue(const TileParams& p, hipStream_t stream) {
    const TileShape s = tile_shape(p.M, p.N, TileStreams<EPI>::n);
#define TILE_CASE(ID, BM, BN, WGM, WGN, STAGES) \
    if (s.id == ID) return launch_tiles<BM, BN, WGM, WGN, STAGES, EPI>(p, stream);
    TILE_SHAPES(TILE_CASE)
#undef TILE_CASE
    return static_cast<int>(hipErrorInvalidValue);
}

// Number of partial sums of squares a row gets from the "residual" epilogue for these
// sizes (one per tile column): the caller sizes stats_out [>= M, >= blocks].
extern "C" int celeg_gemm_tiles_blocks(int M, int N, int K) {
    (void)K;
    const TileShape s = tile_shape(M, N, 1);
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
    if (p.out_bf16 && ((p.ld_bf16 % 4) || p.ld_bf16 < p.N)) return static_cast<int>(hipErrorInvalidValue);
    if (epi == T_SWIGLU && p.stream_rows < p.N) return static_cast<int>(hipErrorInvalidValue);
    switch (epi) {
        case T_STORE: return launch_epilogue<T_STORE>(p, stream);
        case T_RESIDUAL: return launch_epilogue<T_RESIDUAL>(p, stream);
        case T_SWIGLU: return launch_epilogue<T_SWIGLU>(p, stream);
        default: return static_cast<int>(hipErrorInvalidValue);
    }
}
