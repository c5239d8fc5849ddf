// Skinny bfloat16 products that end a sub-block, for up to 16 rows on gfx950:
//   h[M,N] += A[M,K] W[N,K]^T (+ bias),  h the 32-bit residual stream,
// leaving partial sums of squares of the new rows for the norm that follows.
//
// Such a product has few output columns (the model's width) and a long K, so a layout
// with 16 columns a workgroup leaves most of the chip idle.  Here the 16x16 tile of the
// MFMA is cut in G x G blocks of MP x MP (MP = 16 / G >= M): the instruction's row index
// is (k-slice g, row m) and its column index (k-slice g', column j); A rows of slice g
// hold A[m, g*K/G + k] and B columns of slice g' hold W[n0 + j, g'*K/G + k], so the
// diagonal blocks g == g' are G partial products over G parts of K for the same MP x MP
// outputs, and the others are dropped.  A workgroup then owns only MP columns (G times as
// many workgroups), every lane's loads are useful for M == MP, and the rows of A are read
// straight from cache into the instruction's operand layout (no staging).  KW wavefronts
// split each slice's K; their tiles meet in LDS and MP x MP threads finish one output each,
// always adding in the same order.
//
// Reference semantics: projections y = x W^T src/model/weight_plan.cpp:82-130; the residual
// addition fused into the product as with beta = 1 in
// src/backend/cuda/model/prefill_batched/non_attention.cpp:175-201.
#include "common.h"
#include "gemv_params.h"

typedef short bf16x4_t __attribute__((ext_vector_type(4)));
typedef float floatx4_t __attribute__((ext_vector_type(4)));
struct __attribute__((aligned(16))) Frag2 {   // 16 bytes = 8 bfloat16 = two MFMA operands
    bf16x4_t lo, hi;
};

// U: chunks of 64 along K that a wavefront keeps in flight at a time.
template <int G, int KW, int U>
__global__ __launch_bounds__(KW * 64) void gemv_slices_residual_kernel(const GemvParams p) {
    constexpr int MP = 16 / G;
    __shared__ floatx4_t red[KW][64];
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
    const int c16 = lane & 15, q = lane >> 4;
    const int idx = c16 & (MP - 1), slice = c16 / MP;
    const int M = p.M, N = p.N, K = p.K;
    const int Ks = K / G;                       // K % (8 G) == 0 (checked by the host)
    const int n0 = blockIdx.x * MP;
    const int t = threadIdx.x;                  // threads 0 .. MP*MP-1 finish one output each
    const int em = t / MP, ej = t % MP;
    const bool e_ok = t < MP * MP && em < M && n0 + ej < N;
    float* hp = static_cast<float*>(p.out) + static_cast<size_t>(min(em, M - 1)) * p.ldo + min(n0 + ej, N - 1);
    // what the end needs is asked for first
    const float old = e_ok ? *hp : 0.f;
    const float bias = (e_ok && p.bias) ? p.bias[n0 + ej] : 0.f;

    const bf16* wrow = p.w + static_cast<size_t>(min(n0 + idx, N - 1)) * K + slice * Ks;
    const bf16* arow = static_cast<const bf16*>(p.a) + static_cast<size_t>(min(idx, M - 1)) * p.lda + slice * Ks;
    const int chunks = (Ks + 63) >> 6;
    const int c_begin = wave * chunks / KW, c_end = (wave + 1) * chunks / KW;
    floatx4_t acc = {0.f, 0.f, 0.f, 0.f};
    for (int c0 = c_begin; c0 < c_end; c0 += U) {
        Frag2 wv[U][2], av[U][2];
#pragma unroll
        for (int u = 0; u < U; ++u)
#pragma unroll
            for (int v = 0; v < 2; ++v) {
                const int k = (c0 + u) * 64 + v * 32 + q * 8;
                const bool in = c0 + u < c_end && k + 8 <= Ks;
                wv[u][v] = in ? *reinterpret_cast<const Frag2*>(wrow + k) : Frag2{};
                av[u][v] = in ? *reinterpret_cast<const Frag2*>(arow + k) : Frag2{};
            }
#pragma unroll
        for (int u = 0; u < U; ++u)
#pragma unroll
            for (int v = 0; v < 2; ++v) {
                acc = __builtin_amdgcn_mfma_f32_16x16x16bf16_1k(av[u][v].lo, wv[u][v].lo, acc, 0, 0, 0);
                acc = __builtin_amdgcn_mfma_f32_16x16x16bf16_1k(av[u][v].hi, wv[u][v].hi, acc, 0, 0, 0);
            }
    }
    // acc: lane l holds column l%16 of rows 4*(l/16)..+3 of the 16x16 tile
    red[wave][lane] = acc;
    __syncthreads();
    if (wave * 64 >= MP * MP) return;           // whole wavefronts leave; the rest finish
    float sum = 0.f;
#pragma unroll
    for (int g = 0; g < G; ++g) {
        const int r = g * MP + (em & (MP - 1)), c = g * MP + ej;
        const int src = c + 16 * (r >> 2), reg = r & 3;
#pragma unroll
        for (int w = 0; w < KW; ++w) sum += red[w][src][reg];
    }
    // the product enters the sum rounded to bfloat16, as where it is a tensor of its own
    const float v = e_ok ? old + to_float(from_float<bf16>(sum + bias)) : 0.f;
    if (e_ok) *hp = v;
    if (p.stats_out) {
        float sq = v * v;                       // the MP columns of a row sit in MP neighbouring lanes
#pragma unroll
        for (int off = MP / 2; off > 0; off >>= 1) sq += __shfl_xor(sq, off, 64);
        if (ej == 0 && em < M && t < MP * MP)
            p.stats_out[static_cast<size_t>(blockIdx.x) * p.stats_ld_out + em] = sq;
    }
}

template <int G, int KW>
static int launch_slices(const GemvParams& p, int chunks_per_wave, hipStream_t stream) {
    dim3 grid((p.N + 16 / G - 1) / (16 / G)), block(KW * 64);
    if (chunks_per_wave <= 2) hipLaunchKernelGGL((gemv_slices_residual_kernel<G, KW, 2>), grid, block, 0, stream, p);
    else if (chunks_per_wave <= 4) hipLaunchKernelGGL((gemv_slices_residual_kernel<G, KW, 4>), grid, block, 0, stream, p);
    else hipLaunchKernelGGL((gemv_slices_residual_kernel<G, KW, 6>), grid, block, 0, stream, p);
    return CELEG_LAUNCH_RESULT();
}

// How many k-slices share the matrix instruction's tile for this many rows and this K.
static int slices_for(int M, int K) {
    int g = M <= 4 ? 4 : (M <= 8 ? 2 : 1);
    while (g > 1 && K % (8 * g)) g >>= 1;
    return g;
}

// Number of partial sums of squares a row gets (= workgroups): the caller sizes stats_out
// [blocks, >= M] with it.
extern "C" int celeg_gemv_slices_blocks(int M, int N, int K) {
    const int mp = 16 / slices_for(M, K);
    return (N + mp - 1) / mp;
}

// h[M,N] += a[M,K] w[N,K]^T + bias with partial sums of squares; M <= 16, K % 8 == 0.
// Uses of GemvParams: a, lda, w, bias, M, N, K, out, ldo, stats_out, stats_ld_out.
extern "C" int celeg_gemv_slices_residual(const GemvParams* params, hipStream_t stream) {
    const GemvParams& p = *params;
    if (p.M <= 0 || p.N <= 0) return 0;
    if (p.M > 16 || p.K <= 0 || (p.K % 8) || (p.lda % 8) || p.rows) return static_cast<int>(hipErrorInvalidValue);
    const int g = slices_for(p.M, p.K);
    const int chunks = (p.K / g + 63) / 64;
    const int kw = chunks >= 24 ? 8 : 4;
    const int cpw = (chunks + kw - 1) / kw;
    if (g == 4) return kw == 8 ? launch_slices<4, 8>(p, cpw, stream) : launch_slices<4, 4>(p, cpw, stream);
    if (g == 2) return kw == 8 ? launch_slices<2, 8>(p, cpw, stream) : launch_slices<2, 4>(p, cpw, stream);
    return kw == 8 ? launch_slices<1, 8>(p, cpw, stream) : launch_slices<1, 4>(p, cpw, stream);
}
