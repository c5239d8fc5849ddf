// True 32-bit matrix product for the 32-bit path: Y[M,N] = X[M,K] W[N,K]^T (+ bias).
// No reduced-precision matrix mode: plain fused multiply-adds in float, and every
// output element is accumulated over k = 0..K-1 in that order whatever M, the tile or
// the batch is, so the logits of a row do not depend on how rows were batched.
// The reference's projections: y = x W^T, weights [out, in] row-major
// (src/model/weight_plan.cpp:82-130).
#include "common.h"

#define BM 64
#define BN 64
#define BK 16

__global__ __launch_bounds__(256) void gemm_f32_kernel(
    const float* __restrict__ X, int ldx, const float* __restrict__ W, int ldw,
    const float* __restrict__ bias, float* __restrict__ Y, int ldy, int M, int N, int K) {
    __shared__ float Xs[BK][BM + 1];
    __shared__ float Ws[BK][BN + 1];
    const int tid = threadIdx.x;
    const int tx = tid % 16, ty = tid / 16;
    const int row0 = blockIdx.y * BM, col0 = blockIdx.x * BN;
    float acc[4][4];
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j) acc[i][j] = 0.f;

    for (int k0 = 0; k0 < K; k0 += BK) {
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const int e = tid + i * 256;
            const int r = e / BK, c = e % BK;
            const int gr = row0 + r, gc = col0 + r, gk = k0 + c;
            Xs[c][r] = (gr < M && gk < K) ? X[static_cast<size_t>(gr) * ldx + gk] : 0.f;
            Ws[c][r] = (gc < N && gk < K) ? W[static_cast<size_t>(gc) * ldw + gk] : 0.f;
        }
        __syncthreads();
#pragma unroll
        for (int kk = 0; kk < BK; ++kk) {
            float a[4], b[4];
#pragma unroll
            for (int i = 0; i < 4; ++i) a[i] = Xs[kk][ty * 4 + i];
#pragma unroll
            for (int j = 0; j < 4; ++j) b[j] = Ws[kk][tx * 4 + j];
#pragma unroll
            for (int i = 0; i < 4; ++i)
#pragma unroll
                for (int j = 0; j < 4; ++j) acc[i][j] = fmaf(a[i], b[j], acc[i][j]);
        }
        __syncthreads();
    }
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const int gr = row0 + ty * 4 + i;
        if (gr >= M) continue;
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const int gc = col0 + tx * 4 + j;
            if (gc >= N) continue;
            Y[static_cast<size_t>(gr) * ldy + gc] = acc[i][j] + (bias ? bias[gc] : 0.f);
        }
    }
}

extern "C" int celeg_gemm_f32(const float* X, int ldx, const float* W, int ldw, const float* bias,
                              float* Y, int ldy, int M, int N, int K, hipStream_t stream) {
    if (M <= 0 || N <= 0) return 0;
    if (K <= 0) return static_cast<int>(hipErrorInvalidValue);
    dim3 grid((N + BN - 1) / BN, (M + BM - 1) / BM), block(256);
    hipLaunchKernelGGL(gemm_f32_kernel, grid, block, 0, stream, X, ldx, W, ldw, bias, Y, ldy, M, N,
                       K);
    return CELEG_LAUNCH_RESULT();
}
