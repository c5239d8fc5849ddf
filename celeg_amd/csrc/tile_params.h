// Arguments of the tiled products of many rows (gemm_tiles.hip).
#pragma once
#include "common.h"

struct TileParams {
    const bf16* a;          // [M, lda]
    int lda;
    const bf16* w;          // [streams * stream_rows, ldw]; stream s starts at row s * stream_rows
    int ldw;
    int stream_rows;
    const float* bias;      // optional [streams * stream_rows]
    const float* stats;     // optional partial sums of squares [M, stats_ld], n_stat_blocks valid a row
    int n_stat_blocks, stats_ld;
    float eps;
    int M, N, K;            // N: output columns (per stream)
    void* out;              // bf16 [M, ldo] (store, SwiGLU) or the 32-bit stream [M, ldo] (residual)
    int ldo;
    bf16* out_bf16;         // residual: the stream's bfloat16 copy [M, ld_bf16], or null
    int ld_bf16;
    float* stats_out;       // residual: [M, stats_ld_out], one partial sum per tile column and row; or null
    int stats_ld_out;
};
