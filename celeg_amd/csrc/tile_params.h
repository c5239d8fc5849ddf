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
    // The q/k/v epilogue: the columns are heads of 64, q_heads query heads, then kv_heads key
    // heads, then kv_heads value heads.  Query heads are normalised (weight, eps; null: not),
    // turned by their row's position (cos_sin [positions, 32, 2]; null: not) and stored to out;
    // key heads likewise and stored to the cache pages of their rows; value heads are stored to
    // the pages, transposed.  The layout of the pools and of the block table is the attention's.
    const int* positions;   // [M]
    const int* token_slot;  // [M]
    const int* table;       // [slots, table_stride]
    int table_stride;
    bf16* k_pool;
    bf16* v_pool;
    int n_layers, layer, page_tokens, q_heads, kv_heads;
    const float* q_weight;  // [64]
    const float* k_weight;  // [64]
    float qk_eps;
    const float* cos_sin;
};
