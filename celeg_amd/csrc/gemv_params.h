// Arguments of the fused skinny products (one struct for every prologue and epilogue, so
// that the caller fills one block of memory whatever the combination).
#pragma once
#include "common.h"

struct GemvParams {
    // A side
    const void* a;          // bf16 [M, lda] or float [*, lda]
    int lda;
    const int* rows;        // optional: A row of output row m is rows[m]
    const float* norm_w;    // A_NORM: [K]
    float eps;
    const float* stats;     // partial sums of squares of the rows of the stream: [rows, stats_ld], n_stat_blocks valid per row; or null
    int n_stat_blocks, stats_ld;
    // weights: stream s starts at row s * stream_rows
    const bf16* w;
    int stream_rows;
    const float* bias;      // optional [streams * stream_rows]
    int M, N, K;
    // outputs
    void* out;              // bf16 or float [M, ldo]; E_RESIDUAL: the residual stream itself
    int ldo;
    float* stats_out;       // E_RESIDUAL: [rows, stats_ld_out], one partial sum per workgroup and row; or null
    int stats_ld_out;
    // E_CONV
    const float* conv_w;    // [N, taps]
    const float* conv_b;    // optional [N]
    float* state;           // [slots, taps, N]
    size_t state_slot_stride;
    const int* seq_slot;    // [M]
    int taps;
    // E_RESIDUAL of the k-sliced kernels: the bfloat16 copy of the stream, or null
    void* out_bf16;
    int ld_bf16;
    // weight layout of the k-sliced kernels: element (n, k) of w lies at
    //   n * w_row_stride + (k / 32) * w_kb_stride + k % 32
    // (rows one after the other: K and 32; blocks of 32 k-values with the rows side by side
    // inside a block: 32 and rows * 32)
    long long w_row_stride, w_kb_stride;
    // layouts that only the kernel for 9 to 64 rows reads: element (m, k) of a lies at
    //   m * lda + (k / 8) * a_k8_stride + k % 8
    // (rows one after the other: 8; groups of 8 k-values with the rows side by side: rows * 8),
    // bfloat16 outputs out and out_bf16 likewise with ldo / out_k8_stride and ld_bf16 /
    // bf16_k8_stride, and element (n, k) of w at
    //   n * w_row_stride + (k / 32) * w_kb_stride + (k % 32 / 8) * w_q_stride + k % 8
    long long a_k8_stride, out_k8_stride, bf16_k8_stride, w_q_stride;
    // 32-bit store of an output head (the kernels for staged rows and for 9 to 64 rows): beside the
    // logits, the best (logit, index) of every workgroup's (or wavefront's) columns, packed as
    // packed_logit packs them: [parts, row_best_ld >= rows], part j from the j-th share of columns
    // (the rows of a part side by side: a workgroup's values are one run of memory); or null
    unsigned long long* row_best;
    int row_best_ld, row_best_parts;     // (room for row_best_parts parts: a launch that would leave more is refused)
};
