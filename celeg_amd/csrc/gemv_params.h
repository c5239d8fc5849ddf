// Arguments of the fused skinny products (one struct for every prologue and epilogue, so
// that the caller fills one block of memory whatever the combination).
//
// The order of the fields is by who reads them: a kernel's wavefronts fetch the arguments they use
// through the scalar cache, 64 bytes a line, before they can do anything else, and every line more
// showed in the time of the products of few rows (a struct of 240 bytes with the last argument
// behind it against the same with that argument in a fifth line: 0.15 to 0.25 us a launch).  The
// first two lines hold what every product of up to 64 bfloat16 rows reads; the third the short
// convolution's operands and the norm weight of the older form; the fourth the strides that only the
// kernel for 9 to 64 rows reads and what an output head leaves for greedy rows.
#pragma once
#include <cstddef>

#include "common.h"

struct GemvParams {
    // ---- bytes 0..63
    const void* a;          // bf16 [M, lda] or float [*, lda]
    // weights: stream s starts at row s * stream_rows
    const bf16* w;
    void* out;              // bf16 or float [M, ldo]; E_RESIDUAL: the residual stream itself
    const float* stats;     // partial sums of squares of the rows of the stream: [rows, stats_ld], n_stat_blocks valid per row; or null
    const int* rows;        // optional: A row of output row m is rows[m]
    const float* bias;      // optional [streams * stream_rows]
    void* out_bf16;         // E_RESIDUAL of the k-sliced kernels: the bfloat16 copy of the stream, or null
    float* stats_out;       // E_RESIDUAL: [rows, stats_ld_out], one partial sum per workgroup and row; or null
    // ---- bytes 64..127
    int M, N, K;
    int lda, ldo;
    int n_stat_blocks, stats_ld, stats_ld_out;
    int stream_rows;
    int ld_bf16;
    float eps;
    int cols;               // the columns a workgroup owns (set by the launching code of the kernels that read it)
    // weight layout of the k-sliced kernels: element (n, k) of w lies at
    //   n * w_row_stride + (k / 32) * w_kb_stride + k % 32
    // (rows one after the other: K and 32; blocks of 32 k-values with the rows side by side
    // inside a block: 32 and rows * 32)
    long long w_row_stride, w_kb_stride;
    // ---- bytes 128..191
    // E_CONV
    const float* conv_w;    // [N, taps]
    const float* conv_b;    // optional [N]
    float* state;           // [slots, taps, N]
    size_t state_slot_stride;
    const int* seq_slot;    // [M]
    int taps;
    int reserved_;
    const float* norm_w;    // A_NORM: [K]
    // 32-bit store of an output head: beside the logits, the best (logit, index) of every
    // workgroup's (or wavefront's) columns, packed as packed_logit packs them: [rows, row_best_ld >=
    // parts], part j from the j-th share of columns (the parts of a row one after the other: what
    // picks a row's token afterwards reads one run of memory); or null
    unsigned long long* row_best;
    // ---- bytes 192..
    // layouts that only the kernel for 9 to 64 rows reads: element (m, k) of a lies at
    //   m * lda + (k / 8) * a_k8_stride + k % 8
    // (rows one after the other: 8; groups of 8 k-values with the rows side by side: rows * 8),
    // bfloat16 outputs out and out_bf16 likewise with ldo / out_k8_stride and ld_bf16 /
    // bf16_k8_stride, and element (n, k) of w at
    //   n * w_row_stride + (k / 32) * w_kb_stride + (k % 32 / 8) * w_q_stride + k % 8
    long long a_k8_stride, out_k8_stride, bf16_k8_stride, w_q_stride;
    int row_best_ld, row_best_rows;     // (room for row_best_rows rows of row_best_ld parts: a launch that would leave more is refused)
};
static_assert(offsetof(GemvParams, M) == 64 && offsetof(GemvParams, conv_w) == 128 && offsetof(GemvParams, a_k8_stride) == 192,
              "the fields of GemvParams are grouped by 64-byte lines");
