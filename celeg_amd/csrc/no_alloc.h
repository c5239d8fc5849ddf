// An entry point that allocates nothing.
//
// It has no counterpart in the reference.  It is for callers that cannot allocate device
// memory: code under HIP graph capture, tight serving loops, harnesses that forbid hipMalloc.
//
// celeg_attention_decode_bf16 (attention_fast.hip) cuts every request's context into parts,
// lets one workgroup per part leave a partial (maximum, sum, output) in a workspace that the
// caller allocated, and joins the parts with a second kernel.  The entry point below runs the
// same two kernels with the workspace in a file-scope device array of CELEG_NO_ALLOC_SCRATCH_BYTES
// bytes that every GPU the library runs on holds until the process ends.  It calls no
// hipMalloc, hipFree or allocating library routine, and refuses (hipErrorInvalidValue, nothing
// launched) sizes whose partial results, n_rows * q_heads * n_parts * (head_dim + 2) floats,
// exceed the array.
//
// All calls on one GPU share that GPU's array, which keeps the last call's contents.  Nothing
// in it has to start at zero: every part that the joining kernel reads was written by the same
// call.  Calls that overlap on one GPU (two streams, two threads) race on it: the caller keeps
// them in order.
#pragma once
#include <hip/hip_runtime.h>

#define CELEG_NO_ALLOC_SCRATCH_BYTES (16u << 20)

extern "C" {
// Looks up the array's address on the current device (once per device; the first call of
// the entry point on a device does it too).  0 or a hipError_t value.
int celeg_attention_decode_no_alloc_init(void);

// out[row, head, :] = attention of the one new token of every request over its paged keys and
// values; the arguments are those of celeg_attention_decode_bf16 without the workspace, the
// context cut into n_parts parts of split_rounds (1, 4 or 16) rounds of 64 keys each, so
// that n_parts * split_rounds * 64 keys cover the longest context.  head_dim 64 or 128.
int celeg_attention_decode_bf16_no_alloc(
    const void* q, int ldq, const void* k_pool, const void* v_pool, const int* table,
    int table_stride, const int* token_slot, const int* positions, void* out, int ldo,
    int n_rows, int q_heads, int kv_heads, int head_dim, int page_tokens, int n_layers, int layer,
    float scale, int window, int split_rounds, int n_parts, hipStream_t stream);
}
