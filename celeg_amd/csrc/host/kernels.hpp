// The entry points of the HIP kernels (the .hip files beside this folder), as the host calls
// them: raw device pointers, sizes and a stream in, 0 or a hipError_t value out.  Shapes are
// checked by the callers in ops.cpp; a kernel never sees a size it was not written for.
#pragma once
#include <hip/hip_runtime_api.h>

#include <cstddef>
#include <cstdint>

#include "../gemv_params.h"
#include "../tile_params.h"
#include "../no_alloc.h"

extern "C" {
// elementwise.hip
int celeg_embed(const void* table, int table_dtype, const int* ids, float* out, int rows, int width, int vocab,
                hipStream_t stream);
int celeg_rmsnorm(void* x, int x_dtype, const void* delta, int delta_dtype, const float* w, void* out, int out_dtype,
                  const int* rows, int n_rows, int width, float eps, int write_back, hipStream_t stream);
int celeg_swiglu(const void* gu, void* out, int dtype, int rows, int ff, hipStream_t stream);
int celeg_add_bias(void* x, int dtype, const float* bias, int rows, int width, hipStream_t stream);
int celeg_cast(const void* src, int src_dtype, void* dst, int dst_dtype, size_t total, hipStream_t stream);
int celeg_table_update(int* table, int stride, int n_slots, const int* updates, int capacity, hipStream_t stream);
int celeg_step_prologue(int* table, int stride, int n_slots, const int* updates, int capacity, int* token_ids,
                        const int* token_slot, const int* last_tokens, int n, hipStream_t stream);
int celeg_resolve_tokens(int* token_ids, const int* token_slot, const int* last_tokens, int n, hipStream_t stream);
int celeg_fold_weight(const void* w, const float* scale, void* out, int rows, int K, int packed, hipStream_t stream);
int celeg_zero_words(void* p, size_t words, hipStream_t stream);
// gemm_f32.hip
int celeg_gemm_f32(const float* X, int ldx, const float* W, int ldw, const float* bias, float* Y, int ldy, int M,
                   int N, int K, hipStream_t stream);
// short_conv.hip
int celeg_short_conv(const void* bcx, int ld_bcx, int dtype, const float* w, const float* bias, float* state,
                     size_t state_slot_stride, void* out, const int* positions, const int* token_seq,
                     const int* seq_start, const int* seq_slot, const int* cu_seqlens, int n_tokens, int n_seqs,
                     int width, int taps, hipStream_t stream);
// attention.hip
int celeg_rope_table(const float* inv_freq, int half, int n_positions, float* out, hipStream_t stream);
int celeg_qk_norm_rope_store(void* q, int ldq, const void* k, int ldk, const void* v, int ldv, int dtype,
                             const float* q_weight, const float* k_weight, float eps, const float* inv_freq,
                             const float* cos_sin, int rotary_dim, int pairing, const int* positions, const int* token_slot,
                             const int* table, int table_stride, void* k_pool, void* v_pool, int n_layers, int layer,
                             int page_tokens, int n_tokens, int q_heads, int kv_heads, int head_dim, int store_kv,
                             hipStream_t stream);
int celeg_paged_attention(const void* q, int ldq, const void* k_pool, const void* v_pool, int dtype, const int* table,
                          int table_stride, const int* token_slot, const int* positions, void* out, int ldo,
                          int n_tokens, int q_heads, int kv_heads, int head_dim, int page_tokens, int n_layers,
                          int layer, float scale, int window, hipStream_t stream);
// attention_fast.hip
int celeg_attention_rows_bf16(const void* q, int ldq, const void* k_pool, const void* v_pool, const int* table,
                              int table_stride, const int* cu_seqlens, const int* seq_slot, const int* seq_start,
                              int n_seqs, int n_tokens, void* out, int ldo, int q_heads, int kv_heads, int head_dim,
                              int page_tokens, int n_layers, int layer, float scale, int window, int rows_per_tile,
                              int form, int context_hint, hipStream_t stream);
int celeg_attention_decode_bf16(const void* q, int ldq, const void* k_pool, const void* v_pool, const int* table,
                                int table_stride, const int* token_slot, const int* positions, float* ws_o,
                                float* ws_ml, int n_splits, void* out, int ldo, int n_rows, int q_heads,
                                int kv_heads, int head_dim, int page_tokens, int n_layers, int layer, float scale,
                                int window, int whole, int split_rounds, int n_parts, hipStream_t stream);
int celeg_attention_decode_fresh_bf16(const void* q, int ldq, const void* k, int ldk, const void* v, int ldv,
                                      const float* q_weight, const float* k_weight, float eps, const float* cos_sin,
                                      void* k_pool, void* v_pool, const int* table, int table_stride, const int* token_slot,
                                      const int* positions, float* ws_o, float* ws_ml, int n_splits, void* out, int ldo,
                                      int n_rows, int q_heads, int kv_heads, int head_dim, int page_tokens, int n_layers,
                                      int layer, float scale, int window, int whole, int split_rounds, int n_parts,
                                      hipStream_t stream);
// sampling.hip
int celeg_argmax_rows(const float* logits, int ld, int rows, int vocab, const float* fparams, const int* iparams,
                      uint8_t* seen, size_t seen_stride, int* out_tokens, int* last_tokens,
                      unsigned long long* best, unsigned int* arrived, hipStream_t stream);
int celeg_argmax_merge(const unsigned long long* best, int ld, int parts, int rows, const int* iparams, int* out_tokens,
                       int* last_tokens, hipStream_t stream);
int celeg_sample(const float* logits, int ld, int rows, int vocab, const float* fparams, const int* iparams,
                 uint8_t* seen, size_t seen_stride, int* out_tokens, int* last_tokens, const unsigned long long* best,
                 int best_ld, int best_parts, int best_cols, hipStream_t stream);
int celeg_mark_seen(uint8_t* seen, size_t stride, int n_slots, int vocab, const int* tokens, const int* slots, int n,
                    hipStream_t stream);
// gemv_slices.hip, gemm_rows.hip, gemv_fused.hip: the fused products for up to 64 rows
int celeg_gemv_params_size();
int celeg_gemv_slices_blocks(int M, int N, int K);
int celeg_gemv_slices_cols(int M, int N, int K);
int celeg_gemv_slices(const GemvParams* params, int epi, hipStream_t stream);
int celeg_stream_prepare(const float* h, int ldh, void* xb, int ldx, long long xb_k8, float* stats, int stats_ld,
                         int rows, int width, hipStream_t stream);
int celeg_embed_stream(const void* table, const int* ids, float* out, void* xb, int ldx, long long xb_k8, float* stats,
                       int stats_ld, int rows, int width, int vocab, hipStream_t stream);
int celeg_embed_stream_prologue(const void* table, int* ids, float* out, void* xb, int ldx, long long xb_k8, float* stats,
                                int stats_ld, int rows, int width, int vocab, int* block_table, int stride, int n_slots,
                                const int* updates, int capacity, const int* token_slot, const int* last_tokens,
                                hipStream_t stream);
int celeg_gemm_rows_blocks(int M, int N, int K, int epi);
int celeg_gemm_rows_workgroups(int M, int N, int K, int epi);
int celeg_gemm_rows_cols(int M, int N, int K, int epi);
int celeg_gemm_rows(const GemvParams* params, int epi, hipStream_t stream);
int celeg_gemv_fused(const GemvParams* params, int amode, int epi, int shape, hipStream_t stream);
int celeg_embed_stats(const void* table, const int* ids, float* out, float* stats, int stats_ld, int rows, int width,
                      int vocab, hipStream_t stream);
// gemm_tiles.hip: the fused products of many rows
int celeg_gemm_tiles_blocks(int M, int N, int K);
int celeg_gemm_tiles_params_size();
int celeg_gemm_tiles(const TileParams* params, int epi, hipStream_t stream);
}
