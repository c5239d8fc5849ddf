// Plain C++ functions for what the kernels compute (reference.cpp): host memory, 32-bit floats,
// loops.  For tests; nothing on the product path calls them.
#pragma once
#include <cstddef>

namespace celeg {
namespace reference {

void embed(const float* table, int vocab, int width, const int* ids, int rows, float* out);
void rmsnorm(float* x, const float* delta, const float* weight, float eps, int rows, int width, float* out);
void linear(const float* x, const float* w, const float* bias, int M, int N, int K, float* out);
void swiglu(const float* gate_up, int rows, int ff, float* out);
void short_conv(const float* bcx, const float* w, const float* bias, float* state, const int* seq_slot, const int* seq_start,
                const int* cu_seqlens, int n_seqs, int width, int taps, float* out);
void qk_norm_rope(float* x, const float* weight, float eps, const float* inv_freq, int rotary_dim, int pairing,
                  const int* positions, int rows, int heads, int head_dim);
void kv_store(const float* k, const float* v, float* k_pool, float* v_pool, const int* table, int table_stride,
              const int* token_slot, const int* positions, int rows, int kv_heads, int head_dim, int page_tokens,
              int n_layers, int layer);
void paged_attention(const float* q, const float* k_pool, const float* v_pool, const int* table, int table_stride,
                     const int* token_slot, const int* positions, int rows, int heads, int kv_heads, int head_dim,
                     int page_tokens, int n_layers, int layer, float scale, int window, float* out);
int sample(const float* logits, int vocab, float temperature, int top_k, float top_p, float penalty, const unsigned char* seen,
           float u);

}  // namespace reference
}  // namespace celeg
