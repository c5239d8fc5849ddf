// Plain C++ functions for what the kernels compute, one beside each kernel, on host memory:
// loops in 32-bit floats, no tiles, no vectors, the same arguments and the same layouts of the
// cache pages and the state slots as the kernels take.  The reference keeps such functions
// beside its CUDA kernels (src/model/reference.cpp:24-262: rmsnorm_bf16, rope_bf16_inplace,
// gqa_decode_strict_bf16, conv_decode_bf16); tests hold the kernels and the plain Python
// implementation against these.  Nothing on the product path calls them.
#include "reference.hpp"

#include <algorithm>
#include <cmath>
#include <stdexcept>
#include <vector>

namespace celeg {
namespace reference {

// out[r] = table[ids[r]]  (src/backend/cpu/model_forward_token.cpp:28-60)
void embed(const float* table, int vocab, int width, const int* ids, int rows, float* out) {
    for (int r = 0; r < rows; ++r) {
        if (ids[r] < 0 || ids[r] >= vocab) throw std::invalid_argument("embed: token id out of range");
        for (int i = 0; i < width; ++i) out[static_cast<size_t>(r) * width + i] = table[static_cast<size_t>(ids[r]) * width + i];
    }
}

// x += delta (if given; written back to x), then out = x / sqrt(mean(x^2) + eps) * weight
// (src/backend/cpu/kernels/elementwise.cpp:56-76).  The sum of squares runs in double here.
void rmsnorm(float* x, const float* delta, const float* weight, float eps, int rows, int width, float* out) {
    for (int r = 0; r < rows; ++r) {
        float* xr = x + static_cast<size_t>(r) * width;
        double sum = 0.0;
        for (int i = 0; i < width; ++i) {
            if (delta) xr[i] += delta[static_cast<size_t>(r) * width + i];
            sum += static_cast<double>(xr[i]) * xr[i];
        }
        const float inv = static_cast<float>(1.0 / std::sqrt(sum / width + eps));
        for (int i = 0; i < width; ++i) out[static_cast<size_t>(r) * width + i] = xr[i] * inv * weight[i];
    }
}

// out[M, N] = x[M, K] w[N, K]^T (+ bias)  (src/model/weight_plan.cpp:82-130)
void linear(const float* x, const float* w, const float* bias, int M, int N, int K, float* out) {
    for (int m = 0; m < M; ++m)
        for (int n = 0; n < N; ++n) {
            double sum = 0.0;
            for (int k = 0; k < K; ++k) sum += static_cast<double>(x[static_cast<size_t>(m) * K + k]) * w[static_cast<size_t>(n) * K + k];
            out[static_cast<size_t>(m) * N + n] = static_cast<float>(sum + (bias ? bias[n] : 0.f));
        }
}

// out = silu(gate) * up, gate_up = [gate | up]  (src/backend/cpu/kernels/elementwise.cpp:101-119)
void swiglu(const float* gate_up, int rows, int ff, float* out) {
    for (int r = 0; r < rows; ++r)
        for (int i = 0; i < ff; ++i) {
            const float g = gate_up[static_cast<size_t>(r) * 2 * ff + i], u = gate_up[static_cast<size_t>(r) * 2 * ff + ff + i];
            out[static_cast<size_t>(r) * ff + i] = g / (1.0f + std::exp(-g)) * u;
        }
}

// The double-gated short convolution over the rows of a step (sequence s holds rows
// cu_seqlens[s] .. cu_seqlens[s+1], the first of them at position seq_start[s]), continuing from
// each request's state and leaving the new one:  bcx = [B | C | x]; bx = B * x;
// conv[t] = sum_tap w[ch, tap] * bx[pos(t) - (taps - 1 - tap)], zero before position 0; y = C * (conv + bias).
// state [slots, taps, width]: entry j of a slot holds bx at position (tokens seen) - taps + j.
// (src/backend/cpu/kernels/convolution.cpp:7-60)
void short_conv(const float* bcx, const float* w, const float* bias, float* state, const int* seq_slot, const int* seq_start,
                const int* cu_seqlens, int n_seqs, int width, int taps, float* out) {
    for (int s = 0; s < n_seqs; ++s) {
        const int row0 = cu_seqlens[s], n = cu_seqlens[s + 1] - row0, start = seq_start[s];
        float* st = state + static_cast<size_t>(seq_slot[s]) * taps * width;
        // bx at positions start - taps .. start + n - 1: the state first, then the rows
        std::vector<float> bx(static_cast<size_t>(taps + n) * width);
        for (int j = 0; j < taps; ++j)
            for (int ch = 0; ch < width; ++ch)
                bx[static_cast<size_t>(j) * width + ch] = start - taps + j >= 0 ? st[static_cast<size_t>(j) * width + ch] : 0.f;
        for (int t = 0; t < n; ++t)
            for (int ch = 0; ch < width; ++ch) {
                const float* row = bcx + static_cast<size_t>(row0 + t) * 3 * width;
                bx[static_cast<size_t>(taps + t) * width + ch] = row[ch] * row[2 * width + ch];
            }
        for (int t = 0; t < n; ++t)
            for (int ch = 0; ch < width; ++ch) {
                float conv = 0.f;
                for (int tap = 0; tap < taps; ++tap)       // tap taps-1 multiplies the token's own bx
                    conv = std::fma(w[static_cast<size_t>(ch) * taps + tap], bx[static_cast<size_t>(t + 1 + tap) * width + ch], conv);
                if (bias) conv += bias[ch];
                out[static_cast<size_t>(row0 + t) * width + ch] = bcx[static_cast<size_t>(row0 + t) * 3 * width + width + ch] * conv;
            }
        for (int j = 0; j < taps; ++j)
            for (int ch = 0; ch < width; ++ch) st[static_cast<size_t>(j) * width + ch] = bx[static_cast<size_t>(n + j) * width + ch];
    }
}

// Per head: x = x / sqrt(mean(x^2) + eps) * weight (if a weight is given), then the rotation of
// pair i by angle = float(position) * inv_freq[i] (a 32-bit product), the pair being (i, i + rotary/2)
// (pairing 0) or (2i, 2i + 1) (pairing 1); x is [rows, heads, head_dim], in place.
// (src/backend/cpu/kernels/rope.cpp:61-111)
void qk_norm_rope(float* x, const float* weight, float eps, const float* inv_freq, int rotary_dim, int pairing,
                  const int* positions, int rows, int heads, int head_dim) {
    const int half = rotary_dim / 2;
    for (int r = 0; r < rows; ++r)
        for (int h = 0; h < heads; ++h) {
            float* v = x + (static_cast<size_t>(r) * heads + h) * head_dim;
            if (weight) {
                double sum = 0.0;
                for (int d = 0; d < head_dim; ++d) sum += static_cast<double>(v[d]) * v[d];
                const float inv = static_cast<float>(1.0 / std::sqrt(sum / head_dim + eps));
                for (int d = 0; d < head_dim; ++d) v[d] = v[d] * inv * weight[d];
            }
            if (!inv_freq) continue;
            for (int i = 0; i < half; ++i) {
                const float angle = static_cast<float>(positions[r]) * inv_freq[i];
                const float c = std::cos(angle), s = std::sin(angle);
                const int ia = pairing ? 2 * i : i, ib = pairing ? 2 * i + 1 : i + half;
                const float a = v[ia], b = v[ib];
                v[ia] = a * c - b * s;
                v[ib] = b * c + a * s;
            }
        }
}

// Where a key lies in the pool: pages of page_tokens tokens, a page holding every layer of its
// group, [page][layer][kv_head][token][head_dim]; a value likewise but with the token innermost,
// [page][layer][kv_head][head_dim][token].
static size_t key_at(int page, int n_layers, int layer, int kv_heads, int head, int page_tokens, int in_page, int head_dim) {
    return (((static_cast<size_t>(page) * n_layers + layer) * kv_heads + head) * page_tokens + in_page) * head_dim;
}
static size_t value_at(int page, int n_layers, int layer, int kv_heads, int head, int page_tokens, int in_page, int head_dim, int d) {
    return (((static_cast<size_t>(page) * n_layers + layer) * kv_heads + head) * head_dim + d) * page_tokens + in_page;
}

// The rows' keys and values into the pages of their requests (table [slots, table_stride]: the
// physical page of every logical one).
void kv_store(const float* k, const float* v, float* k_pool, float* v_pool, const int* table, int table_stride,
              const int* token_slot, const int* positions, int rows, int kv_heads, int head_dim, int page_tokens,
              int n_layers, int layer) {
    for (int r = 0; r < rows; ++r) {
        const int page = table[static_cast<size_t>(token_slot[r]) * table_stride + positions[r] / page_tokens];
        for (int h = 0; h < kv_heads; ++h)
            for (int d = 0; d < head_dim; ++d) {
                const size_t src = (static_cast<size_t>(r) * kv_heads + h) * head_dim + d;
                k_pool[key_at(page, n_layers, layer, kv_heads, h, page_tokens, positions[r] % page_tokens, head_dim) + d] = k[src];
                v_pool[value_at(page, n_layers, layer, kv_heads, h, page_tokens, positions[r] % page_tokens, head_dim, d)] = v[src];
            }
    }
}

// Row r (query head j) attends over the keys of its request at positions 0 .. positions[r] (from
// positions[r] - window + 1 with a window), read from the pages; key/value head j / (heads / kv_heads).
// (src/backend/cpu/attention/paged_attention.cpp:229-283)
void paged_attention(const float* q, const float* k_pool, const float* v_pool, const int* table, int table_stride,
                     const int* token_slot, const int* positions, int rows, int heads, int kv_heads, int head_dim,
                     int page_tokens, int n_layers, int layer, float scale, int window, float* out) {
    const int group = heads / kv_heads;
    std::vector<double> score;
    for (int r = 0; r < rows; ++r)
        for (int j = 0; j < heads; ++j) {
            const int g = j / group, last = positions[r];
            const int first = window > 0 ? std::max(0, last - window + 1) : 0;
            const float* qv = q + (static_cast<size_t>(r) * heads + j) * head_dim;
            const int* pages = table + static_cast<size_t>(token_slot[r]) * table_stride;
            score.assign(static_cast<size_t>(last - first + 1), 0.0);
            double top = -INFINITY;
            for (int u = first; u <= last; ++u) {
                const float* kv = k_pool + key_at(pages[u / page_tokens], n_layers, layer, kv_heads, g, page_tokens, u % page_tokens, head_dim);
                double s = 0.0;
                for (int d = 0; d < head_dim; ++d) s += static_cast<double>(qv[d]) * kv[d];
                score[static_cast<size_t>(u - first)] = s * scale;
                top = std::max(top, s * scale);
            }
            double total = 0.0;
            for (double& s : score) { s = std::exp(s - top); total += s; }
            for (int d = 0; d < head_dim; ++d) {
                double o = 0.0;
                for (int u = first; u <= last; ++u)
                    o += score[static_cast<size_t>(u - first)] *
                         v_pool[value_at(pages[u / page_tokens], n_layers, layer, kv_heads, g, page_tokens, u % page_tokens, head_dim, d)];
                out[(static_cast<size_t>(r) * heads + j) * head_dim + d] = static_cast<float>(o / total);
            }
        }
}

// One token from a row of logits, in 32-bit floats as the reference samples
// (src/backend/cpu/sampler.cpp:26-101): seen tokens are penalised (positive logits divided,
// negative ones multiplied); greedy when temperature <= 0 or top_k == 1 (the lowest index wins a
// tie); else the top_k by (score descending, index ascending) of logit / temperature, softmax,
// the shortest prefix whose mass reaches top_p, and a walk down it by u * mass.
int sample(const float* logits, int vocab, float temperature, int top_k, float top_p, float penalty, const unsigned char* seen,
           float u) {
    std::vector<float> pen(logits, logits + vocab);
    if (penalty > 1.0f && seen)
        for (int t = 0; t < vocab; ++t)
            if (seen[t]) pen[static_cast<size_t>(t)] = pen[static_cast<size_t>(t)] >= 0.f ? pen[static_cast<size_t>(t)] / penalty
                                                                                           : pen[static_cast<size_t>(t)] * penalty;
    if (temperature <= 0.0f || top_k == 1) {
        int best = 0;
        for (int t = 1; t < vocab; ++t)
            if (pen[static_cast<size_t>(t)] > pen[static_cast<size_t>(best)]) best = t;
        return best;
    }
    const int k = std::min(top_k, vocab);
    std::vector<float> score(static_cast<size_t>(vocab));
    for (int t = 0; t < vocab; ++t) score[static_cast<size_t>(t)] = pen[static_cast<size_t>(t)] / temperature;
    std::vector<int> order(static_cast<size_t>(vocab));
    for (int t = 0; t < vocab; ++t) order[static_cast<size_t>(t)] = t;
    std::partial_sort(order.begin(), order.begin() + k, order.end(), [&](int a, int b) {
        return score[static_cast<size_t>(a)] > score[static_cast<size_t>(b)] || (score[static_cast<size_t>(a)] == score[static_cast<size_t>(b)] && a < b);
    });
    std::vector<float> prob(static_cast<size_t>(k));
    const float top = score[static_cast<size_t>(order[0])];
    float total = 0.f;
    for (int i = 0; i < k; ++i) {
        prob[static_cast<size_t>(i)] = std::exp(score[static_cast<size_t>(order[static_cast<size_t>(i)])] - top);
        total += prob[static_cast<size_t>(i)];
    }
    for (float& p : prob) p /= total;
    int active = k;
    total = 1.f;
    if (top_p < 1.0f) {
        float cumulative = 0.f;
        active = 0;
        do {
            cumulative += prob[static_cast<size_t>(active)];
            ++active;
        } while (active < k && cumulative < top_p);
        total = 0.f;
        for (int i = 0; i < active; ++i) total += prob[static_cast<size_t>(i)];
    }
    float target = u * total;
    for (int i = 0; i < active; ++i) {
        target -= prob[static_cast<size_t>(i)];
        if (target <= 0.f) return order[static_cast<size_t>(i)];
    }
    return order[static_cast<size_t>(active - 1)];
}

}  // namespace reference
}  // namespace celeg

// ---------------------------------------------------------------------------- by name, for tests
// celeg_reference_call(op, arguments): host addresses and sizes in a JSON object, the function's
// name in `op`; returns JSON ({} or {"token": n}) or null with the reason in celeg_last_error().
#include "../include/celeg_amd.h"
#include "json.hpp"

extern "C" void celeg_set_last_error_(const char* message);

namespace {
using celeg::Json;
template <typename T>
T* at(const Json& a, const char* key) {
    if (!a.contains(key) || a[key].is_null()) return nullptr;
    return reinterpret_cast<T*>(static_cast<uintptr_t>(a[key].as_int()));
}
int num(const Json& a, const char* key) { return static_cast<int>(a[key].as_int()); }
float real(const Json& a, const char* key) { return static_cast<float>(a[key].as_double()); }
thread_local std::string g_answer;
}  // namespace

extern "C" const char* celeg_reference_call(const char* op_name, const char* args_json) {
    namespace ref = celeg::reference;
    try {
        if (!op_name || !args_json) throw std::invalid_argument("celeg_reference_call: op and arguments must not be null");
        const std::string op = op_name;
        const Json a = Json::parse(args_json);
        Json out = Json::object();
        if (op == "embed") {
            ref::embed(at<const float>(a, "table"), num(a, "vocab"), num(a, "width"), at<const int>(a, "ids"), num(a, "rows"), at<float>(a, "out"));
        } else if (op == "rmsnorm") {
            ref::rmsnorm(at<float>(a, "x"), at<const float>(a, "delta"), at<const float>(a, "weight"), real(a, "eps"), num(a, "rows"),
                         num(a, "width"), at<float>(a, "out"));
        } else if (op == "linear") {
            ref::linear(at<const float>(a, "x"), at<const float>(a, "w"), at<const float>(a, "bias"), num(a, "M"), num(a, "N"), num(a, "K"),
                        at<float>(a, "out"));
        } else if (op == "swiglu") {
            ref::swiglu(at<const float>(a, "gate_up"), num(a, "rows"), num(a, "ff"), at<float>(a, "out"));
        } else if (op == "short_conv") {
            ref::short_conv(at<const float>(a, "bcx"), at<const float>(a, "w"), at<const float>(a, "bias"), at<float>(a, "state"),
                            at<const int>(a, "seq_slot"), at<const int>(a, "seq_start"), at<const int>(a, "cu_seqlens"), num(a, "n_seqs"),
                            num(a, "width"), num(a, "taps"), at<float>(a, "out"));
        } else if (op == "qk_norm_rope") {
            ref::qk_norm_rope(at<float>(a, "x"), at<const float>(a, "weight"), real(a, "eps"), at<const float>(a, "inv_freq"),
                              num(a, "rotary_dim"), num(a, "pairing"), at<const int>(a, "positions"), num(a, "rows"), num(a, "heads"),
                              num(a, "head_dim"));
        } else if (op == "kv_store") {
            ref::kv_store(at<const float>(a, "k"), at<const float>(a, "v"), at<float>(a, "k_pool"), at<float>(a, "v_pool"),
                          at<const int>(a, "table"), num(a, "table_stride"), at<const int>(a, "token_slot"), at<const int>(a, "positions"),
                          num(a, "rows"), num(a, "kv_heads"), num(a, "head_dim"), num(a, "page_tokens"), num(a, "n_layers"), num(a, "layer"));
        } else if (op == "paged_attention") {
            ref::paged_attention(at<const float>(a, "q"), at<const float>(a, "k_pool"), at<const float>(a, "v_pool"), at<const int>(a, "table"),
                                 num(a, "table_stride"), at<const int>(a, "token_slot"), at<const int>(a, "positions"), num(a, "rows"),
                                 num(a, "heads"), num(a, "kv_heads"), num(a, "head_dim"), num(a, "page_tokens"), num(a, "n_layers"),
                                 num(a, "layer"), real(a, "scale"), num(a, "window"), at<float>(a, "out"));
        } else if (op == "sample") {
            out.set("token", ref::sample(at<const float>(a, "logits"), num(a, "vocab"), real(a, "temperature"), num(a, "top_k"),
                                         real(a, "top_p"), real(a, "penalty"), at<const unsigned char>(a, "seen"), real(a, "u")));
        } else {
            throw std::invalid_argument("celeg_reference_call: unknown function '" + op + "'");
        }
        g_answer = out.dump();
        return g_answer.c_str();
    } catch (const std::exception& e) {
        celeg_set_last_error_(e.what());
        return nullptr;
    }
}
