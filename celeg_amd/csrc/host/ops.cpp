#include "ops.hpp"

#include <algorithm>
#include <functional>

#include "kernels.hpp"

namespace celeg {

namespace {
int dt(const Tensor& t, const char* name) {
    if (t.dtype != DType::F32 && t.dtype != DType::BF16)
        throw KernelError(std::string(name) + ": dtype " + dtype_name(t.dtype) + " is not supported (float32, bfloat16)");
    return static_cast<int>(t.dtype);
}
void need(bool ok, const std::string& message) {
    if (!ok) throw KernelError(message);
}
void dev(const Tensor& t, const char* name) {
    if (!t.defined()) throw KernelError(std::string(name) + " is missing");
}
void dev(const Tensor& t, const char* name, DType dtype, bool contiguous = true) {
    dev(t, name);
    if (t.dtype != dtype)
        throw KernelError(std::string(name) + " must be " + dtype_name(dtype) + ", got " + dtype_name(t.dtype));
    if (contiguous && !t.contiguous()) throw KernelError(std::string(name) + " must be contiguous");
}
// row stride of a 2-D tensor whose rows are dense
int rows_of(const Tensor& t, const char* name) {
    if (t.ndim != 2 || (t.shape[1] > 1 && t.stride[1] != 1))
        throw KernelError(std::string(name) + " must be 2-D with dense rows");
    return static_cast<int>(t.row_stride());
}
struct Operand {
    long long rows, width, ld, k8;
};
// (rows, width, row stride, stride of a group of 8 values) of a bfloat16 operand: [rows, width]
// with dense rows, or [rows, width/8, 8], a view of a buffer in which the rows lie side by side
// inside every group of 8 values
Operand operand(const Tensor& t, const char* name) {
    if (t.ndim == 2) return {t.shape[0], t.shape[1], rows_of(t, name), 8};
    if (t.ndim != 3 || t.shape[2] != 8 || t.stride[2] != 1)
        throw KernelError(std::string(name) + " must be [rows, width] or [rows, width/8, 8]");
    return {t.shape[0], t.shape[1] * 8, t.stride[0], t.stride[1]};
}
}  // namespace

const char* path_name(Path p) {
    switch (p) {
        case Path::AttentionDecode: return "attention_decode";
        case Path::AttentionDecodeFresh: return "attention_decode_fresh";
        case Path::AttentionRows: return "attention_rows";
        case Path::AttentionGeneral: return "attention_general";
        case Path::LinearF32: return "linear_f32";
        case Path::LinearLibrary: return "linear_library";
        case Path::LinearStandIn: return "linear_stand_in";
        case Path::FusedSliced: return "fused_sliced";
        case Path::FusedRows: return "fused_rows";
        case Path::FusedStaged: return "fused_staged";
        case Path::ArgmaxMerged: return "argmax_merged";
        case Path::Tiled: return "tiled";
        case Path::TiledQkv: return "tiled_qkv";
        default: return "?";
    }
}

Json Ops::paths_json() const {
    Json out = Json::object();
    for (int i = 0; i < static_cast<int>(Path::Count); ++i) out.set(path_name(static_cast<Path>(i)), path_count[i]);
    return out;
}

// the bound on the context that a step's decode attention is launched for: the step's longest
// context, or what the step's recorded graph is good for
static int hint_of(const StepBatch& batch, const KVView& kv) {
    const int max_context = kv.table_stride * kv.page_tokens;
    const int hint = batch.context_hint();
    return hint ? std::min(hint, max_context) : max_context;
}

// ---------------------------------------------------------------------------- row-wise
void Ops::embed(const Tensor& table, const int* token_ids, const Tensor& out) {
    dev(table, "table");
    dev(out, "out", DType::F32);
    need(table.ndim == 2 && out.ndim == 2 && table.shape[1] == out.shape[1] && table.contiguous(), "embed: shapes do not fit");
    kernel_check(celeg_embed(table.data, dt(table, "table"), token_ids, out.as<float>(), static_cast<int>(out.shape[0]),
                             static_cast<int>(out.shape[1]), static_cast<int>(table.shape[0]), stream), "embed");
}

void Ops::rmsnorm(const Tensor& x, const Tensor& weight, float eps, const Tensor& out, const Tensor* delta, const int* rows) {
    dev(x, "x");
    dev(weight, "weight", DType::F32);
    dev(out, "out");
    need(x.ndim == 2 && out.ndim == 2 && x.contiguous() && out.contiguous(), "rmsnorm: x and out must be contiguous matrices");
    const long long width = x.shape[1], n_rows = out.shape[0];
    need(out.shape[1] == width && weight.numel() == width, "rmsnorm: shapes do not fit");
    if (delta) {
        dev(*delta, "delta");
        need(delta->ndim == 2 && delta->shape[0] == x.shape[0] && delta->shape[1] == width && delta->contiguous(),
             "rmsnorm: delta must have the shape of x");
    }
    if (!rows) need(n_rows == x.shape[0], "rmsnorm: out must have the rows of x");
    const int write_back = delta && !rows ? 1 : 0;
    need(!write_back || x.dtype == DType::F32, "rmsnorm: the sum can only be written back to a 32-bit x");
    kernel_check(celeg_rmsnorm(x.data, dt(x, "x"), delta ? delta->data : nullptr, delta ? dt(*delta, "delta") : 0,
                               weight.as<float>(), out.data, dt(out, "out"), rows, static_cast<int>(n_rows),
                               static_cast<int>(width), eps, write_back, stream), "rmsnorm");
}

void Ops::swiglu(const Tensor& gate_up, const Tensor& out) {
    dev(gate_up, "gate_up");
    dev(out, "out", gate_up.dtype);
    need(out.ndim == 2 && gate_up.ndim == 2 && gate_up.shape[0] == out.shape[0] && gate_up.shape[1] == 2 * out.shape[1] &&
             gate_up.contiguous() && out.contiguous(), "swiglu: gate_up must be [rows, 2*ff]");
    kernel_check(celeg_swiglu(gate_up.data, out.data, dt(out, "out"), static_cast<int>(out.shape[0]),
                              static_cast<int>(out.shape[1]), stream), "swiglu");
}

void Ops::add_bias(const Tensor& x, const Tensor& bias) {
    dev(x, "x");
    dev(bias, "bias", DType::F32);
    need(x.ndim == 2 && x.contiguous() && bias.numel() == x.shape[1], "add_bias: bias must have the width of x");
    kernel_check(celeg_add_bias(x.data, dt(x, "x"), bias.as<float>(), static_cast<int>(x.shape[0]),
                                static_cast<int>(x.shape[1]), stream), "add_bias");
}

void Ops::cast(const Tensor& src, const Tensor& dst) {
    dev(src, "src");
    dev(dst, "dst");
    need(src.numel() == dst.numel() && src.contiguous() && dst.contiguous(), "cast: sizes differ");
    kernel_check(celeg_cast(src.data, dt(src, "src"), dst.data, dt(dst, "dst"), static_cast<size_t>(src.numel()), stream), "cast");
}

void Ops::apply_table_updates(int* table, int stride, int rows, const int* updates, int capacity) {
    kernel_check(celeg_table_update(table, stride, rows, updates, capacity, stream), "apply_table_updates");
}

void Ops::step_prologue(int* table, int stride, int rows, const int* updates, int capacity, int* token_ids,
                        const int* token_slot, const int* last_tokens, int n) {
    need(capacity > 0, "step_prologue: the update list is shorter than its capacity");
    kernel_check(celeg_step_prologue(table, stride, rows, updates, capacity, token_ids, token_slot, last_tokens, n, stream),
                 "step_prologue");
}

void Ops::resolve_tokens(int* token_ids, const int* token_slot, const int* last_tokens, int n) {
    kernel_check(celeg_resolve_tokens(token_ids, token_slot, last_tokens, n, stream), "resolve_tokens");
}

// ---------------------------------------------------------------------------- products
void Ops::library_product(const Tensor& x, const Tensor& w, const Tensor& out, Workspace& ws) {
    const int M = static_cast<int>(x.shape[0]), K = static_cast<int>(x.shape[1]), N = static_cast<int>(w.shape[0]);
    if (use_blaslt) {
        if (!blaslt_) blaslt_ = std::make_unique<BlasLt>();
        if (blaslt_->matmul(x.data, rows_of(x, "x"), w.data, out.data, rows_of(out, "out"), M, N, K, stream)) {
            took(Path::LinearLibrary);
            return;
        }
    }
    // sizes the library has no kernel for: the tiled product where the sizes fit it, else the
    // 32-bit product on widened copies
    if (K % 64 == 0 && N % 4 == 0 && rows_of(x, "x") % 8 == 0 && rows_of(out, "out") % 4 == 0) {
        tiled_linear(x, w, out, Epilogue::Store, 0.f, nullptr, 0, nullptr, nullptr, nullptr);
        return;
    }
    Tensor xf = ws.buf("product_x32", DType::F32, {M, K}), wf = ws.buf("product_w32", DType::F32, {N, K});
    Tensor yf = ws.buf("product_y32", DType::F32, {M, N});
    if (x.contiguous()) {
        cast(x, xf);
    } else {
        for (int m = 0; m < M; ++m) cast(x.rows(m, 1), xf.rows(m, 1));
    }
    cast(w, wf);
    took(Path::LinearStandIn);
    kernel_check(celeg_gemm_f32(xf.as<float>(), K, wf.as<float>(), K, nullptr, yf.as<float>(), N, M, N, K, stream),
                 "linear (32-bit stand-in)");
    if (out.contiguous()) {
        cast(yf, out);
    } else {
        for (int m = 0; m < M; ++m) cast(yf.rows(m, 1), out.rows(m, 1));
    }
}

// out = x w^T (+ bias).  x [M,K] (rows may be strided), w [N,K], out [M,N] in the dtype of x or
// in 32-bit.
void Ops::linear(const Tensor& x, const Tensor& w, const Tensor& out, const Tensor* bias, Workspace& ws) {
    dev(x, "x");
    dev(w, "w");
    dev(out, "out");
    need(x.ndim == 2 && w.ndim == 2 && out.ndim == 2 && w.contiguous(), "linear: x, w and out must be matrices");
    const long long M = x.shape[0], K = x.shape[1], N = w.shape[0];
    need(w.shape[1] == K && out.shape[0] == M && out.shape[1] == N,
         "linear: shapes do not fit: x [" + std::to_string(M) + ", " + std::to_string(K) + "], w [" + std::to_string(N) +
             ", " + std::to_string(w.shape[1]) + "], out [" + std::to_string(out.shape[0]) + ", " + std::to_string(out.shape[1]) + "]");
    if (bias) {
        dev(*bias, "bias", DType::F32);
        need(bias->numel() == N, "linear: bias must have one entry per output column");
    }
    if (M == 0) return;
    if (x.dtype == DType::F32 && w.dtype == DType::F32) {
        need(out.dtype == DType::F32, "linear: a 32-bit product needs a 32-bit output");
        took(Path::LinearF32);
        kernel_check(celeg_gemm_f32(x.as<float>(), rows_of(x, "x"), w.as<float>(), static_cast<int>(K),
                                    bias ? bias->as<float>() : nullptr, out.as<float>(), rows_of(out, "out"),
                                    static_cast<int>(M), static_cast<int>(N), static_cast<int>(K), stream), "linear (32-bit)");
        return;
    }
    if (x.dtype == DType::BF16 && w.dtype == DType::F32) {
        // a matrix stored in 32-bit stays 32-bit: widen the rows and use the 32-bit product
        Tensor xf = ws.buf("linear_x32", DType::F32, {M, K});
        if (x.contiguous()) {
            cast(x, xf);
        } else {
            for (long long m = 0; m < M; ++m) cast(x.rows(m, 1), xf.rows(m, 1));
        }
        if (out.dtype == DType::F32) {
            linear(xf, w, out, bias, ws);
        } else {
            Tensor yf = ws.buf("linear_y32", DType::F32, {M, N});
            linear(xf, w, yf, bias, ws);
            if (out.contiguous()) {
                cast(yf, out);
            } else {
                for (long long m = 0; m < M; ++m) cast(yf.rows(m, 1), out.rows(m, 1));
            }
        }
        return;
    }
    need(x.dtype == DType::BF16 && w.dtype == DType::BF16,
         std::string("linear: unsupported dtypes ") + dtype_name(x.dtype) + " x " + dtype_name(w.dtype));
    if (out.dtype == DType::BF16) {
        library_product(x, w, out, ws);
        if (bias) add_bias(out, *bias);
    } else if (out.dtype == DType::F32) {
        Tensor tmp = ws.buf("linear_bf16_out", DType::BF16, {M, N});
        library_product(x, w, tmp, ws);
        cast(tmp, out);
        if (bias) add_bias(out, *bias);
    } else {
        throw KernelError("linear: out must be bfloat16 or float32");
    }
}

// ---------------------------------------------------------------------------- short convolution
void Ops::short_conv(const Tensor& bcx, const Tensor& weight, const Tensor* bias, const Tensor& state, const Tensor& out,
                     const StepBatch& batch) {
    dev(bcx, "bcx");
    dev(weight, "weight", DType::F32);
    dev(state, "state", DType::F32, false);
    dev(out, "out", bcx.dtype);
    need(out.ndim == 2 && bcx.ndim == 2 && weight.ndim == 2 && bcx.contiguous() && out.contiguous(), "short_conv: shapes do not fit");
    const long long T = out.shape[0], width = out.shape[1], taps = weight.shape[1];
    need(bcx.shape[0] == T && bcx.shape[1] == 3 * width && weight.shape[0] == width && T == batch.n_tokens,
         "short_conv: shapes do not fit");
    need(state.ndim == 3 && state.shape[1] == taps && state.shape[2] == width && state.stride[2] == 1 && state.stride[1] == width,
         "short_conv: state must be [slots, taps, width] with dense slots");
    if (bias) dev(*bias, "bias", DType::F32);
    kernel_check(celeg_short_conv(bcx.data, static_cast<int>(3 * width), dt(bcx, "bcx"), weight.as<float>(),
                                  bias ? bias->as<float>() : nullptr, state.as<float>(), static_cast<size_t>(state.stride[0]),
                                  out.data, batch.positions, batch.token_seq, batch.seq_start, batch.seq_slot,
                                  batch.cu_seqlens, batch.n_tokens, batch.n_seqs, static_cast<int>(width),
                                  static_cast<int>(taps), stream), "short_conv");
}

// ---------------------------------------------------------------------------- attention
static void check_kv(const KVView& kv, int kv_heads, int head_dim, DType dtype) {
    need(kv.kv_heads == kv_heads && kv.head_dim == head_dim, "attention: the cache has other head sizes than the mixer");
    need(kv.v_head_dim == head_dim, "attention: these kernels take values of the keys' width only");
    need(kv.k && kv.v && kv.table, "attention: the cache has no device memory");
    need(kv.dtype == dtype, std::string("attention: the cache holds ") + dtype_name(kv.dtype) + ", the rows are " + dtype_name(dtype));
    need(kv.layer >= 0 && kv.layer < kv.n_layers, "attention: layer index outside the cache");
}

// cos and sin of position * frequency for every position a request can reach
// ([n_positions, rotary_dim/2, 2], 32-bit), made once per frequency table
const float* Ops::rope_table(const Tensor& inv_freq, int n_positions) {
    const auto key = std::make_pair(static_cast<const void*>(inv_freq.data), n_positions);
    auto it = rope_tables_.find(key);
    if (it == rope_tables_.end()) {
        auto table = device_tensor(DType::F32, {n_positions, inv_freq.numel(), 2});
        kernel_check(celeg_rope_table(inv_freq.as<float>(), static_cast<int>(inv_freq.numel()), n_positions,
                                      table->view.as<float>(), stream), "rope_table");
        it = rope_tables_.emplace(key, table).first;
    }
    return it->second->view.as<float>();
}

void Ops::forget_rope_tables(const void* inv_freq) {
    for (auto it = rope_tables_.begin(); it != rope_tables_.end();) {
        if (it->first.first == inv_freq) {
            retired_rope_tables_.push_back(it->second);
            it = rope_tables_.erase(it);
        } else {
            ++it;
        }
    }
}

void Ops::qk_norm_rope_store(const Tensor& q, const Tensor* k, const Tensor* v, const Tensor* q_weight,
                             const Tensor* k_weight, float eps, const Tensor* inv_freq, int rotary_dim, int pairing, int heads,
                             int kv_heads, int head_dim, const StepBatch& batch, const KVView& kv) {
    dev(q, "q");
    const long long T = q.shape[0];
    need(q.ndim == 2 && T == batch.n_tokens && q.shape[1] == static_cast<long long>(heads) * head_dim,
         "qk_norm_rope_store: q must be [rows, heads*head_dim]");
    need(head_dim % 2 == 0 && head_dim <= 1024,
         "qk_norm_rope_store: head_dim " + std::to_string(head_dim) + " must be even and <= 1024");
    check_kv(kv, kv_heads, head_dim, q.dtype);
    const bool store = k != nullptr;
    if (store) {
        need(v != nullptr, "qk_norm_rope_store: k without v");
        dev(*k, "k", q.dtype, false);
        dev(*v, "v", q.dtype, false);
        const long long kvw = static_cast<long long>(kv_heads) * head_dim;
        need(k->ndim == 2 && v->ndim == 2 && k->shape[0] == T && k->shape[1] == kvw && v->shape[0] == T && v->shape[1] == kvw,
             "qk_norm_rope_store: k and v must be [rows, kv_heads*head_dim]");
    }
    for (const Tensor* wt : {q_weight, k_weight})
        if (wt) {
            dev(*wt, "q/k norm weight", DType::F32);
            need(wt->numel() == head_dim, "qk_norm_rope_store: a norm weight must have head_dim entries");
        }
    if (inv_freq) {
        dev(*inv_freq, "inv_freq", DType::F32);
        need(rotary_dim % 2 == 0 && rotary_dim <= head_dim && inv_freq->numel() == rotary_dim / 2,
             "qk_norm_rope_store: rotary_dim and the frequency table disagree");
        need(pairing == 0 || pairing == 1, "qk_norm_rope_store: pairing is 0 (halves) or 1 (neighbours)");
    }
    const float* cos_sin = nullptr;
    if (inv_freq && rotary_dim > 0 && use_rope_table) cos_sin = rope_table(*inv_freq, kv.table_stride * kv.page_tokens);
    kernel_check(celeg_qk_norm_rope_store(
                     q.data, rows_of(q, "q"), store ? k->data : nullptr, store ? rows_of(*k, "k") : 0,
                     store ? v->data : nullptr, store ? rows_of(*v, "v") : 0, dt(q, "q"),
                     q_weight ? q_weight->as<float>() : nullptr, (store && k_weight) ? k_weight->as<float>() : nullptr, eps,
                     inv_freq ? inv_freq->as<float>() : nullptr, cos_sin, rotary_dim, pairing, batch.positions, batch.token_slot,
                     kv.table, kv.table_stride, kv.k, kv.v, kv.n_layers, kv.layer, kv.page_tokens, static_cast<int>(T),
                     heads, kv_heads, head_dim, store ? 1 : 0, stream), "qk_norm_rope_store");
}

// The conditions under which paged_attention hands a decode-only step to the kernels for single
// rows, and those can prepare the step's own keys and values (the rotation: none, or of the whole
// head by split halves from the table).
bool Ops::attention_fresh_ok(int heads, int head_dim, const Tensor* inv_freq, int rotary_dim, int pairing, const StepBatch& batch,
                             const KVView& kv, DType dtype) const {
    if (!use_fresh_decode || dtype != DType::BF16 || kv.dtype != DType::BF16 || attention_general) return false;
    if (kv.page_tokens < 16 || (kv.page_tokens & (kv.page_tokens - 1))) return false;
    if ((head_dim != 64 && head_dim != 128) || kv.head_dim != head_dim || (kv.v_head_dim && kv.v_head_dim != head_dim)) return false;
    if (!batch.decode_only || batch.n_seqs != batch.n_tokens) return false;
    // (measured with heads of 64 only)
    if (head_dim != 64) return false;
    // Which kernel attention_decode will take: one workgroup a (request, key/value head), or parts
    // of 1, 4 or 16 rounds.  In parts of many rounds every wavefront prepares q before it asks for
    // its keys, which pays where a compute unit runs one such workgroup and costs more than the
    // kernel it saves where it runs many in turn (8 requests at 8,192 and 32,768 tokens, 2,112
    // workgroups: 1 and 5 us a layer slower; 1 request at 16,384, 136 workgroups: 4 us a layer
    // faster; 264 workgroups: 1 us a layer faster).
    const int chunks = (heads / kv.kv_heads + 15) / 16;
    const long long groups = static_cast<long long>(kv.kv_heads) * chunks * batch.n_tokens;
    const int rounds = (hint_of(batch, kv) + 63) / 64;
    const bool whole = decode_whole(groups, rounds);
    if (whole) {
        // the kernel's loop over the rounds runs 1.7 % slower in this form, which outweighs the
        // kernel saved from about 8,192 tokens for each of 64 requests on (at 32,768: 4.94 against
        // 4.86 ms a step; at 2,048: 0.906 against 0.916)
        if (static_cast<long long>(batch.n_tokens) * rounds > 4096) return false;
    } else {
        const int split_rounds = decode_split_rounds(groups, rounds);
        if (split_rounds > 1 && groups * ((rounds + split_rounds - 1) / split_rounds) > 512) return false;
    }
    return !inv_freq || (rotary_dim == head_dim && pairing == 0 && use_rope_table);
}

void Ops::paged_attention(const Tensor& q, const Tensor& out, int heads, int kv_heads, int head_dim, float scale,
                          int window, const StepBatch& batch, const KVView& kv, Workspace& ws, const FreshKV* fresh) {
    dev(q, "q");
    dev(out, "out", q.dtype);
    const long long T = q.shape[0], qw = static_cast<long long>(heads) * head_dim;
    need(q.ndim == 2 && out.ndim == 2 && T == batch.n_tokens && q.shape[1] == qw && out.shape[0] == T && out.shape[1] == qw &&
             out.contiguous(), "paged_attention: q and out must be [rows, heads*head_dim]");
    need(head_dim <= 256, "paged_attention: head_dim " + std::to_string(head_dim) + " exceeds 256");
    need(heads % kv_heads == 0, "paged_attention: heads must be a multiple of kv_heads");
    check_kv(kv, kv_heads, head_dim, q.dtype);
    const int ldq = rows_of(q, "q");
    if (q.dtype == DType::BF16 && !attention_general && kv.page_tokens >= 16 &&
        (kv.page_tokens & (kv.page_tokens - 1)) == 0 && ldq % 8 == 0) {
        const bool decode_hd = head_dim == 64 || head_dim == 128;
        if (batch.decode_only && decode_hd && batch.n_seqs == T) {
            attention_decode(q, out, heads, kv_heads, head_dim, scale, window, batch, kv, static_cast<int>(T), ws, fresh);
            return;
        }
        need(!fresh, "paged_attention: fresh keys and values go with decode-only steps");
        if (head_dim == 32 || head_dim == 64 || head_dim == 96 || head_dim == 128) {
            // entries of one token lie first: they go to the kernel for single rows (a tile of
            // the rows kernel would hold one row), the portions to the rows kernel
            const int single = decode_hd ? batch.single_rows : 0;
            if (single) attention_decode(q, out, heads, kv_heads, head_dim, scale, window, batch, kv, single, ws);
            if (single < batch.n_seqs) took(Path::AttentionRows);
            if (single < batch.n_seqs)
                kernel_check(celeg_attention_rows_bf16(
                                 q.data, ldq, kv.k, kv.v, kv.table, kv.table_stride, batch.cu_seqlens + single,
                                 batch.seq_slot + single, batch.seq_start + single, batch.n_seqs - single,
                                 static_cast<int>(T) - single, out.data, static_cast<int>(qw), heads, kv_heads, head_dim,
                                 kv.page_tokens, kv.n_layers, kv.layer, scale, window, attention_rows_per_tile,
                                 attention_rows_form, batch.context_hint(), stream), "attention over rows (bfloat16)");
            return;
        }
    }
    need(!fresh, "paged_attention: fresh keys and values go with the kernels for single rows");
    took(Path::AttentionGeneral);
    kernel_check(celeg_paged_attention(q.data, ldq, kv.k, kv.v, dt(q, "q"), kv.table, kv.table_stride, batch.token_slot,
                                       batch.positions, out.data, static_cast<int>(qw), static_cast<int>(T), heads,
                                       kv_heads, head_dim, kv.page_tokens, kv.n_layers, kv.layer, scale, window, stream),
                 "paged_attention");
}

// Where the context of few requests is cut into parts: how many wavefronts a part's workgroup has
// (1, 4 or 16: as many rounds of 64 keys does it take at a time; a request's rounds are shared out
// evenly over its parts).  Workgroups of 16 where they give every compute unit just one (8 requests
// of 8 key/value heads at up to 4,096 tokens: 0.463 against 0.475 and 0.479 ms a decode step; 2
// requests at up to 16,384: 3 % faster); else by the length, so that a long context gets longer
// parts rather than hundreds of them, and at short lengths workgroups of 4 once there are enough
// of them for half the compute units (1, 2, 4 and 16 requests at 2,048 tokens: 0.5 to 1.4 % faster
// than single wavefronts).  Measured at 1 to 16 requests, 2,048 and 8,192 tokens.
// One workgroup a (request, key/value head), its wavefronts taking the rounds in turn and no second
// kernel, once there are enough of them: 192 (24 requests of 8 key/value heads) at any length, 96 at
// contexts up to 4,096 tokens (12 and 16 requests at 2,048 tokens: 1 and 3 % of a decode step
// faster than in parts; 16 requests at 8,192: 3 % slower).
bool Ops::decode_whole(long long groups, int rounds) const {
    if (attention_decode_whole >= 0) return attention_decode_whole > 0;
    return groups >= 192 || (groups >= 96 && rounds <= 64);
}

int Ops::decode_split_rounds(long long groups, int rounds) const {
    const long long long_parts = groups * ((rounds + 15) / 16);
    if (decode_parts_fill && rounds > 16 && long_parts >= 192 && long_parts <= 256) return 16;
    if (rounds <= decode_part_thresholds[0]) return decode_parts_fill && rounds > 4 && groups * ((rounds + 3) / 4) >= 128 ? 4 : 1;
    return rounds <= decode_part_thresholds[1] ? 4 : 16;
}

// The first T rows of the step, each the one new token of its request.
void Ops::attention_decode(const Tensor& q, const Tensor& out, int heads, int kv_heads, int head_dim, float scale,
                           int window, const StepBatch& batch, const KVView& kv, int T, Workspace& ws, const FreshKV* fresh) {
    const int max_context = kv.table_stride * kv.page_tokens;
    // where the context is cut into parts (few requests): parts of 1, 4 or 16 rounds of 64 keys,
    // so that a long context gets longer parts rather than hundreds of them; the bound is the
    // step's longest context, or what the step's recorded graph is good for
    const int hint = batch.context_hint();
    const int bound = hint ? std::min(hint, max_context) : max_context;
    const int rounds = (bound + 63) / 64;
    const int chunks = (heads / kv_heads + 15) / 16;
    const int whole = decode_whole(static_cast<long long>(kv_heads) * chunks * T, rounds) ? 1 : 0;
    const int split_rounds = decode_split_rounds(static_cast<long long>(kv_heads) * chunks * T, rounds);
    const int n_parts = (rounds + split_rounds - 1) / split_rounds;
    const size_t parts = static_cast<size_t>(T) * heads * n_parts;
    float* workspace = static_cast<float*>(ws.raw("attention_decode_parts", parts * (head_dim + 2) * sizeof(float)));
    if (fresh) {
        need(fresh->k && fresh->v, "attention_decode: fresh keys and values are missing");
        const long long kvw = static_cast<long long>(kv_heads) * head_dim;
        for (const Tensor* t : {fresh->k, fresh->v}) {
            dev(*t, "fresh k/v", DType::BF16, false);
            need(t->ndim == 2 && t->shape[0] == T && t->shape[1] == kvw, "attention_decode: fresh k and v must be [rows, kv_heads*head_dim]");
        }
        for (const Tensor* wt : {fresh->q_weight, fresh->k_weight})
            if (wt) {
                dev(*wt, "q/k norm weight", DType::F32);
                need(wt->numel() == head_dim, "attention_decode: a norm weight must have head_dim entries");
            }
        const float* cos_sin = nullptr;
        if (fresh->inv_freq) {
            dev(*fresh->inv_freq, "inv_freq", DType::F32);
            need(fresh->inv_freq->numel() == head_dim / 2, "attention_decode: the frequency table must have head_dim / 2 entries");
            cos_sin = rope_table(*fresh->inv_freq, kv.table_stride * kv.page_tokens);
        }
        took(Path::AttentionDecodeFresh);
        kernel_check(celeg_attention_decode_fresh_bf16(
                         q.data, rows_of(q, "q"), fresh->k->data, rows_of(*fresh->k, "k"), fresh->v->data, rows_of(*fresh->v, "v"),
                         fresh->q_weight ? fresh->q_weight->as<float>() : nullptr, fresh->k_weight ? fresh->k_weight->as<float>() : nullptr,
                         fresh->eps, cos_sin, kv.k, kv.v, kv.table, kv.table_stride, batch.token_slot, batch.positions, workspace,
                         workspace + parts * head_dim, n_parts, out.data, heads * head_dim, T, heads, kv_heads, head_dim,
                         kv.page_tokens, kv.n_layers, kv.layer, scale, window, whole, split_rounds, n_parts, stream),
                     "attention for decode rows with fresh keys (bfloat16)");
        return;
    }
    took(Path::AttentionDecode);
    kernel_check(celeg_attention_decode_bf16(q.data, rows_of(q, "q"), kv.k, kv.v, kv.table, kv.table_stride, batch.token_slot,
                                             batch.positions, workspace, workspace + parts * head_dim, n_parts, out.data,
                                             heads * head_dim, T, heads, kv_heads, head_dim, kv.page_tokens, kv.n_layers,
                                             kv.layer, scale, window, whole, split_rounds, n_parts, stream),
                 "attention for decode rows (bfloat16)");
}

// ---------------------------------------------------------------------------- sampling
void Ops::sample(const Tensor& logits, const float* fparams, const int* iparams, uint8_t* seen, size_t seen_stride,
                 int* out_tokens, int* last_tokens, bool all_greedy, Workspace& ws, const HeadBest* head_best, bool penalised) {
    dev(logits, "logits", DType::F32, false);
    const int R = static_cast<int>(logits.shape[0]), V = static_cast<int>(logits.shape[1]);
    if (R == 0) return;
    // what the head's product left beside these very logits, if it did
    const bool left = use_head_argmax && head_best && head_best->logits == logits.data && head_best->rows >= R &&
                      head_best->parts > 0 && head_best->cols > 0;
    if (all_greedy && !penalised && left) {
        // greedy rows without a penalty (the caller's word): the head's kernel left the best of every
        // share of a row's columns, so the logits need not be read again
        took(Path::ArgmaxMerged);
        kernel_check(celeg_argmax_merge(head_best->best, head_best->ld, head_best->parts, R, iparams, out_tokens, last_tokens,
                                        stream), "argmax from the head's parts");
        return;
    }
    if (all_greedy && use_argmax_parts && R <= 16) {     // (64 rows: 23 us against 12 us, one workgroup a row)
        // per row: the best (value, index) so far and a count of the parts that have arrived;
        // zero at first, and the kernel leaves both at zero for its next launch
        if (!argmax_state_.ptr()) argmax_state_ = DeviceBuffer(64 * (sizeof(unsigned long long) + sizeof(unsigned int)), true);
        char* state = argmax_state_.as<char>();
        kernel_check(celeg_argmax_rows(logits.as<float>(), rows_of(logits, "logits"), R, V, fparams, iparams, seen,
                                       seen_stride, out_tokens, last_tokens, reinterpret_cast<unsigned long long*>(state),
                                       reinterpret_cast<unsigned int*>(state + 64 * sizeof(unsigned long long)), stream),
                     "argmax of rows");
        return;
    }
    // (A row of a sampled step cut into parts over many workgroups, the last one to arrive merging
    // the parts' lists, was measured: 21 against 23 us for one row of 65,536 logits and top_k 50,
    // slower from 8 rows on and at top_k 128: what the kernel spends lies in the ranking and the
    // sums, not in reading the logits.)
    // (sampled rows find their candidates among the columns of the parts whose best logit is large enough,
    // without reading the row, where the head left such parts)
    kernel_check(celeg_sample(logits.as<float>(), rows_of(logits, "logits"), R, V, fparams, iparams, seen, seen_stride,
                              out_tokens, last_tokens, left ? head_best->best : nullptr, left ? head_best->ld : 0,
                              left ? head_best->parts : 0, left ? head_best->cols : 0, stream), "sample");
}

void Ops::mark_seen(uint8_t* seen, size_t stride, int n_slots, int vocab, const int* token_ids, const int* token_slot, int n) {
    kernel_check(celeg_mark_seen(seen, stride, n_slots, vocab, token_ids, token_slot, n, stream), "mark_seen");
}

// ---------------------------------------------------------------------------- fused skinny products
bool Ops::fused_linear_ok(int rows, std::initializer_list<long long> inner) const {
    if (rows <= 0 || rows > 64) return false;
    for (long long k : inner)
        if (k <= 0 || k % 8) return false;
    return true;
}

bool Ops::rows_kernel_ok(int rows, std::initializer_list<long long> inner) const {
    if (!use_rows_kernel || rows < rows_kernel_min_rows || rows > 64) return false;
    for (long long k : inner)
        if (k % 32) return false;
    return true;
}

int Ops::residual_stat_blocks(int rows, int n, int k) const {
    if (rows_kernel_ok(rows, {k})) return celeg_gemm_rows_blocks(rows, n, k, static_cast<int>(Epilogue::Residual));
    if (rows <= 16 && use_sliced) return celeg_gemv_slices_blocks(rows, n, k);
    return (n + 15) / 16;
}

void Ops::stream_prepare(const Tensor& h, const Tensor& xb, const Tensor& stats) {
    dev(h, "h", DType::F32, false);
    dev(xb, "xb", DType::BF16, false);
    dev(stats, "stats", DType::F32);
    const long long rows = h.shape[0], width = h.shape[1];
    const Operand o = operand(xb, "xb");
    need(o.rows >= rows && o.width == width && stats.shape[0] >= rows, "stream_prepare: shapes do not fit");
    kernel_check(celeg_stream_prepare(h.as<float>(), rows_of(h, "h"), xb.data, static_cast<int>(o.ld), o.k8,
                                      stats.as<float>(), static_cast<int>(stats.stride[0]), static_cast<int>(rows),
                                      static_cast<int>(width), stream), "stream_prepare");
}

void Ops::embed_stream(const Tensor& table, const int* token_ids, const Tensor& out, const Tensor& xb, const Tensor& stats,
                       const StepPrologue* prologue) {
    dev(table, "table", DType::BF16);
    dev(out, "out", DType::F32);
    dev(xb, "xb", DType::BF16, false);
    dev(stats, "stats", DType::F32);
    const long long rows = out.shape[0], width = out.shape[1];
    const Operand o = operand(xb, "xb");
    need(table.shape[1] == width && stats.shape[0] >= rows && o.rows == rows && o.width == width, "embed_stream: shapes do not fit");
    if (prologue) {
        need(prologue->token_ids == token_ids && prologue->n == rows && prologue->capacity > 0 && prologue->table && prologue->updates,
             "embed_stream: the step's prologue is not for these rows");
        kernel_check(celeg_embed_stream_prologue(table.data, prologue->token_ids, out.as<float>(), xb.data, static_cast<int>(o.ld), o.k8,
                                                 stats.as<float>(), static_cast<int>(stats.stride[0]), static_cast<int>(rows),
                                                 static_cast<int>(width), static_cast<int>(table.shape[0]), prologue->table,
                                                 prologue->stride, prologue->n_slots, prologue->updates, prologue->capacity,
                                                 prologue->token_slot, prologue->last_tokens, stream), "embed_stream with the step's prologue");
        return;
    }
    kernel_check(celeg_embed_stream(table.data, token_ids, out.as<float>(), xb.data, static_cast<int>(o.ld), o.k8,
                                    stats.as<float>(), static_cast<int>(stats.stride[0]), static_cast<int>(rows),
                                    static_cast<int>(width), static_cast<int>(table.shape[0]), stream), "embed_stream");
}

void Ops::embed_stats(const Tensor& table, const int* token_ids, const Tensor& out, const Tensor& stats) {
    dev(table, "table", DType::BF16);
    dev(out, "out", DType::F32);
    dev(stats, "stats", DType::F32);
    const long long rows = out.shape[0], width = out.shape[1];
    need(table.shape[1] == width && stats.shape[0] >= rows, "embed_stats: shapes do not fit");
    kernel_check(celeg_embed_stats(table.data, token_ids, out.as<float>(), stats.as<float>(), static_cast<int>(stats.stride[0]),
                                   static_cast<int>(rows), static_cast<int>(width), static_cast<int>(table.shape[0]), stream),
                 "embed_stats");
}

// out = epilogue(prologue(a) w^T) for up to 64 rows, bfloat16 weights.
//
// a: bfloat16 rows [M, K], or, with norm_weight, the 32-bit residual stream, normalised on the
// fly (stats[row, :stat_blocks] holding partial sums of squares of its rows if stat_blocks > 0).
// rows picks rows of a.  Epilogues: Store (bfloat16 [M, N]), StoreF32, Residual (out is the
// stream, [M, N] 32-bit, added to in place; stats_out [>= M, residual_stat_blocks] receives
// partial sums of squares of the new rows, last_stat_blocks says how many a row), Swiglu (w is
// [2N, K]: gate rows then up rows), Conv (w is [3N, K]: B, C, x rows; one new token per request).
//
// Up to 16 bfloat16 rows go to the k-sliced kernels, and 9 to 64 rows with an inner size that
// is a multiple of 32 to the kernel that streams the weights.  Both also take the form behind a
// norm whose weight the caller has folded into w: a is then the bfloat16 copy of the stream and
// stats[row, :stat_blocks] its partial sums of squares, from which the rows' 1/rms (with eps)
// scales the sums; their Residual epilogue refreshes out_bf16, the bfloat16 copy of the stream,
// if given.  They also take w in the layout of fold_weight(packed).
void Ops::fused_linear(const Tensor& a, const Tensor& w, const Tensor& out, const FusedArgs& args) {
    dev(w, "w", DType::BF16);
    const Epilogue epi = args.epilogue;
    const int streams = epi == Epilogue::Swiglu ? 2 : epi == Epilogue::Conv ? 3 : 1;
    const bool packed = args.packed;
    need(!packed || (w.ndim == 3 && w.shape[2] == 32), "fused_linear: a packed weight is [K/32, rows, 32]");
    need(packed || w.ndim == 2, "fused_linear: w must be a matrix");
    const long long w_rows = packed ? w.shape[1] : w.shape[0], K = packed ? w.shape[0] * 32 : w.shape[1];
    need(w_rows % streams == 0, "fused_linear: weight rows do not split into the epilogue's streams");
    const long long N = w_rows / streams;
    dev(a, "a");
    const Operand ao = operand(a, "a");
    const int M = args.n_rows >= 0 ? args.n_rows : static_cast<int>(ao.rows);
    need(fused_linear_ok(M, {K}), "fused_linear: " + std::to_string(M) + " rows with inner size " + std::to_string(K) +
                                      " are not supported (1..64 rows, inner size a multiple of 8)");
    need(ao.width == K && (args.rows || ao.rows >= M), "fused_linear: a does not fit the weights");
    const bool norm = args.norm_weight.defined();
    if (norm) {
        need(a.dtype == DType::F32, "fused_linear: the normalising prologue reads a 32-bit stream");
        dev(args.norm_weight, "norm_weight", DType::F32);
        need(args.norm_weight.numel() == K, "fused_linear: norm weight must have the inner size");
        need(epi != Epilogue::Residual, "fused_linear: this combination is not built");
    } else {
        need(a.dtype == DType::BF16, "fused_linear: rows must be bfloat16 (or 32-bit with a norm weight)");
        if ((epi == Epilogue::Swiglu || epi == Epilogue::Conv || args.stat_blocks > 0) && !(M <= 16 && use_sliced) &&
            !rows_kernel_ok(M, {K}))
            throw KernelError("fused_linear: this combination is not built");
    }
    need(ao.ld % 8 == 0, "fused_linear: the row stride of a must be a multiple of 8");
    const DType out_dtype = (epi == Epilogue::StoreF32 || epi == Epilogue::Residual) ? DType::F32 : DType::BF16;
    dev(out, "out", out_dtype, false);
    const Operand oo = operand(out, "out");
    need(oo.rows >= M && oo.width == N, "fused_linear: out must be [" + std::to_string(M) + ", " + std::to_string(N) + "]");
    if (args.bias.defined()) {
        dev(args.bias, "bias", DType::F32);
        need(args.bias.numel() == streams * N, "fused_linear: bias does not fit");
    }
    GemvParams prm{};
    prm.a = a.data;
    prm.lda = static_cast<int>(ao.ld);
    prm.rows = args.rows;
    prm.norm_w = norm ? args.norm_weight.as<float>() : nullptr;
    prm.eps = args.eps;
    if (args.stat_blocks > 0) {
        dev(args.stats, "stats", DType::F32);
        need(args.stats.ndim == 2 && args.stats.shape[1] >= args.stat_blocks, "fused_linear: fewer partial sums than stat_blocks");
        prm.stats = args.stats.as<float>();
        prm.n_stat_blocks = args.stat_blocks;
        prm.stats_ld = static_cast<int>(args.stats.stride[0]);
    }
    prm.w = w.as<bf16>();
    prm.stream_rows = static_cast<int>(N);
    prm.bias = args.bias.defined() ? args.bias.as<float>() : nullptr;
    prm.M = M;
    prm.N = static_cast<int>(N);
    prm.K = static_cast<int>(K);
    prm.out = out.data;
    prm.ldo = static_cast<int>(oo.ld);
    const bool streamed = !norm && rows_kernel_ok(M, {K});
    const bool sliced = !norm && !streamed && M <= 16 && use_sliced;
    prm.a_k8_stride = ao.k8;
    prm.out_k8_stride = oo.k8;
    prm.w_q_stride = 8;
    if ((a.ndim == 3 || out.ndim == 3 || (args.out_bf16.defined() && args.out_bf16.ndim == 3)) && !streamed)
        throw KernelError("fused_linear: operands with the rows side by side go with the kernel for 9 to 64 rows");
    need(!(out.ndim == 3 && out_dtype != DType::BF16), "fused_linear: a 32-bit output has its rows one after the other");
    need(!packed || sliced || streamed || K % 32 == 0, "fused_linear: a packed weight has an inner size that is a multiple of 32");
    prm.w_row_stride = packed ? 32 : K;
    prm.w_kb_stride = packed ? w_rows * 32 : 32;
    if (args.out_bf16.defined()) {
        need((sliced || streamed) && epi == Epilogue::Residual,
             "fused_linear: out_bf16 goes with the residual epilogue of bfloat16 rows");
        dev(args.out_bf16, "out_bf16", DType::BF16, false);
        const Operand bo = operand(args.out_bf16, "out_bf16");
        need(bo.rows >= M && bo.width == N, "fused_linear: out_bf16 does not fit");
        prm.out_bf16 = args.out_bf16.data;
        prm.ld_bf16 = static_cast<int>(bo.ld);
        prm.bf16_k8_stride = bo.k8;
    }
    if (epi == Epilogue::Residual) {
        // partial sums of squares: one per workgroup and row
        last_stat_blocks = (sliced || streamed) ? residual_stat_blocks(M, static_cast<int>(N), static_cast<int>(K))
                                                : static_cast<int>((N + 15) / 16);
        if (args.stats_out.defined()) {
            dev(args.stats_out, "stats_out", DType::F32);
            need(args.stats_out.shape[1] >= last_stat_blocks && args.stats_out.shape[0] >= M,
                 "fused_linear: stats_out must be [>= rows, >= " + std::to_string(last_stat_blocks) + "]");
            prm.stats_out = args.stats_out.as<float>();
            prm.stats_ld_out = static_cast<int>(args.stats_out.stride[0]);
        }
    }
    if (epi == Epilogue::Conv) {
        need(args.conv != nullptr, "fused_linear: the convolution epilogue needs its operands");
        const ConvOperands& c = *args.conv;
        dev(c.taps, "conv taps", DType::F32);
        dev(c.state, "state", DType::F32, false);
        const long long L = c.taps.shape[1];
        need(L <= 8, "fused_linear: the convolution epilogue holds up to 8 taps, not " + std::to_string(L));
        need(c.taps.shape[0] == N && c.state.ndim == 3 && c.state.shape[1] == L && c.state.shape[2] == N &&
                 c.state.stride[1] == N && c.state.stride[2] == 1 && c.seq_slot,
             "fused_linear: convolution operands do not fit");
        prm.conv_w = c.taps.as<float>();
        prm.conv_b = c.bias.defined() ? c.bias.as<float>() : nullptr;
        prm.state = c.state.as<float>();
        prm.state_slot_stride = static_cast<size_t>(c.state.stride[0]);
        prm.seq_slot = c.seq_slot;
        prm.taps = static_cast<int>(L);
    }
    last_best_parts = 0;
    last_best_cols = 0;
    if (args.row_best) {
        need(epi == Epilogue::StoreF32, "fused_linear: row_best goes with the 32-bit store");
        last_best_parts = streamed ? celeg_gemm_rows_blocks(M, static_cast<int>(N), static_cast<int>(K), static_cast<int>(epi))
                          : sliced ? celeg_gemv_slices_blocks(M, static_cast<int>(N), static_cast<int>(K))
                                   : static_cast<int>((N + 15) / 16);
        need(args.row_best_ld >= last_best_parts && args.row_best_rows >= M,
             "fused_linear: row_best has room for " + std::to_string(args.row_best_rows) + " rows of " +
                 std::to_string(args.row_best_ld) + " parts, the kernel leaves " + std::to_string(M) + " of " + std::to_string(last_best_parts));
        last_best_cols = streamed ? celeg_gemm_rows_cols(M, static_cast<int>(N), static_cast<int>(K), static_cast<int>(epi))
                         : sliced ? celeg_gemv_slices_cols(M, static_cast<int>(N), static_cast<int>(K))
                                  : 16;
        prm.row_best = args.row_best;
        prm.row_best_ld = args.row_best_ld;
        prm.row_best_rows = args.row_best_rows;
    }
    took(sliced ? Path::FusedSliced : streamed ? Path::FusedRows : Path::FusedStaged);
    if (sliced) {
        kernel_check(celeg_gemv_slices(&prm, static_cast<int>(epi), stream), "fused_linear (k-sliced)");
    } else if (streamed) {
        kernel_check(celeg_gemm_rows(&prm, static_cast<int>(epi), stream), "fused_linear (9 to 64 rows)");
    } else {
        kernel_check(celeg_gemv_fused(&prm, norm ? 1 : 0, static_cast<int>(epi), fused_linear_shape, stream), "fused_linear");
    }
}

// ---------------------------------------------------------------------------- fused products of many rows
bool Ops::tiled_linear_ok(int rows, int n, std::initializer_list<long long> inner) const {
    if (!use_tiles || rows < tiles_min_rows || n % 4) return false;
    for (long long k : inner)
        if (k <= 0 || k % 64) return false;
    return true;
}

int Ops::tiled_stat_blocks(int rows, int n, int k) const { return celeg_gemm_tiles_blocks(rows, n, k); }

// out = epilogue(scale * (a w^T) + bias) for many bfloat16 rows (any number; made for more than
// 64), inner size a multiple of 64, columns a multiple of 4.  With stat_blocks > 0, a is the
// bfloat16 copy of the residual stream behind a norm whose weight the caller has folded into w,
// and stats[row, :stat_blocks] are partial sums of squares of its rows, from which the rows'
// 1/rms (with eps) scales the sums.  Epilogues: Store (bfloat16 [M, N]), Residual (out is the
// 32-bit stream, added to in place; out_bf16 receives its bfloat16 copy and stats_out the partial
// sums of squares of the new rows; last_stat_blocks says how many a row), Swiglu (w is [2N, K]).
bool Ops::tiled_qkv_ok(int head_dim, const Tensor* inv_freq, int rotary_dim, int pairing, const KVView& kv) const {
    if (!use_qkv_tail) return false;
    if (head_dim != 64 || kv.dtype != DType::BF16 || kv.head_dim != 64 || (kv.v_head_dim && kv.v_head_dim != 64)) return false;
    if (kv.page_tokens < 4 || (kv.page_tokens & (kv.page_tokens - 1))) return false;
    // the rotation: none, or of the whole head by split halves from the table of cosines and sines
    return !inv_freq || (rotary_dim == head_dim && pairing == 0 && use_rope_table);
}

void Ops::tiled_linear(const Tensor& a, const Tensor& w, const Tensor& out, Epilogue epi, float eps, const Tensor* stats,
                       int stat_blocks, const Tensor* bias, const Tensor* stats_out, const Tensor* out_bf16, const QkvTail* qkv) {
    need(epi == Epilogue::Store || epi == Epilogue::Residual || epi == Epilogue::Swiglu, "tiled_linear: unknown epilogue");
    need(!qkv || epi == Epilogue::Store, "tiled_linear: the q/k/v tail goes with the store epilogue");
    dev(a, "a", DType::BF16, false);
    dev(w, "w", DType::BF16);
    const int streams = epi == Epilogue::Swiglu ? 2 : 1;
    need(a.ndim == 2 && w.ndim == 2, "tiled_linear: a and w must be 2-D");
    const long long M = a.shape[0], K = a.shape[1];
    need(w.shape[1] == K && w.shape[0] % streams == 0, "tiled_linear: a and w do not fit");
    const long long N = w.shape[0] / streams;
    need(K % 64 == 0 && N % 4 == 0, "tiled_linear: inner size " + std::to_string(K) + " must be a multiple of 64 and " +
                                        std::to_string(N) + " columns a multiple of 4");
    const int lda = rows_of(a, "a");
    const DType out_dtype = epi == Epilogue::Residual ? DType::F32 : DType::BF16;
    dev(out, "out", out_dtype, false);
    const int ldo = rows_of(out, "out");
    need(out.shape[0] == M && out.shape[1] == N && lda % 8 == 0 && ldo % 4 == 0 &&
             reinterpret_cast<uintptr_t>(a.data) % 16 == 0 && reinterpret_cast<uintptr_t>(w.data) % 16 == 0 &&
             reinterpret_cast<uintptr_t>(out.data) % 16 == 0, "tiled_linear: out must be [M, N] and the rows aligned");
    TileParams prm{};
    prm.a = a.as<bf16>();
    prm.lda = lda;
    prm.w = w.as<bf16>();
    prm.ldw = static_cast<int>(K);
    prm.stream_rows = static_cast<int>(N);
    if (bias) {
        dev(*bias, "bias", DType::F32);
        need(bias->numel() == streams * N, "tiled_linear: bias does not fit");
        prm.bias = bias->as<float>();
    }
    if (stat_blocks > 0) {
        need(stats != nullptr, "tiled_linear: stats are missing");
        dev(*stats, "stats", DType::F32);
        need(stats->ndim == 2 && stats->shape[0] >= M && stats->shape[1] >= stat_blocks && stats->stride[1] == 1,
             "tiled_linear: stats must be [>= rows, >= stat_blocks]");
        prm.stats = stats->as<float>();
        prm.n_stat_blocks = stat_blocks;
        prm.stats_ld = static_cast<int>(stats->stride[0]);
    }
    prm.eps = eps;
    prm.M = static_cast<int>(M);
    prm.N = static_cast<int>(N);
    prm.K = static_cast<int>(K);
    prm.out = out.data;
    prm.ldo = ldo;
    if (epi == Epilogue::Residual) {
        last_stat_blocks = tiled_stat_blocks(static_cast<int>(M), static_cast<int>(N), static_cast<int>(K));
        if (out_bf16) {
            dev(*out_bf16, "out_bf16", DType::BF16, false);
            const int ldb = rows_of(*out_bf16, "out_bf16");
            need(out_bf16->shape[0] == M && out_bf16->shape[1] == N && ldb % 4 == 0 &&
                     reinterpret_cast<uintptr_t>(out_bf16->data) % 8 == 0, "tiled_linear: out_bf16 does not fit");
            prm.out_bf16 = out_bf16->as<bf16>();
            prm.ld_bf16 = ldb;
        }
        if (stats_out) {
            dev(*stats_out, "stats_out", DType::F32);
            need(stats_out->ndim == 2 && stats_out->shape[0] >= M && stats_out->shape[1] >= last_stat_blocks &&
                     stats_out->stride[1] == 1, "tiled_linear: stats_out must be [>= rows, >= " + std::to_string(last_stat_blocks) + "]");
            prm.stats_out = stats_out->as<float>();
            prm.stats_ld_out = static_cast<int>(stats_out->stride[0]);
        }
    } else {
        need(!out_bf16 && !stats_out, "tiled_linear: out_bf16 and stats_out go with the residual epilogue");
    }
    int kernel_epilogue = static_cast<int>(epi);
    if (qkv) {
        need(qkv->batch && qkv->kv, "tiled_linear: the q/k/v tail needs the step and the cache");
        const KVView& kv = *qkv->kv;
        need(tiled_qkv_ok(qkv->head_dim, qkv->inv_freq, qkv->head_dim, 0, kv), "tiled_linear: the q/k/v tail does not take these sizes");
        check_kv(kv, qkv->kv_heads, qkv->head_dim, DType::BF16);
        need(N == (static_cast<long long>(qkv->heads) + 2LL * qkv->kv_heads) * qkv->head_dim && M == qkv->batch->n_tokens,
             "tiled_linear: the q/k/v tail needs all heads of every row of the step");
        for (const Tensor* wt : {qkv->q_weight, qkv->k_weight})
            if (wt) {
                dev(*wt, "q/k norm weight", DType::F32);
                need(wt->numel() == qkv->head_dim, "tiled_linear: a norm weight must have head_dim entries");
            }
        prm.positions = qkv->batch->positions;
        prm.token_slot = qkv->batch->token_slot;
        prm.table = kv.table;
        prm.table_stride = kv.table_stride;
        prm.k_pool = static_cast<bf16*>(kv.k);
        prm.v_pool = static_cast<bf16*>(kv.v);
        prm.n_layers = kv.n_layers;
        prm.layer = kv.layer;
        prm.page_tokens = kv.page_tokens;
        prm.q_heads = qkv->heads;
        prm.kv_heads = qkv->kv_heads;
        prm.q_weight = qkv->q_weight ? qkv->q_weight->as<float>() : nullptr;
        prm.k_weight = qkv->k_weight ? qkv->k_weight->as<float>() : nullptr;
        prm.qk_eps = qkv->eps;
        if (qkv->inv_freq) {
            dev(*qkv->inv_freq, "inv_freq", DType::F32);
            need(qkv->inv_freq->numel() == qkv->head_dim / 2, "tiled_linear: the frequency table must have head_dim / 2 entries");
            prm.cos_sin = rope_table(*qkv->inv_freq, kv.table_stride * kv.page_tokens);
        }
        kernel_epilogue = 5;
    }
    took(qkv ? Path::TiledQkv : Path::Tiled);
    kernel_check(celeg_gemm_tiles(&prm, kernel_epilogue, stream), "tiled_linear");
}

std::shared_ptr<DeviceTensor> Ops::fold_weight(const Tensor& w, const Tensor* scale, bool packed) {
    dev(w, "w", DType::BF16);
    need(w.ndim == 2, "fold_weight: w must be a matrix");
    const long long rows = w.shape[0], K = w.shape[1];
    need(!packed || K % 32 == 0, "fold_weight: the inner size must be a multiple of 32");
    if (scale) {
        dev(*scale, "scale", DType::F32);
        need(scale->numel() == K, "fold_weight: the scale must have the inner size");
    }
    auto out = packed ? device_tensor(DType::BF16, {K / 32, rows, 32}) : device_tensor(DType::BF16, {rows, K});
    kernel_check(celeg_fold_weight(w.data, scale ? scale->as<float>() : nullptr, out->view.data, static_cast<int>(rows),
                                   static_cast<int>(K), packed ? 1 : 0, stream), "fold_weight");
    return out;
}

}  // namespace celeg
