// The registries of parts and block arrangements, and the parts this library brings:
// RMS norm, rotary and no position encoding, grouped-query attention over the paged cache,
// the double-gated short convolution, the SwiGLU feed-forward, token embedding, tied and own
// output head, and the pre-norm block; beside them the neutral parts ("none" mixer and
// feed-forward, "identity" norm, "hidden" head) with which a test runs a single part alone
// through the step function.
#include "parts.hpp"

#include <cmath>
#include <mutex>

#include "kernels.hpp"

namespace celeg {

// ---------------------------------------------------------------------------- registries
namespace {
struct Registries {
    std::map<std::string, std::map<std::string, PartFactory>> parts{
        {"norm", {}}, {"mixer", {}}, {"ffn", {}}, {"position", {}}, {"embedding", {}}, {"head", {}}};
    std::map<std::string, BlockFactory> blocks;
    std::mutex lock;
};
Registries& registries() {
    static Registries r;
    return r;
}
void register_builtin_parts();
void ensure_builtin() {
    static std::once_flag once;
    std::call_once(once, register_builtin_parts);
}
std::string names_of(const std::vector<std::string>& names) {
    std::string out = "[";
    for (size_t i = 0; i < names.size(); ++i) out += (i ? ", '" : "'") + names[i] + "'";
    return out + "]";
}
}  // namespace

void register_part(const std::string& role, const std::string& kind, PartFactory factory, bool replace) {
    ensure_builtin();
    Registries& r = registries();
    std::lock_guard<std::mutex> guard(r.lock);
    auto table = r.parts.find(role);
    if (table == r.parts.end()) {
        std::vector<std::string> roles;
        for (const auto& e : r.parts) roles.push_back(e.first);
        throw SpecError("unknown role '" + role + "'; roles: " + names_of(roles));
    }
    if (table->second.count(kind) && !replace) throw SpecError(role + " '" + kind + "' is already registered");
    table->second[kind] = std::move(factory);
}

void register_block(const std::string& arrangement, BlockFactory factory, bool replace) {
    ensure_builtin();
    Registries& r = registries();
    std::lock_guard<std::mutex> guard(r.lock);
    if (r.blocks.count(arrangement) && !replace) throw SpecError("block '" + arrangement + "' is already registered");
    r.blocks[arrangement] = std::move(factory);
}

std::vector<std::string> registered_parts(const std::string& role) {
    ensure_builtin();
    Registries& r = registries();
    std::lock_guard<std::mutex> guard(r.lock);
    std::vector<std::string> out;
    if (role == "block") {
        for (const auto& e : r.blocks) out.push_back(e.first);
    } else if (r.parts.count(role)) {
        for (const auto& e : r.parts[role]) out.push_back(e.first);
    }
    return out;
}

std::unique_ptr<Part> build_part(const std::string& role, const PartSpec& spec) {
    ensure_builtin();
    PartFactory factory;
    {
        Registries& r = registries();
        std::lock_guard<std::mutex> guard(r.lock);
        auto table = r.parts.find(role);
        if (table == r.parts.end()) throw SpecError("unknown role '" + role + "'");
        auto it = table->second.find(spec.kind);
        if (it != table->second.end()) factory = it->second;
    }
    if (!factory)
        throw SpecError("no " + role + " of kind '" + spec.kind + "' is registered; registered: " + names_of(registered_parts(role)));
    return factory(spec);
}

std::unique_ptr<Block> build_block(const LayerSpec& layer) {
    ensure_builtin();
    BlockFactory factory;
    {
        Registries& r = registries();
        std::lock_guard<std::mutex> guard(r.lock);
        auto it = r.blocks.find(layer.arrangement);
        if (it != r.blocks.end()) factory = it->second;
    }
    if (!factory)
        throw SpecError("no block arrangement '" + layer.arrangement + "' is registered; registered: " +
                        names_of(registered_parts("block")));
    return factory(layer);
}

namespace {

std::shared_ptr<DeviceTensor> get(const PartTensors& t, const std::string& role) {
    auto it = t.find(role);
    if (it == t.end()) throw SpecError("tensor for role '" + role + "' was not handed over");
    return it->second;
}
std::shared_ptr<DeviceTensor> maybe(const PartTensors& t, const std::string& role) {
    auto it = t.find(role);
    return it == t.end() ? nullptr : it->second;
}
WeightSpec matrix(long long rows, long long cols) { return WeightSpec{{rows, cols}, "matrix", "normal", {}}; }
WeightSpec vec(long long n, const char* init = "normal") { return WeightSpec{{n}, "vector", init, {}}; }

// ---------------------------------------------------------------------------- norms
// RMSNorm: y = x / sqrt(mean(x^2) + eps) * w, eps inside the root, w a plain scale
// (src/backend/cpu/kernels/elementwise.cpp:56-76; CUDA kernels/norm.cuh:1-44).  The sum of
// squares and the scaling are done in 32-bit whatever the activation dtype.
class RmsNorm final : public Norm {
public:
    explicit RmsNorm(const PartSpec& s) : Norm(s), width_(s.params.get_int("width", 0)), eps_(s.params.get_double("eps", 0.0)) {
        if (width_ <= 0 || !(eps_ > 0)) throw SpecError("rmsnorm: width and eps must be positive");
    }
    bool graph_safe() const override { return true; }
    WeightSpecs weight_specs() const override { return {{"weight", vec(width_, "around_one")}}; }
    void load(const PartTensors& t, Runtime&) override {
        weight_ = get(t, "weight");
        foldable_ = Foldable{weight_->view, static_cast<float>(eps_)};
    }
    void forward(const Tensor& x, const Tensor& out, Runtime& rt, const Tensor* delta, const int* rows) override {
        rt.ops.rmsnorm(x, weight_->view, static_cast<float>(eps_), out, delta, rows);
    }
    const Foldable* foldable() const override { return weight_ ? &foldable_ : nullptr; }

private:
    long long width_;
    double eps_;
    std::shared_ptr<DeviceTensor> weight_;
    Foldable foldable_;
};

// y = x (+ delta): no normalisation, no weight.  With it a test sees a part's rows as they are.
class IdentityNorm final : public Norm {
public:
    using Norm::Norm;
    void forward(const Tensor& x, const Tensor& out, Runtime& rt, const Tensor* delta, const int* rows) override {
        const long long n_rows = out.shape[0], width = out.shape[1];
        if (rows) {
            // listed rows: gather on the host side of the stream, row by row (a test path)
            std::vector<int> picked(static_cast<size_t>(n_rows));
            CELEG_HIP(hipMemcpyAsync(picked.data(), rows, picked.size() * sizeof(int), hipMemcpyDeviceToHost, rt.stream));
            CELEG_HIP(hipStreamSynchronize(rt.stream));
            Tensor sum = rt.ws.buf("identity_norm_sum", DType::F32, {1, width});
            for (long long r = 0; r < n_rows; ++r) {
                Tensor src = x.rows(picked[static_cast<size_t>(r)], 1);
                if (delta) {
                    rt.ops.cast(src, sum);
                    add(rt, sum, delta->rows(picked[static_cast<size_t>(r)], 1));
                    rt.ops.cast(sum, out.rows(r, 1));
                } else {
                    rt.ops.cast(src, out.rows(r, 1));
                }
            }
            return;
        }
        if (delta) add(rt, x, *delta);
        rt.ops.cast(x, out);
    }

private:
    // x += delta through the norm kernel's own addition (weight one, result discarded)
    static void add(Runtime& rt, const Tensor& x, const Tensor& delta) {
        const long long width = x.shape[1];
        Tensor ones = rt.ws.buf("identity_norm_ones", DType::F32, {width});
        std::vector<float> host(static_cast<size_t>(width), 1.0f);
        CELEG_HIP(hipMemcpyAsync(ones.data, host.data(), host.size() * 4, hipMemcpyHostToDevice, rt.stream));
        CELEG_HIP(hipStreamSynchronize(rt.stream));
        Tensor scratch = rt.ws.buf("identity_norm_scratch", DType::F32, {x.shape[0], width});
        rt.ops.rmsnorm(x, ones, 1e-6f, scratch, &delta, nullptr);
    }
};

// ---------------------------------------------------------------------------- position encodings
// rope: rotary encoding: for i < rotary_dim/2 pair i is rotated by the angle
// position * theta^(-2i/rotary_dim); the pair is (x[i], x[i + rotary_dim/2]) ("pairing":
// "halves", the default and the reference's, src/backend/cpu/kernels/rope.cpp:30-36, 95-108)
// or (x[2i], x[2i+1]) ("neighbours").  The frequencies are computed on the host
// in double (include/celeg/model/position.hpp:77-78) and handed to the kernel as a 32-bit
// table; the angle is the 32-bit product float(position) * frequency.
class Rope final : public PositionEncoding {
public:
    explicit Rope(const PartSpec& s) : PositionEncoding(s) {
        theta_ = s.params.get_double("theta", 0.0);
        head_dim_ = static_cast<int>(s.params.get_int("head_dim", 0));
        rotary_dim_ = static_cast<int>(s.params.get_int("rotary_dim", head_dim_));
        if (!(theta_ > 0)) throw SpecError("rope: theta must be positive");
        if (rotary_dim_ <= 0 || rotary_dim_ % 2 || rotary_dim_ > head_dim_)
            throw SpecError("rope: rotary_dim must be even, positive and at most head_dim");
        const std::string pairing = s.params.get_string("pairing", "halves");
        if (pairing != "halves" && pairing != "neighbours") throw SpecError("rope: pairing is 'halves' or 'neighbours', not '" + pairing + "'");
        pairing_ = pairing == "neighbours" ? 1 : 0;
    }
    bool graph_safe() const override { return true; }
    Tables tables(Runtime&) override {
        if (!table_) {
            std::vector<float> freq(static_cast<size_t>(rotary_dim_ / 2));
            for (int i = 0; i < rotary_dim_ / 2; ++i)
                freq[static_cast<size_t>(i)] = static_cast<float>(std::pow(theta_, -2.0 * i / rotary_dim_));
            table_ = from_host_floats(freq, DType::F32, {rotary_dim_ / 2});
        }
        return Tables{table_->view, rotary_dim_, pairing_};
    }

private:
    double theta_;
    int head_dim_, rotary_dim_, pairing_ = 0;
    std::shared_ptr<DeviceTensor> table_;
};

class NoPosition final : public PositionEncoding {
public:
    using PositionEncoding::PositionEncoding;
    bool graph_safe() const override { return true; }
    Tables tables(Runtime&) override { return Tables{}; }
};

// ---------------------------------------------------------------------------- attention
// Grouped-query attention over the paged cache.
//
// Order of work (src/backend/cpu/model_forward_token.cpp:100-120;
// src/backend/cuda/model/prefill_batched/attention/regular.cpp:23-131): q, k, v projections;
// RMSNorm of every q and k head over head_dim with one weight [head_dim] for all heads
// (src/backend/cpu/kernels/rope.cpp:84-94); position encoding of q and k; k and v of ALL rows
// of the step are written into the pages before any row attends
// (src/backend/cpu/model_forward_chunk.cpp:440-520); scores (q.k)/sqrt(head_dim) over the keys
// at positions <= the row's position (and inside the window, if there is one), softmax in
// 32-bit, weighted sum of values, output projection.  The scale is applied once
// (include/celeg/backend/cuda/attention_norm.hpp:13-23).
class GqaAttention final : public Mixer {
public:
    explicit GqaAttention(const PartSpec& s) : Mixer(s) {
        const Json& p = s.params;
        width_ = p.get_int("width", 0);
        heads_ = static_cast<int>(p.get_int("heads", 0));
        kv_heads_ = static_cast<int>(p.get_int("kv_heads", heads_));
        head_dim_ = static_cast<int>(p.get_int("head_dim", 0));
        qk_norm_ = p.get_bool("qk_norm", false);
        eps_ = static_cast<float>(p.get_double("eps", 1e-6));
        if (!p["window"].is_null()) {
            window_ = static_cast<int>(p["window"].as_int());
            if (*window_ <= 0) throw SpecError("gqa_attention: window must be positive");
        }
        if (width_ <= 0 || heads_ <= 0 || kv_heads_ <= 0 || heads_ % kv_heads_)
            throw SpecError("gqa_attention: heads must be a positive multiple of kv_heads");
        if (head_dim_ <= 0 || head_dim_ % 2) throw SpecError("gqa_attention: head_dim must be even");
        scale_ = p["scale"].is_null() ? static_cast<float>(1.0 / std::sqrt(static_cast<double>(head_dim_)))
                                      : static_cast<float>(p["scale"].as_double());
        PartSpec none;
        none.kind = "none";
        position_ = build_as<PositionEncoding>(
            "position", PartSpec::is_part(p["position"]) ? PartSpec::from_json(p["position"], "gqa_attention.position") : none);
    }
    bool graph_safe() const override { return true; }
    std::vector<const Part*> children() const override { return {position_.get()}; }
    void set_reads_foreign_kv() override { own_kv_ = false; }
    std::optional<KVNeed> kv_need() const override { return KVNeed{kv_heads_, head_dim_, window_}; }
    WeightSpecs weight_specs() const override {
        const long long qw = static_cast<long long>(heads_) * head_dim_, kvw = static_cast<long long>(kv_heads_) * head_dim_;
        WeightSpecs specs{{"q_proj", matrix(qw, width_)}, {"out_proj", matrix(width_, qw)}};
        if (own_kv_) {
            specs.push_back({"k_proj", matrix(kvw, width_)});
            specs.push_back({"v_proj", matrix(kvw, width_)});
        }
        if (qk_norm_) {
            specs.push_back({"q_norm", vec(head_dim_, "around_one")});
            if (own_kv_) specs.push_back({"k_norm", vec(head_dim_, "around_one")});
        }
        return specs;
    }
    void load(const PartTensors& t, Runtime&) override {
        // q, k and v projections run as one matrix product (the reference's fused_projections,
        // src/backend/cuda/execution_plan.cpp:113)
        if (own_kv_) {
            auto q = get(t, "q_proj"), k = get(t, "k_proj"), v = get(t, "v_proj");
            if (q->view.dtype != k->view.dtype || q->view.dtype != v->view.dtype)
                throw SpecError("gqa_attention: q, k and v projections are stored in different dtypes");
            w_qkv_ = concat_rows({q, k, v});
            w_q_ = std::make_shared<DeviceTensor>();
            w_q_->view = w_qkv_->view.rows(0, static_cast<long long>(heads_) * head_dim_);
        } else {
            w_q_ = get(t, "q_proj");
        }
        w_o_ = get(t, "out_proj");
        q_norm_ = maybe(t, "q_norm");
        k_norm_ = maybe(t, "k_norm");
    }
    Tensor forward(const Tensor& x, const StepBatch& batch, const LayerCache& cache, Runtime& rt) override {
        Tensor attended = project_and_attend(x, nullptr, batch, cache, rt);
        Tensor out = rt.ws.buf("mixer_out", rt.dtype, {x.shape[0], width_});
        rt.ops.linear(attended, w_o_->view, out, nullptr, rt.ws);
        return out;
    }
    // h += mixer(norm(h)) with the norm folded into the q/k/v product and the residual addition
    // into the output product
    bool forward_fused(const Tensor& h, const Norm::Foldable& norm, const StepBatch& batch, const LayerCache& cache,
                       Runtime& rt) override {
        const long long qw = static_cast<long long>(heads_) * head_dim_;
        const Tensor& w_in = cache.writes_kv ? w_qkv_->view : w_q_->view;
        if (!fused::fused_rows_ok(rt, batch, {width_, qw}) || w_in.dtype != rt.dtype || w_o_->view.dtype != rt.dtype)
            return false;
        Tensor attended = project_and_attend(h, &norm, batch, cache, rt);
        fused::linear_into_stream(rt, attended, w_o_->view, h);
        return true;
    }

private:
    // norm null: x are normalised rows; else x is the residual stream and the norm is applied
    // inside the product
    Tensor project_and_attend(const Tensor& x, const Norm::Foldable* norm, const StepBatch& batch, const LayerCache& cache,
                              Runtime& rt) {
        const long long T = x.shape[0];
        const long long qw = static_cast<long long>(heads_) * head_dim_, kvw = static_cast<long long>(kv_heads_) * head_dim_;
        const bool writes = cache.writes_kv;
        if (!cache.kv) throw SpecError("gqa_attention: the cache has no keys and values for this layer");
        if (writes && !own_kv_)
            throw SpecError("gqa_attention: built without key/value projections but asked to write a cache");
        auto project = [&](const std::shared_ptr<DeviceTensor>& w, const Tensor& out) {
            if (norm) fused::norm_linear(rt, x, *norm, w->view, out, Epilogue::Store);
            else rt.ops.linear(x, w->view, out, nullptr, rt.ws);
        };
        const PositionEncoding::Tables tables = position_->tables(rt);
        const Tensor* inv_freq = tables.inv_freq.defined() ? &tables.inv_freq : nullptr;
        Tensor q, k, v;
        bool finished = false;      // norm, rotation and cache write made by the product's own kernel
        if (writes) {
            Tensor qkv = rt.ws.buf("attn_qkv", rt.dtype, {T, qw + 2 * kvw});
            if (norm && fused::qkv_tail_ok(rt, static_cast<int>(T), width_) && T == batch.n_tokens &&
                rt.ops.tiled_qkv_ok(head_dim_, inv_freq, tables.rotary_dim, tables.pairing, *cache.kv)) {
                QkvTail tail;
                tail.heads = heads_;
                tail.kv_heads = kv_heads_;
                tail.head_dim = head_dim_;
                tail.q_weight = q_norm_ ? &q_norm_->view : nullptr;
                tail.k_weight = k_norm_ ? &k_norm_->view : nullptr;
                tail.eps = eps_;
                tail.inv_freq = inv_freq;
                tail.batch = &batch;
                tail.kv = &*cache.kv;
                fused::LinearExtras extras;
                extras.qkv = &tail;
                fused::norm_linear(rt, x, *norm, w_qkv_->view, qkv, Epilogue::Store, extras);
                finished = true;
            } else {
                project(w_qkv_, qkv);
            }
            q = qkv.cols(0, qw);
            k = qkv.cols(qw, kvw);
            v = qkv.cols(qw + kvw, kvw);
        } else {
            q = rt.ws.buf("attn_q", rt.dtype, {T, qw});
            project(w_q_, q);
        }
        Tensor attended = rt.ws.buf("attn_out", rt.dtype, {T, qw});
        // a decode-only step: the attention kernel prepares and writes the step's own keys and values
        if (!finished && writes && T == batch.n_tokens &&
            rt.ops.attention_fresh_ok(heads_, head_dim_, inv_freq, tables.rotary_dim, tables.pairing, batch, *cache.kv, rt.dtype)) {
            FreshKV fresh;
            fresh.k = &k;
            fresh.v = &v;
            fresh.q_weight = q_norm_ ? &q_norm_->view : nullptr;
            fresh.k_weight = k_norm_ ? &k_norm_->view : nullptr;
            fresh.eps = eps_;
            fresh.inv_freq = inv_freq;
            rt.ops.paged_attention(q, attended, heads_, kv_heads_, head_dim_, scale_, window_ ? *window_ : 0, batch, *cache.kv, rt.ws,
                                   &fresh);
            return attended;
        }
        if (!finished)
            rt.ops.qk_norm_rope_store(q, writes ? &k : nullptr, writes ? &v : nullptr, q_norm_ ? &q_norm_->view : nullptr,
                                      k_norm_ ? &k_norm_->view : nullptr, eps_, inv_freq,
                                      tables.rotary_dim, tables.pairing, heads_, kv_heads_, head_dim_, batch, *cache.kv);
        rt.ops.paged_attention(q, attended, heads_, kv_heads_, head_dim_, scale_, window_ ? *window_ : 0, batch, *cache.kv, rt.ws);
        return attended;
    }

    long long width_ = 0;
    int heads_ = 0, kv_heads_ = 0, head_dim_ = 0;
    bool qk_norm_ = false, own_kv_ = true;
    float eps_ = 1e-6f, scale_ = 1.f;
    std::optional<int> window_;
    std::unique_ptr<PositionEncoding> position_;
    std::shared_ptr<DeviceTensor> w_qkv_, w_q_, w_o_, q_norm_, k_norm_;
};

// ---------------------------------------------------------------------------- short convolution
// Double-gated short causal convolution.
//
// bcx = x W_in^T splits into B = [0,H), C = [H,2H), x = [2H,3H)
// (src/backend/cpu/kernels/convolution.cpp:16-18); bx = B*x;
// conv[t,ch] = sum_tap w[ch,tap] * bx[t-(L-1-tap), ch], zero before position 0, so the last tap
// multiplies the current token (convolution.cpp:19-26); y = C*conv; out = y W_out^T
// (src/backend/cpu/operators/recurrent.cpp:212-240).  A step continues from the request's saved
// state wherever the previous step stopped, as the reference's ragged kernel does
// (src/backend/cuda/kernels/shortconv.cuh:34-64).
//
// State per request: the last L values of bx, [L, H] in 32-bit, entry j holding position
// (tokens seen so far) - L + j; every row of a step reads the old state, then the state is
// replaced.
//
// With bias (the reference's ShortConvolutionSpec.bias is never true,
// include/celeg/model/graph.hpp:316-320): in_proj bias [3H] is added to bcx, the convolution
// bias [H] to conv before the C gate, out_proj bias [H] to the output.
class ShortConv final : public Mixer {
public:
    explicit ShortConv(const PartSpec& s) : Mixer(s) {
        width_ = s.params.get_int("width", 0);
        taps_ = s.params.get_int("taps", 0);
        bias_ = s.params.get_bool("bias", false);
        if (width_ <= 0 || taps_ <= 0) throw SpecError("short_conv: width and taps must be positive");
    }
    bool graph_safe() const override { return true; }
    std::vector<StateNeed> state_needs() const override { return {StateNeed{"bx", {taps_, width_}, DType::F32}}; }
    WeightSpecs weight_specs() const override {
        WeightSpec conv{{width_, 1, taps_}, "vector", "normal", {{width_, taps_}}};
        WeightSpecs specs{{"in_proj", matrix(3 * width_, width_)}, {"conv", conv}, {"out_proj", matrix(width_, width_)}};
        if (bias_) {
            specs.push_back({"in_proj_bias", vec(3 * width_)});
            specs.push_back({"conv_bias", vec(width_)});
            specs.push_back({"out_proj_bias", vec(width_)});
        }
        return specs;
    }
    void load(const PartTensors& t, Runtime&) override {
        w_in_ = get(t, "in_proj");
        w_out_ = get(t, "out_proj");
        w_conv_ = get(t, "conv");
        taps_view_ = Tensor::make(w_conv_->view.data, DType::F32, {width_, taps_});     // [H, 1, L] and [H, L] lie alike
        if (bias_) {
            b_in_ = get(t, "in_proj_bias");
            b_conv_ = get(t, "conv_bias");
            b_out_ = get(t, "out_proj_bias");
        }
    }
    Tensor forward(const Tensor& x, const StepBatch& batch, const LayerCache& cache, Runtime& rt) override {
        const long long T = x.shape[0];
        Tensor bcx = rt.ws.buf("conv_bcx", rt.dtype, {T, 3 * width_});
        rt.ops.linear(x, w_in_->view, bcx, b_in_ ? &b_in_->view : nullptr, rt.ws);
        Tensor y = rt.ws.buf("conv_y", rt.dtype, {T, width_});
        rt.ops.short_conv(bcx, taps_view_, b_conv_ ? &b_conv_->view : nullptr, cache.states.at("bx"), y, batch);
        Tensor out = rt.ws.buf("mixer_out", rt.dtype, {T, width_});
        rt.ops.linear(y, w_out_->view, out, b_out_ ? &b_out_->view : nullptr, rt.ws);
        return out;
    }
    // h += mixer(norm(h)) with the norm, the convolution (for one new token per request) and the
    // residual addition folded into the two products
    bool forward_fused(const Tensor& h, const Norm::Foldable& norm, const StepBatch& batch, const LayerCache& cache,
                       Runtime& rt) override {
        if (!fused::fused_rows_ok(rt, batch, {width_}) || w_in_->view.dtype != rt.dtype || w_out_->view.dtype != rt.dtype)
            return false;
        const int T = batch.n_tokens;
        fused::LinearExtras extras;
        if (b_in_) extras.bias = b_in_->view;
        Tensor y;
        if (batch.decode_only && batch.n_seqs == T && taps_ <= 8 && !fused::tiled_step(rt, T, width_)) {   // the fused form holds 8 taps
            y = fused::operand_rows(rt, "conv_y_fused", T, width_, {width_});
            ConvOperands conv;
            conv.taps = taps_view_;
            if (b_conv_) conv.bias = b_conv_->view;
            conv.state = cache.states.at("bx");
            conv.seq_slot = batch.seq_slot;
            extras.conv = &conv;
            fused::norm_linear(rt, h, norm, w_in_->view, y, Epilogue::Conv, extras);
        } else {
            y = rt.ws.buf("conv_y", rt.dtype, {T, width_});
            Tensor bcx = rt.ws.buf("conv_bcx", rt.dtype, {T, 3 * width_});
            fused::norm_linear(rt, h, norm, w_in_->view, bcx, Epilogue::Store, extras);
            rt.ops.short_conv(bcx, taps_view_, b_conv_ ? &b_conv_->view : nullptr, cache.states.at("bx"), y, batch);
        }
        fused::linear_into_stream(rt, y, w_out_->view, h, b_out_ ? &b_out_->view : nullptr);
        return true;
    }

private:
    long long width_ = 0, taps_ = 0;
    bool bias_ = false;
    std::shared_ptr<DeviceTensor> w_in_, w_conv_, w_out_, b_in_, b_conv_, b_out_;
    Tensor taps_view_;
};

// a mixer that adds nothing and keeps nothing
class NoMixer final : public Mixer {
public:
    explicit NoMixer(const PartSpec& s) : Mixer(s), width_(s.params.get_int("width", 0)) {}
    bool graph_safe() const override { return true; }
    Tensor forward(const Tensor& x, const StepBatch&, const LayerCache&, Runtime& rt) override { return zeros(rt, x.shape[0], width_ ? width_ : x.shape[1]); }
    static Tensor zeros(Runtime& rt, long long rows, long long width) {
        // (a fill kernel, not a memset: a recorded graph may hold it)
        const size_t words = (static_cast<size_t>(rows * width) * dtype_size(rt.dtype) + 3) / 4;
        void* p = rt.ws.raw("none_out", words * 4);
        kernel_check(celeg_zero_words(p, words, rt.stream), "zero fill");
        return Tensor::make(p, rt.dtype, {rows, width});
    }

private:
    long long width_;
};

// ---------------------------------------------------------------------------- feed-forward
// SwiGLU feed-forward: (silu(x W1^T) * (x W3^T)) W2^T, silu(g) = g / (1 + exp(-g))
// (src/backend/cpu/model_forward_token.cpp:163-172; kernels/elementwise.cpp:101-119).  Gate and
// up projections run as one matrix product on the concatenation [W1; W3] (rows [0,ff) gate,
// [ff,2ff) up), as the reference's w13 (src/backend/cuda/model/weight_setup.cpp:289-306).
class SwiGlu final : public FeedForward {
public:
    explicit SwiGlu(const PartSpec& s) : FeedForward(s), width_(s.params.get_int("width", 0)), ff_(s.params.get_int("ff", 0)) {
        if (width_ <= 0 || ff_ <= 0) throw SpecError("swiglu: width and ff must be positive");
    }
    bool graph_safe() const override { return true; }
    WeightSpecs weight_specs() const override {
        return {{"gate", matrix(ff_, width_)}, {"up", matrix(ff_, width_)}, {"down", matrix(width_, ff_)}};
    }
    void load(const PartTensors& t, Runtime&) override {
        auto gate = get(t, "gate"), up = get(t, "up");
        if (gate->view.dtype != up->view.dtype) throw SpecError("swiglu: gate and up projections are stored in different dtypes");
        w_gate_up_ = concat_rows({gate, up});
        w_down_ = get(t, "down");
    }
    Tensor forward(const Tensor& x, const StepBatch&, Runtime& rt) override {
        const long long T = x.shape[0];
        Tensor gate_up = rt.ws.buf("ffn_gate_up", rt.dtype, {T, 2 * ff_});
        rt.ops.linear(x, w_gate_up_->view, gate_up, nullptr, rt.ws);
        Tensor act = rt.ws.buf("ffn_act", rt.dtype, {T, ff_});
        rt.ops.swiglu(gate_up, act);
        Tensor out = rt.ws.buf("ffn_out", rt.dtype, {T, width_});
        rt.ops.linear(act, w_down_->view, out, nullptr, rt.ws);
        return out;
    }
    // h += ffn(norm(h)): the norm and the SwiGLU folded into the first product, the residual
    // addition into the second
    bool forward_fused(const Tensor& h, const Norm::Foldable& norm, const StepBatch& batch, Runtime& rt) override {
        if (!fused::fused_rows_ok(rt, batch, {width_, ff_}) || w_gate_up_->view.dtype != rt.dtype || w_down_->view.dtype != rt.dtype)
            return false;
        Tensor act = fused::operand_rows(rt, "ffn_act_fused", batch.n_tokens, ff_, {width_});
        fused::norm_linear(rt, h, norm, w_gate_up_->view, act, Epilogue::Swiglu);
        fused::linear_into_stream(rt, act, w_down_->view, h);
        return true;
    }

private:
    long long width_, ff_;
    std::shared_ptr<DeviceTensor> w_gate_up_, w_down_;
};

// a layer without a feed-forward (the reference's LayerSpec may hold none,
// src/model/inference/rules.cpp:44-46)
class NoFeedForward final : public FeedForward {
public:
    explicit NoFeedForward(const PartSpec& s) : FeedForward(s) {}
    bool graph_safe() const override { return true; }
    Tensor forward(const Tensor& x, const StepBatch&, Runtime& rt) override { return NoMixer::zeros(rt, x.shape[0], x.shape[1]); }
};

// ---------------------------------------------------------------------------- embedding and heads
// h0[t] = E[token[t]], nothing added and no scaling (src/backend/cpu/model_forward_token.cpp:28-60);
// logits = x E_out^T with E_out = E when the head is tied, else lm_head
// (src/backend/cpu/model_forward_token.cpp:213-218; src/model/inference/layer_bindings.cpp:24-95).
// Logits leave in 32-bit.
class TokenEmbedding final : public Embedding {
public:
    explicit TokenEmbedding(const PartSpec& s) : Embedding(s), vocab_(s.params.get_int("vocab", 0)), width_(s.params.get_int("width", 0)) {
        if (vocab_ <= 0 || width_ <= 0) throw SpecError("embedding: vocab and width must be positive");
    }
    bool graph_safe() const override { return true; }
    WeightSpecs weight_specs() const override { return {{"table", matrix(vocab_, width_)}}; }
    void load(const PartTensors& t, Runtime&) override { table_ = get(t, "table"); }
    Tensor table() const override { return table_->view; }
    bool takes_step_prologue() const override { return true; }
    void forward(const int* token_ids, const Tensor& out, Runtime& rt, const StepBatch* batch) override {
        const int rows = static_cast<int>(out.shape[0]);
        if (batch && table_->view.dtype == DType::BF16 && fused::fused_rows_ok(rt, *batch, {width_})) {
            // few rows: leave every row's sum of squares (and the bfloat16 copy of the stream)
            // for the first norm
            if (fused::sliced(rt, rows, width_) || fused::tiled_step(rt, rows, width_)) {
                // (the step's prologue rides along where it is for these rows)
                const bool along = rt.prologue.pending && rt.prologue.token_ids == token_ids && rt.prologue.n == rows;
                if (!along) rt.flush_prologue();
                rt.ops.embed_stream(table_->view, token_ids, out, fused::stream_bf16(rt, rows, width_),
                                    fused::stream_stats(rt, width_, rows), along ? &rt.prologue : nullptr);
                rt.prologue.pending = false;
                rt.stream_has_bf16 = true;
            } else {
                rt.flush_prologue();
                rt.ops.embed_stats(table_->view, token_ids, out, fused::stream_stats(rt, width_));
                rt.stream_has_bf16 = false;
            }
            rt.stream_stat_blocks = 1;
        } else {
            rt.flush_prologue();
            rt.ops.embed(table_->view, token_ids, out);
        }
    }

private:
    long long vocab_, width_;
    std::shared_ptr<DeviceTensor> table_;
};

// final norm and output product in one kernel for few wanted rows, 32-bit logits
bool head_fused(const Tensor& h, const Norm::Foldable& norm, const StepBatch& batch, const Tensor& out, Runtime& rt,
                const Tensor& weight) {
    const int R = batch.n_logit_rows;
    if (!(weight.defined() && weight.dtype == DType::BF16 && fused::fused_rows_ok(rt, batch, {h.shape[1]}) && R > 0 && R <= 64 &&
          !fused::tiled_step(rt, batch.n_tokens, h.shape[1])))
        return false;
    fused::LinearExtras extras;
    extras.rows = batch.logit_rows;
    extras.n_rows = R;
    // beside the logits: the best (logit, index) of every share of a row's columns, from which a
    // greedy row's token follows without the logits being read again
    const int room = Ops::head_best_parts(weight.shape[0]);
    if (rt.ops.use_head_argmax) {
        extras.row_best = static_cast<unsigned long long*>(rt.ws.raw("head_best", static_cast<size_t>(64) * room * sizeof(unsigned long long)));
        extras.row_best_ld = room;     // the parts of a row one after the other (R <= 64 rows)
        extras.row_best_rows = 64;
    }
    fused::norm_linear(rt, h, norm, weight, out, Epilogue::StoreF32, extras);
    if (extras.row_best && rt.ops.last_best_parts > 0) {
        rt.head_best.logits = out.data;
        rt.head_best.best = extras.row_best;
        rt.head_best.ld = extras.row_best_ld;
        rt.head_best.parts = rt.ops.last_best_parts;
        rt.head_best.cols = rt.ops.last_best_cols;
        rt.head_best.rows = R;
    }
    return true;
}

// uses the embedding table; wants no tensor of its own
class TiedHead final : public Head {
public:
    explicit TiedHead(const PartSpec& s) : Head(s), vocab_(static_cast<int>(s.params.get_int("vocab", 0))) {}
    bool graph_safe() const override { return true; }
    int vocab() const override { return vocab_; }
    void forward(const Tensor& x, const Tensor& out, Runtime& rt, const Embedding* embedding) override {
        rt.ops.linear(x, table_of(embedding), out, nullptr, rt.ws);
    }
    bool forward_fused(const Tensor& h, const Norm::Foldable& norm, const StepBatch& batch, const Tensor& out, Runtime& rt,
                       const Embedding* embedding) override {
        return head_fused(h, norm, batch, out, rt, table_of(embedding));
    }

private:
    static Tensor table_of(const Embedding* embedding) {
        const Tensor t = embedding ? embedding->table() : Tensor();
        if (!t.defined()) throw SpecError("tied_head: the model's embedding has no table to share");
        return t;
    }
    int vocab_;
};

class LinearHead final : public Head {
public:
    explicit LinearHead(const PartSpec& s)
        : Head(s), vocab_(static_cast<int>(s.params.get_int("vocab", 0))), width_(s.params.get_int("width", 0)) {}
    bool graph_safe() const override { return true; }
    int vocab() const override { return vocab_; }
    WeightSpecs weight_specs() const override { return {{"weight", matrix(vocab_, width_)}}; }
    void load(const PartTensors& t, Runtime&) override { weight_ = get(t, "weight"); }
    void forward(const Tensor& x, const Tensor& out, Runtime& rt, const Embedding*) override {
        rt.ops.linear(x, weight_->view, out, nullptr, rt.ws);
    }
    bool forward_fused(const Tensor& h, const Norm::Foldable& norm, const StepBatch& batch, const Tensor& out, Runtime& rt,
                       const Embedding*) override {
        return head_fused(h, norm, batch, out, rt, weight_->view);
    }

private:
    int vocab_;
    long long width_;
    std::shared_ptr<DeviceTensor> weight_;
};

// "logits" = the (normalised) hidden rows themselves, [rows, width] in 32-bit: what a test of a
// single part reads
class HiddenHead final : public Head {
public:
    explicit HiddenHead(const PartSpec& s) : Head(s), width_(static_cast<int>(s.params.get_int("width", 0))) {}
    bool graph_safe() const override { return true; }
    int vocab() const override { return width_; }
    void forward(const Tensor& x, const Tensor& out, Runtime& rt, const Embedding*) override { rt.ops.cast(x, out); }

private:
    int width_;
};

// ---------------------------------------------------------------------------- the block
// pre_norm: h += mixer(norm1(h)); h += ffn(norm2(h))
// (src/backend/cpu/model_forward_token.cpp:93-172).  The residual stream h is 32-bit in every
// mode and each sum into it is made in 32-bit; an addition is carried forward as delta and made
// by the next norm's kernel, which reads h anyway.
class PreNormBlock final : public Block {
public:
    explicit PreNormBlock(const LayerSpec& layer)
        : mixer_norm_(build_as<Norm>("norm", layer.mixer_norm)), mixer_(build_as<Mixer>("mixer", layer.mixer)),
          ffn_norm_(build_as<Norm>("norm", layer.ffn_norm)), ffn_(build_as<FeedForward>("ffn", layer.ffn)) {}
    std::vector<std::pair<std::string, Part*>> parts() override {
        return {{"mixer_norm", mixer_norm_.get()}, {"mixer", mixer_.get()}, {"ffn_norm", ffn_norm_.get()}, {"ffn", ffn_.get()}};
    }
    Mixer& mixer() override { return *mixer_; }
    Tensor forward(const Tensor& h, const Tensor& delta, const StepBatch& batch, const LayerCache& cache, Runtime& rt) override {
        const long long T = h.shape[0], width = h.shape[1];
        Tensor normed = rt.ws.buf("normed", rt.dtype, {T, width});
        // Few rows: parts that can, take the norm in front of them and the addition behind them
        // into their own products and write the stream themselves.
        const Norm::Foldable* fold1 = mixer_norm_->foldable();
        const Norm::Foldable* fold2 = ffn_norm_->foldable();
        const bool fusable = fold1 && fold2;
        Tensor mixed;
        if (fusable && !delta.defined() && mixer_->forward_fused(h, *fold1, batch, cache, rt)) {
            // the stream holds the mixer's sum already
        } else {
            rt.stream_stat_blocks = 0;
            mixer_norm_->forward(h, normed, rt, delta.defined() ? &delta : nullptr, nullptr);
            mixed = mixer_->forward(normed, batch, cache, rt);
        }
        rt.mark("mixer " + mixer_->spec.kind);
        if (fusable && !mixed.defined() && ffn_->forward_fused(h, *fold2, batch, rt)) {
            rt.mark("ffn " + ffn_->spec.kind);
            return Tensor();
        }
        rt.stream_stat_blocks = 0;
        ffn_norm_->forward(h, normed, rt, mixed.defined() ? &mixed : nullptr, nullptr);
        Tensor out = ffn_->forward(normed, batch, rt);
        rt.mark("ffn " + ffn_->spec.kind);
        return out;
    }

private:
    std::unique_ptr<Norm> mixer_norm_;
    std::unique_ptr<Mixer> mixer_;
    std::unique_ptr<Norm> ffn_norm_;
    std::unique_ptr<FeedForward> ffn_;
};

template <typename T>
PartFactory factory_of() {
    return [](const PartSpec& s) { return std::unique_ptr<Part>(new T(s)); };
}

void register_builtin_parts() {
    Registries& r = registries();
    std::lock_guard<std::mutex> guard(r.lock);
    r.parts["norm"]["rmsnorm"] = factory_of<RmsNorm>();
    r.parts["norm"]["identity"] = factory_of<IdentityNorm>();
    r.parts["position"]["rope"] = factory_of<Rope>();
    r.parts["position"]["none"] = factory_of<NoPosition>();
    r.parts["mixer"]["gqa_attention"] = factory_of<GqaAttention>();
    r.parts["mixer"]["short_conv"] = factory_of<ShortConv>();
    r.parts["mixer"]["none"] = factory_of<NoMixer>();
    r.parts["ffn"]["swiglu"] = factory_of<SwiGlu>();
    r.parts["ffn"]["none"] = factory_of<NoFeedForward>();
    r.parts["embedding"]["embedding"] = factory_of<TokenEmbedding>();
    r.parts["head"]["tied_head"] = factory_of<TiedHead>();
    r.parts["head"]["linear_head"] = factory_of<LinearHead>();
    r.parts["head"]["hidden"] = factory_of<HiddenHead>();
    r.blocks["pre_norm"] = [](const LayerSpec& layer) { return std::unique_ptr<Block>(new PreNormBlock(layer)); };
}

}  // namespace

}  // namespace celeg
