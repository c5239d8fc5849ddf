#include "model.hpp"

#include <sys/stat.h>

#include <algorithm>
#include <chrono>
#include <cstdio>
#include <cstdlib>
#include <set>

namespace celeg {

// ---------------------------------------------------------------------------- the model
Model::Model(ModelSpec s) : spec(std::move(s)) {
    spec.validate();
    embedding_ = build_as<Embedding>("embedding", spec.embedding);
    for (const LayerSpec& layer : spec.layers) blocks_.push_back(build_block(layer));
    final_norm_ = build_as<Norm>("norm", spec.final_norm);
    head_ = build_as<Head>("head", spec.head);
    resolve_cache_sharing();
    graph_safe_ = true;
    std::function<void(const Part*)> visit = [&](const Part* p) {
        graph_safe_ = graph_safe_ && p->graph_safe();
        for (const Part* c : p->children()) visit(c);
    };
    for (const auto& np : named_parts()) visit(np.second);
}

void Model::resolve_cache_sharing() {
    const auto& order = spec.order;
    std::set<int> writes_somewhere;
    for (const RunStep& step : order)
        if (!step.kv_from) writes_somewhere.insert(step.layer);
    for (size_t i = 0; i < order.size(); ++i) {
        const RunStep& step = order[i];
        if (!step.kv_from) continue;
        const auto mine = mixer_of(step.layer).kv_need();
        const RunStep& source = order[static_cast<size_t>(*step.kv_from)];
        if (source.kv_from)
            throw SpecError("run order entry " + std::to_string(i) + " reads the cache of entry " +
                            std::to_string(*step.kv_from) + ", which has none of its own");
        const auto theirs = mixer_of(source.layer).kv_need();
        if (!mine || !theirs)
            throw SpecError("run order entry " + std::to_string(i) + ": only a mixer with keys and values can read " +
                            "another entry's cache, and only from such a mixer");
        if (mine->kv_heads != theirs->kv_heads || mine->head_dim != theirs->head_dim || mine->value_dim() != theirs->value_dim())
            throw SpecError("run order entry " + std::to_string(i) + ": its mixer and the one of entry " +
                            std::to_string(*step.kv_from) + " differ in kv_heads, head_dim or the width of the values");
    }
    for (int layer = 0; layer < static_cast<int>(blocks_.size()); ++layer) {
        bool used = false;
        for (const RunStep& s : order) used = used || s.layer == layer;
        if (used && !writes_somewhere.count(layer) && mixer_of(layer).kv_need()) mixer_of(layer).set_reads_foreign_kv();
    }
}

std::vector<std::pair<std::string, Part*>> Model::named_parts() {
    std::vector<std::pair<std::string, Part*>> out{{"embedding", embedding_.get()}};
    for (size_t i = 0; i < blocks_.size(); ++i)
        for (const auto& p : blocks_[i]->parts()) out.emplace_back("layers." + std::to_string(i) + "." + p.first, p.second);
    out.emplace_back("final_norm", final_norm_.get());
    out.emplace_back("head", head_.get());
    return out;
}

ExpectedTensors Model::expected_tensors() {
    ExpectedTensors expected;
    std::map<std::string, size_t> index;
    for (const auto& np : named_parts())
        for (const auto& ws : np.second->weight_specs()) {
            const std::string* name = np.second->spec.tensor(ws.first);
            if (!name)
                throw SpecError(np.first + " (" + np.second->spec.kind + ") wants a tensor for role '" + ws.first +
                                "', but the model description names none");
            auto it = index.find(*name);
            if (it != index.end()) {
                if (expected[it->second].second.shape != ws.second.shape)
                    throw SpecError("tensor " + *name + " is wanted with two different shapes");
                continue;
            }
            index[*name] = expected.size();
            expected.emplace_back(*name, ws.second);
        }
    return expected;
}

long long Model::weight_count() {
    long long total = 0;
    for (const auto& e : expected_tensors()) {
        long long n = 1;
        for (long long d : e.second.shape) n *= d;
        total += n;
    }
    return total;
}

CacheLayout Model::cache_layout() {
    CacheLayout layout;
    for (size_t i = 0; i < spec.order.size(); ++i) {
        const RunStep& step = spec.order[i];
        Mixer& mixer = mixer_of(step.layer);
        const auto need = mixer.kv_need();
        if (need) {
            if (step.kv_from) {
                const auto& src = layout.kv_of_step.at(*step.kv_from);
                layout.kv_of_step[static_cast<int>(i)] = CacheLayout::KvUse{src.group, src.layer, false};
            } else {
                int g = -1;
                for (size_t k = 0; k < layout.kv_groups.size(); ++k)
                    if (layout.kv_groups[k] == *need) g = static_cast<int>(k);
                if (g < 0) {
                    g = static_cast<int>(layout.kv_groups.size());
                    layout.kv_groups.push_back(*need);
                    layout.group_layers.push_back(0);
                }
                layout.kv_of_step[static_cast<int>(i)] = CacheLayout::KvUse{g, layout.group_layers[static_cast<size_t>(g)], true};
                ++layout.group_layers[static_cast<size_t>(g)];
            }
        }
        for (const StateNeed& s : mixer.state_needs()) layout.states.emplace_back(static_cast<int>(i), s);
    }
    return layout;
}

void Model::load(const WeightMap& tensors, Runtime& rt) {
    for (const auto& np : named_parts()) {
        PartTensors mine;
        for (const auto& ws : np.second->weight_specs()) {
            const std::string* name = np.second->spec.tensor(ws.first);
            auto it = name ? tensors.find(*name) : tensors.end();
            if (it == tensors.end()) throw SpecError("tensor for " + np.first + "." + ws.first + " was not loaded");
            mine[ws.first] = it->second;
        }
        np.second->load(mine, rt);
    }
}

void Model::bind_cache(const CacheManager& cache) {
    caches_.clear();
    for (size_t i = 0; i < spec.order.size(); ++i) caches_.push_back(cache.layer_cache(static_cast<int>(i)));
    bound_ = true;
}

Tensor Model::forward(const StepBatch& batch, Runtime& rt) {
    if (!bound_) throw StepError("model: bind_cache() has not been called");
    const long long T = batch.n_tokens, R = batch.n_logit_rows;
    const long long width = spec.hidden_size, vocab = head_->vocab();
    Tensor h = rt.ws.buf("hidden", DType::F32, {T, width});
    rt.stream_stat_blocks = 0;
    rt.stream_has_bf16 = false;
    rt.head_best = HeadBest{};
    if (!embedding_->takes_step_prologue()) rt.flush_prologue();
    embedding_->forward(batch.token_ids, h, rt, &batch);
    rt.flush_prologue();      // (an embedding that said it would and did not)
    rt.mark("embedding");
    Tensor delta;
    for (size_t i = 0; i < spec.order.size(); ++i) {
        delta = blocks_[static_cast<size_t>(spec.order[i].layer)]->forward(h, delta, batch, caches_[i], rt);
        if (rt.after_layer) rt.after_layer(static_cast<int>(i), h, delta.defined() ? &delta : nullptr);
    }
    Tensor logits = rt.ws.buf("logits", DType::F32, {R, vocab});
    if (R == 0) return logits;
    const Norm::Foldable* fold = final_norm_->foldable();
    if (!delta.defined() && fold && head_->forward_fused(h, *fold, batch, logits, rt, embedding_.get())) {
        rt.mark("head");
        return logits;
    }
    Tensor normed = rt.ws.buf("final_normed", rt.dtype, {R, width});
    final_norm_->forward(h, normed, rt, delta.defined() ? &delta : nullptr, batch.logit_rows);
    head_->forward(normed, logits, rt, embedding_.get());
    rt.mark("head");
    return logits;
}

// ---------------------------------------------------------------------------- the step function
ModelRunner::ModelRunner(Model& m, CacheManager& c, Runtime& r, int max_tokens)
    : model(m), cache(c), rt(r), max_batched_tokens(max_tokens) {
    model.bind_cache(cache);
    const int S = cache.max_requests;
    // room for the largest step, with as many table updates as rows plus requests
    update_room_ = max_batched_tokens / cache.page_tokens + 2 * S + 8;
    std::vector<PackedField> fields;
    const size_t ints = packed_layout(max_batched_tokens, S, max_batched_tokens,
                                      std::vector<int>(static_cast<size_t>(cache.n_groups()), update_room_), fields);
    builder_ = std::make_unique<BatchBuilder>(ints, cache.n_groups(), true, rt.stream);
    std::set<int> buckets;
    for (int i = 0; i < 12; ++i) buckets.insert(std::min(1 << i, S));
    buckets_.assign(buckets.begin(), buckets.end());
}

ModelRunner::~ModelRunner() { drop_graphs(); }

void ModelRunner::drop_graphs() {
    for (auto& g : graphs_) {
        if (g.second.exec) (void)hipGraphExecDestroy(g.second.exec);
        if (g.second.graph) (void)hipGraphDestroy(g.second.graph);
    }
    graphs_.clear();
    n_portion_graphs_ = 0;
}

void ModelRunner::set_token_source(int* last_tokens) {
    if (last_tokens != token_source_) drop_graphs();     // recorded steps do or do not hold the lookup
    token_source_ = last_tokens;
}

void ModelRunner::validate(const std::vector<StepEntry>& entries) const {
    if (entries.empty()) throw StepError("step: no entries");
    if (static_cast<int>(entries.size()) > cache.max_requests)
        throw StepError("step: " + std::to_string(entries.size()) + " requests exceed max_requests " +
                        std::to_string(cache.max_requests));
    std::set<int> seen;
    long long total = 0;
    const int vocab = model.spec.vocab_size;
    for (const StepEntry& e : entries) {
        const int n = static_cast<int>(e.tokens.size());
        if (n == 0) throw StepError("step: an entry has no tokens");
        if (!seen.insert(e.slot).second) throw StepError("step: slot " + std::to_string(e.slot) + " appears twice in one step");
        if (e.start_pos < 0 || e.start_pos + n > cache.max_context)
            throw StepError("context limit reached: position " + std::to_string(e.start_pos + n) + " exceeds " +
                            std::to_string(cache.max_context));
        bool in_range = true;
        if (n == 1 && e.tokens[0] == TOKEN_FROM_DEVICE) {
            in_range = token_source_ != nullptr;
        } else {
            for (int t : e.tokens) in_range = in_range && t >= 0 && t < vocab;
        }
        if (!in_range) throw StepError("step: token id out of range [0, " + std::to_string(vocab) + ")");
        for (int w : e.want)
            if (w < 0 || w >= n)
                throw StepError("wanted place " + std::to_string(w) + " is outside the entry's " + std::to_string(n) + " tokens");
        if (!cache.covers(e.slot, e.start_pos, n))
            throw StepError("step: the pages of slot " + std::to_string(e.slot) + " do not cover positions [" +
                            std::to_string(e.start_pos) + ", " + std::to_string(e.start_pos + n) + ")");
        total += n;
    }
    if (total > max_batched_tokens)
        throw StepError("step: " + std::to_string(total) + " tokens exceed max_batched_tokens " + std::to_string(max_batched_tokens));
}

// The block-table updates since the last step, per group.  A group with more of them than the
// step's metadata has room for (a large reservation made at once) has them shipped on their
// own, ahead of the step.
std::vector<std::vector<TableUpdate>> ModelRunner::drain_updates(const std::vector<int>& caps) {
    auto updates = cache.drain_table_updates();
    for (size_t g = 0; g < updates.size(); ++g)
        if (static_cast<int>(updates[g].size()) > caps[g]) {
            ship_table_updates(static_cast<int>(g), updates[g]);
            updates[g].clear();
        }
    return updates;
}

// builder.build; if it refuses the step, the drained updates go back to the cache manager, so
// that the device's block tables still get them with the next step.
StepBatch ModelRunner::build(const std::vector<StepEntry>& entries, std::vector<std::vector<TableUpdate>>& updates,
                             const BuildOptions& options) {
    try {
        return builder_->build(entries, updates, options);
    } catch (...) {
        cache.requeue_table_updates(updates);
        throw;
    }
}

void ModelRunner::ship_table_updates(int group, const std::vector<TableUpdate>& updates) {
    std::vector<int> flat{static_cast<int>(updates.size())};
    for (const TableUpdate& u : updates) {
        flat.push_back(u.slot);
        flat.push_back(u.logical);
        flat.push_back(u.page);
    }
    int* staged = static_cast<int*>(rt.ws.raw("table_update_burst", flat.size() * sizeof(int)));
    // (a synchronous copy: the host vector goes away)
    CELEG_HIP(hipMemcpyAsync(staged, flat.data(), flat.size() * sizeof(int), hipMemcpyHostToDevice, rt.stream));
    rt.ops.apply_table_updates(cache.device_table(group), cache.max_pages_per_request, cache.max_requests + 1, staged,
                               static_cast<int>(updates.size()));
    CELEG_HIP(hipStreamSynchronize(rt.stream));
}

// The block-table updates the step brings and the tokens it takes from the device: one launch
// where there is one cache group.
void ModelRunner::begin_step(const StepBatch& batch) {
    const auto& caps = batch.table_update_caps;
    if (caps.size() == 1 && caps[0] > 0) {
        StepPrologue& p = rt.prologue;
        p.table = cache.device_table(0);
        p.stride = cache.max_pages_per_request;
        p.n_slots = cache.max_requests + 1;
        p.updates = batch.table_updates[0];
        p.capacity = caps[0];
        p.token_ids = batch.token_ids;
        p.token_slot = batch.token_slot;
        p.last_tokens = token_source_;
        p.n = batch.n_tokens;
        p.pending = true;
        // left to the embedding's kernel (one kernel fewer a step), or run now
        if (!rt.defer_prologue || rt.phases) rt.flush_prologue();
        return;
    }
    for (size_t g = 0; g < caps.size(); ++g)
        if (caps[g] > 0)
            rt.ops.apply_table_updates(cache.device_table(static_cast<int>(g)), cache.max_pages_per_request,
                                       cache.max_requests + 1, batch.table_updates[g], caps[g]);
    if (token_source_) rt.ops.resolve_tokens(batch.token_ids, batch.token_slot, token_source_, batch.n_tokens);
}

Tensor ModelRunner::step(const std::vector<StepEntry>& entries) {
    validate(entries);
    if (graph_applies(entries)) return step_from_graph(entries);
    if (portion_graph_applies(entries)) return step_from_portion_graph(entries);
    auto updates = drain_updates(std::vector<int>(static_cast<size_t>(cache.n_groups()), update_room_));
    BuildOptions options;
    options.null_slot = cache.null_slot;
    StepBatch batch = build(entries, updates, options);
    if (rt.phases) rt.phases->begin();
    begin_step(batch);
    rt.mark("step metadata");
    last_batch_ = batch;
    Tensor logits = model.forward(batch, rt);
    if (rt.phases) rt.phases->end(batch.n_tokens);
    ++steps_run;
    return logits;
}

// A step in which every request brings one token and wants its logits is bound by its number
// of launches: it is recorded once per batch-size bucket as a HIP graph and replayed (the
// reference records its decode step likewise, src/backend/cuda/model/execution.cu:168-246).
// Rows that pad the batch to the bucket use the null slot and the spare page, so they touch no
// request's cache.  Recording and its warm-up run on such padding rows only: a request's state
// is never advanced twice.
bool ModelRunner::graph_applies(const std::vector<StepEntry>& entries) const {
    if (!use_graphs || !model.graph_safe() || rt.after_layer || rt.phases || sync_launches()) return false;
    if (static_cast<int>(entries.size()) > buckets_.back()) return false;
    for (const StepEntry& e : entries)
        if (e.tokens.size() != 1 || e.want.size() != 1 || e.want[0] != 0) return false;
    return true;
}

// A recorded step's launches are fixed, and the attention over few requests sizes its grid by
// the context: a graph is therefore good up to a bound on the context, and there is one per
// (batch-size bucket, bound).
int ModelRunner::context_bound(const std::vector<StepEntry>& entries) const {
    int longest = 0;
    for (const StepEntry& e : entries) longest = std::max(longest, e.start_pos + static_cast<int>(e.tokens.size()));
    for (int bound : {4096, 16384, 65536})
        if (longest <= bound) return std::min(bound, cache.max_context);
    return cache.max_context;
}

Tensor ModelRunner::step_from_graph(const std::vector<StepEntry>& entries) {
    const int S = static_cast<int>(entries.size());
    const int bucket = *std::lower_bound(buckets_.begin(), buckets_.end(), S);
    const int bound = context_bound(entries);
    const std::vector<int> caps(static_cast<size_t>(cache.n_groups()), bucket + 8);
    auto it = graphs_.find({bucket, bound});
    if (it == graphs_.end() || it->second.generation != rt.ws.generation) capture(bucket, caps, bound);
    Captured& captured = graphs_.at({bucket, bound});
    auto updates = drain_updates(caps);
    BuildOptions options;
    options.pad_to = bucket;
    options.null_slot = cache.null_slot;
    options.update_caps = &caps;
    last_batch_ = build(entries, updates, options);
    CELEG_HIP(hipGraphLaunch(captured.exec, rt.stream));
    rt.head_best = captured.head_best;
    ++steps_run;
    ++graph_replays;
    return captured.logits.rows(0, S);
}

ModelRunner::Captured& ModelRunner::capture(int bucket, const std::vector<int>& caps, int bound) {
    const std::vector<std::vector<TableUpdate>> empty(static_cast<size_t>(cache.n_groups()));
    BuildOptions options;
    options.pad_to = bucket;
    options.null_slot = cache.null_slot;
    options.update_caps = &caps;
    StepBatch batch = builder_->build({}, empty, options);
    batch.context_bound = bound;
    return record({bucket, bound}, batch);
}

// Runs `batch` once (buffers, libraries, weights re-laid at first need), then records it.  The
// batch holds rows of the null slot only, which write to the spare page and the spare state row.
ModelRunner::Captured& ModelRunner::record(std::pair<int, int> key, const StepBatch& batch) {
    const auto started = std::chrono::steady_clock::now();
    ++captures;
    auto old = graphs_.find(key);
    if (old != graphs_.end()) {
        if (old->second.exec) (void)hipGraphExecDestroy(old->second.exec);
        if (old->second.graph) (void)hipGraphDestroy(old->second.graph);
        graphs_.erase(old);
    }
    begin_step(batch);
    model.forward(batch, rt);
    CELEG_HIP(hipStreamSynchronize(rt.stream));
    Captured captured;
    rt.ws.frozen = true;
    hipError_t begun = hipStreamBeginCapture(rt.stream, hipStreamCaptureModeThreadLocal);
    if (begun != hipSuccess) {
        rt.ws.frozen = false;
        hip_check(begun, "hipStreamBeginCapture");
    }
    try {
        begin_step(batch);
        captured.logits = model.forward(batch, rt);
        captured.head_best = rt.head_best;
    } catch (...) {
        hipGraph_t broken = nullptr;
        (void)hipStreamEndCapture(rt.stream, &broken);
        if (broken) (void)hipGraphDestroy(broken);
        rt.ws.frozen = false;
        throw;
    }
    rt.ws.frozen = false;
    CELEG_HIP(hipStreamEndCapture(rt.stream, &captured.graph));
    CELEG_HIP(hipGraphInstantiate(&captured.exec, captured.graph, nullptr, nullptr, 0));
    CELEG_HIP(hipStreamSynchronize(rt.stream));
    captured.generation = rt.ws.generation;
    capture_seconds += std::chrono::duration<double>(std::chrono::steady_clock::now() - started).count();
    return graphs_[key] = captured;
}

// A step that is one portion of a prompt is some 150 launches with gaps between them: a size
// that has come before (the portions that a token budget cuts have the same size again and
// again) is recorded too, per number of rows and per context below or from 4,096 tokens (the
// attention over rows chooses its tiles by that).
bool ModelRunner::portion_graph_applies(const std::vector<StepEntry>& entries) {
    if (!use_graphs || !model.graph_safe() || rt.after_layer || rt.phases || sync_launches() || entries.size() != 1) return false;
    const StepEntry& e = entries[0];
    const int T = static_cast<int>(e.tokens.size());
    if (T < portion_graph_min_tokens || e.want.size() != 1 || e.want[0] != T - 1) return false;
    if (graphs_.count({-T, 0}) || graphs_.count({-T, 1})) return true;
    if (portion_sizes_seen_.size() >= 64 && !portion_sizes_seen_.count(T)) return false;     // sizes that never repeat
    return ++portion_sizes_seen_[T] >= 2 && n_portion_graphs_ < 16;
}

Tensor ModelRunner::step_from_portion_graph(const std::vector<StepEntry>& entries) {
    const StepEntry& e = entries[0];
    const int T = static_cast<int>(e.tokens.size());
    const bool far = e.start_pos + T >= 4096;
    const int bound = far ? cache.max_context : std::min(4095, cache.max_context);
    const std::vector<int> caps(static_cast<size_t>(cache.n_groups()), T / cache.page_tokens + 8);
    BuildOptions options;
    options.null_slot = cache.null_slot;
    options.update_caps = &caps;
    const std::pair<int, int> key{-T, far ? 1 : 0};
    auto it = graphs_.find(key);
    if (it == graphs_.end() || it->second.generation != rt.ws.generation) {
        if (it == graphs_.end()) ++n_portion_graphs_;
        const std::vector<std::vector<TableUpdate>> empty(static_cast<size_t>(cache.n_groups()));
        StepEntry spare;
        spare.slot = cache.null_slot;
        spare.start_pos = 0;
        spare.tokens.assign(static_cast<size_t>(T), 0);
        spare.want = {T - 1};
        StepBatch batch = builder_->build({spare}, empty, options);
        batch.context_bound = bound;
        record(key, batch);
    }
    Captured& captured = graphs_.at(key);
    auto updates = drain_updates(caps);
    last_batch_ = build(entries, updates, options);
    CELEG_HIP(hipGraphLaunch(captured.exec, rt.stream));
    rt.head_best = captured.head_best;
    ++steps_run;
    ++graph_replays;
    return captured.logits.rows(0, 1);
}

// ---------------------------------------------------------------------------- loading
LoadedModel::~LoadedModel() {
    if (stream) (void)hipStreamSynchronize(stream);
    if (rt && rt->phases) std::fputs(rt->phases->table().c_str(), stderr);
    runner.reset();
    cache.reset();
    model.reset();
    rt.reset();
    if (stream) (void)hipStreamDestroy(stream);
}

Described describe_model_folder(const std::string& model_dir) {
    const Json config = read_config_file(model_dir);
    Checkpoint ckpt(model_dir);
    const TensorShapes shapes = ckpt.shapes();
    return describe_config(config, &shapes);
}

void install_hidden_dump(Runtime& rt, const std::string& folder) {
    ::mkdir(folder.c_str(), 0777);
    auto step_number = std::make_shared<long long>(-1);
    auto last_layer = std::make_shared<int>(1 << 30);
    Runtime* r = &rt;
    rt.after_layer = [=](int layer, const Tensor& h, const Tensor* delta) {
        if (layer <= *last_layer) ++*step_number;      // a new step begins with entry 0
        *last_layer = layer;
        const size_t n = static_cast<size_t>(h.numel());
        std::vector<float> host(n);
        CELEG_HIP(hipMemcpyAsync(host.data(), h.data, n * 4, hipMemcpyDeviceToHost, r->stream));
        std::vector<float> add;
        if (delta) add = [&] {
            CELEG_HIP(hipStreamSynchronize(r->stream));
            return to_host_floats(*delta);
        }();
        CELEG_HIP(hipStreamSynchronize(r->stream));
        for (size_t i = 0; i < add.size() && i < n; ++i) host[i] += add[i];
        const std::string path = folder + "/step" + std::to_string(*step_number) + "_layer" + std::to_string(layer) + ".f32";
        if (FILE* f = std::fopen(path.c_str(), "wb")) {
            std::fwrite(host.data(), 4, n, f);
            std::fclose(f);
        }
    };
}

std::unique_ptr<LoadedModel> load_model(const std::string& model_dir, const LoadOptions& options) {
    if (options.gemm_backend != "library" && options.gemm_backend != "tiles" && options.gemm_backend != "auto")
        throw ConfigError("gemm_backend must be 'library', 'tiles' or 'auto', not '" + options.gemm_backend + "'");
    const DType dtype = parse_dtype(options.dtype);
    const Json raw = read_config_file(model_dir);
    Checkpoint ckpt(model_dir);
    const TensorShapes shapes = ckpt.shapes();
    Described described = describe_config(raw, &shapes);
    int max_context = options.max_context < 0 ? described.spec.max_context : options.max_context;
    if (max_context > described.spec.max_context)
        throw ConfigError("--context " + std::to_string(max_context) + " exceeds model maximum " +
                          std::to_string(described.spec.max_context));
    int count = 0;
    if (hipGetDeviceCount(&count) != hipSuccess || count <= 0) {
        (void)hipGetLastError();
        throw KernelError("celeg_amd needs a GPU: no HIP device is visible and there is no CPU path");
    }
    if (options.device < 0 || options.device >= count)
        throw KernelError("device " + std::to_string(options.device) + " does not exist (" + std::to_string(count) + " visible)");
    CELEG_HIP(hipSetDevice(options.device));
    auto lm = std::make_unique<LoadedModel>();
    lm->device = options.device;
    lm->config = described.config;
    CELEG_HIP(hipStreamCreate(&lm->stream));
    lm->rt = std::make_unique<Runtime>(dtype, lm->stream);
    // "auto" keeps the runtime's own rule, which goes by the sizes of the products
    if (options.gemm_backend == "tiles") lm->rt->tiled_max_width = 1LL << 40;
    if (options.gemm_backend == "library") lm->rt->tiled_max_width = 0;
    lm->model = std::make_unique<Model>(described.spec);
    {
        WeightMap tensors = load_tensors(ckpt, lm->model->expected_tensors(), dtype, options.strict_weights,
                                         &lm->unused_tensors);
        if (!lm->unused_tensors.empty()) {
            std::string names;
            for (size_t i = 0; i < lm->unused_tensors.size() && i < 8; ++i) names += (i ? ", " : "") + lm->unused_tensors[i];
            if (lm->unused_tensors.size() > 8) names += ", ...";
            std::fprintf(stderr, "[celeg_amd] warning: %zu tensor(s) of %s are not used by the model: %s\n",
                         lm->unused_tensors.size(), model_dir.c_str(), names.c_str());
        }
        lm->model->load(tensors, *lm->rt);
    }
    const int pages_per_request = (max_context + options.page_tokens - 1) / options.page_tokens;
    const int n_pages = options.n_pages < 0 ? pages_per_request * options.max_requests : options.n_pages;
    CacheLayout layout = lm->model->cache_layout();
    lm->cache = std::make_unique<CacheManager>(layout, options.page_tokens,
                                               std::vector<int>(std::max<size_t>(layout.kv_groups.size(), 1), n_pages),
                                               options.max_requests, max_context, dtype, true, lm->stream);
    lm->runner = std::make_unique<ModelRunner>(*lm->model, *lm->cache, *lm->rt, options.max_batched_tokens);
    lm->runner->use_graphs = options.use_graphs;
    if (const char* dump = std::getenv("CELEG_DUMP_HIDDEN"))
        if (*dump) install_hidden_dump(*lm->rt, dump);
    if (const char* timed = std::getenv("CELEG_PROFILE_PHASES"))
        if (*timed && std::string(timed) != "0") lm->rt->phases = std::make_unique<PhaseTimer>(lm->stream);
    CELEG_HIP(hipStreamSynchronize(lm->stream));
    return lm;
}

}  // namespace celeg
