// The C interface (include/celeg_amd.h): option structs and their defaults, the engine, the step
// function alone, descriptions of folders, and the adapters through which parts and
// architectures defined outside this library take part in a model.
#include "../include/celeg_amd.h"

#include <cstring>
#include <mutex>
#include <set>
#include <algorithm>

#include "engine.hpp"
#include "model.hpp"

using namespace celeg;

// One request at a time, driven by prefill / decode calls.
struct ModelSession {
    int slot = -1;
    int position = 0;               // tokens fed so far
    bool ready = false;             // a prefill has succeeded: `logits` are those of its last token
    Tensor logits;                  // [1, width] on the device, the last step's
    std::unique_ptr<Sampler> sampler;
    GenerationConfig generation;
    double prefill_ms = 0.0, decode_ms = 0.0;
    unsigned long long prefill_tokens = 0, decode_tokens = 0;
};

struct celeg_model {
    std::unique_ptr<LoadedModel> owned;
    LoadedModel* lm = nullptr;
    PinnedBuffer logits_stage;      // few rows of logits come to the host through pinned memory
    std::unique_ptr<ModelSession> session;
    // (the session's sampler points into the model's runtime: it goes first)
    ~celeg_model() { session.reset(); }
};
struct celeg_engine {
    std::unique_ptr<Engine> engine;
    celeg_model view;
    std::string last_error;
};

namespace {
thread_local std::string g_error;
thread_local std::string g_text;

const char* text(std::string s) {
    g_text = std::move(s);
    return g_text.c_str();
}

template <typename F>
celeg_status guarded(F&& body, std::string* also = nullptr) {
    try {
        body();
        return CELEG_OK;
    } catch (const ConfigError& e) {
        g_error = e.what();
        if (also) *also = g_error;
        return CELEG_INVALID_ARGUMENT;
    } catch (const std::exception& e) {
        g_error = e.what();
        if (also) *also = g_error;
        return CELEG_ERROR;
    }
}

// fields of an option struct that the caller's (possibly older, shorter) struct does hold
template <typename T>
T options_from(const T* given, void (*init)(T*, size_t)) {
    T full;
    init(&full, sizeof(T));
    if (given) {
        const size_t n = given->struct_size ? std::min(given->struct_size, sizeof(T)) : sizeof(T);
        std::memcpy(&full, given, n);
        full.struct_size = sizeof(T);
    }
    return full;
}

LoadOptions load_options(const celeg_engine_options& o) {
    LoadOptions l;
    l.dtype = o.dtype ? o.dtype : "bfloat16";
    l.device = o.device;
    l.page_tokens = o.page_tokens;
    l.n_pages = o.logical_kv_pages > 0 ? o.logical_kv_pages : -1;
    l.max_requests = o.max_active_requests;
    l.max_context = o.context > 0 ? o.context : -1;
    l.max_batched_tokens = o.max_batched_tokens;
    l.gemm_backend = o.gemm_backend == CELEG_GEMM_TILES ? "tiles" : o.gemm_backend == CELEG_GEMM_LIBRARY ? "library" : "auto";
    l.use_graphs = o.use_graphs != 0;
    l.strict_weights = o.strict_weights != 0;
    return l;
}

GenerationConfig generation_of(const celeg_generation_options& g) {
    GenerationConfig c;
    c.temperature = g.temperature;
    c.top_k = g.top_k;
    c.top_p = g.top_p;
    c.repetition_penalty = g.repetition_penalty;
    c.seed = g.seed;
    if (g.n_forced_prefix < 0 || (g.n_forced_prefix > 0 && !g.forced_prefix))
        throw ConfigError("forced_prefix: a count without tokens (or a negative count)");
    if (g.n_forced_prefix > 0) c.forced_prefix.assign(g.forced_prefix, g.forced_prefix + g.n_forced_prefix);
    return c;
}

Json expected_json(const ExpectedTensors& expected) {
    Json out = Json::array();
    for (const auto& e : expected) {
        Json also = Json::array();
        for (const auto& s : e.second.also) also.push(Json::array_of(s));
        out.push(Json::object().set("name", e.first).set("shape", Json::array_of(e.second.shape))
                     .set("kind", e.second.kind).set("init", e.second.init).set("also", also));
    }
    return out;
}

Json describe_json(const Described& d) {
    Model model(d.spec);
    Json config = d.config;
    if (config.is_object()) config.erase("__spec__");
    return Json::object().set("config", config).set("spec", d.spec.to_json())
        .set("expected_tensors", expected_json(model.expected_tensors()))
        .set("cache_layout", model.cache_layout().to_json()).set("graph_safe", model.graph_safe());
}
}  // namespace

extern "C" {

// ---------------------------------------------------------------------------- options
void celeg_generation_options_init(celeg_generation_options* o, size_t struct_size) {
    if (!o) return;
    celeg_generation_options full{};
    full.struct_size = sizeof(full);
    full.temperature = 0.1f;
    full.top_k = 50;
    full.top_p = 1.0f;
    full.repetition_penalty = 1.05f;
    full.seed = 1;
    std::memcpy(o, &full, std::min(struct_size ? struct_size : sizeof(full), sizeof(full)));
    o->struct_size = std::min(struct_size ? struct_size : sizeof(full), sizeof(full));
}

void celeg_engine_options_init(celeg_engine_options* o, size_t struct_size) {
    if (!o) return;
    celeg_engine_options full{};
    full.struct_size = sizeof(full);
    full.dtype = "bfloat16";
    full.device = 0;
    full.max_active_requests = 8;
    full.max_batched_tokens = 2048;
    full.prefill_chunk_tokens = 1024;
    full.page_tokens = 16;
    full.logical_kv_pages = 0;
    full.scheduler_policy = CELEG_POLICY_MAX_UTILIZATION;
    full.context = 0;
    full.gemm_backend = CELEG_GEMM_AUTO;
    full.use_graphs = 1;
    full.run_ahead = 1;
    full.portion_granule = 1;
    full.strict_weights = 0;
    std::memcpy(o, &full, std::min(struct_size ? struct_size : sizeof(full), sizeof(full)));
    o->struct_size = std::min(struct_size ? struct_size : sizeof(full), sizeof(full));
}

void celeg_request_options_init(celeg_request_options* o, size_t struct_size) {
    if (!o) return;
    celeg_request_options full{};
    full.struct_size = sizeof(full);
    full.max_new_tokens = 128;
    full.eos_token_ids = nullptr;
    full.n_eos_token_ids = -1;
    full.priority = 0;
    celeg_generation_options_init(&full.generation, sizeof(full.generation));
    std::memcpy(o, &full, std::min(struct_size ? struct_size : sizeof(full), sizeof(full)));
    o->struct_size = std::min(struct_size ? struct_size : sizeof(full), sizeof(full));
}

const char* celeg_last_error(void) { return g_error.c_str(); }
void celeg_set_last_error_(const char* message) { g_error = message ? message : ""; }   // for host_api.cpp
const char* celeg_version(void) { return "celeg_amd 0.2 (gfx950)"; }

const char* celeg_backend_capabilities(void) {
    std::string out = "HIP backend for gfx950 (one GPU; bfloat16 and a true float32 path; paged keys and values, "
                      "state slots, portions beside decoding requests in one step; no CPU path): ";
    int count = 0;
    if (hipGetDeviceCount(&count) != hipSuccess || count <= 0) {
        (void)hipGetLastError();
        out += "no device is visible";
    } else {
        out += std::to_string(count) + (count == 1 ? " device" : " devices") + " visible";
        hipDeviceProp_t prop;
        if (hipGetDeviceProperties(&prop, 0) == hipSuccess)
            out += std::string(", device 0 is ") + prop.name + " (" + prop.gcnArchName + ")";
        else
            (void)hipGetLastError();
    }
    return text(out);
}

// ---------------------------------------------------------------------------- the engine
celeg_status celeg_engine_create(const char* model_dir, const celeg_engine_options* options, celeg_engine** out) {
    if (!model_dir || !out) {
        g_error = "celeg_engine_create: model_dir and out must not be null";
        return CELEG_INVALID_ARGUMENT;
    }
    *out = nullptr;
    return guarded([&] {
        const celeg_engine_options o = options_from(options, celeg_engine_options_init);
        EngineOptions eo;
        eo.load = load_options(o);
        eo.prefill_chunk_tokens = o.prefill_chunk_tokens;
        eo.policy = o.scheduler_policy == CELEG_POLICY_GUARANTEED_NO_EVICT ? "guaranteed_no_evict" : "max_utilization";
        eo.portion_granule = o.portion_granule;
        eo.run_ahead = o.run_ahead != 0;
        auto e = std::make_unique<celeg_engine>();
        e->engine = std::make_unique<Engine>(model_dir, eo);
        e->view.lm = &e->engine->loaded();
        *out = e.release();
    });
}

void celeg_engine_destroy(celeg_engine* engine) { delete engine; }

celeg_status celeg_engine_submit(celeg_engine* engine, const int32_t* tokens, int32_t n_tokens,
                                 const celeg_request_options* options, int64_t* request_id) {
    if (!engine || (!tokens && n_tokens > 0) || n_tokens < 0) {
        g_error = "celeg_engine_submit: engine and tokens must not be null";
        return CELEG_INVALID_ARGUMENT;
    }
    return guarded([&] {
        const celeg_request_options o = options_from(options, celeg_request_options_init);
        RequestOptions ro;
        ro.max_new_tokens = o.max_new_tokens;
        ro.priority = o.priority;
        if (o.n_eos_token_ids > 0 && !o.eos_token_ids) throw ConfigError("eos_token_ids: a count without tokens");
        if (o.n_eos_token_ids == 0) ro.eos_token_ids = std::vector<int>();
        if (o.n_eos_token_ids > 0) ro.eos_token_ids = std::vector<int>(o.eos_token_ids, o.eos_token_ids + o.n_eos_token_ids);
        ro.generation = generation_of(o.generation);
        const long long id = engine->engine->submit(std::vector<int>(tokens, tokens + n_tokens), ro);
        if (request_id) *request_id = id;
    }, &engine->last_error);
}

celeg_status celeg_engine_step(celeg_engine* engine, int32_t* tokens_fed) {
    if (!engine) return CELEG_INVALID_ARGUMENT;
    return guarded([&] {
        const int fed = engine->engine->step();
        if (tokens_fed) *tokens_fed = fed;
    }, &engine->last_error);
}

celeg_status celeg_engine_run(celeg_engine* engine) {
    if (!engine) return CELEG_INVALID_ARGUMENT;
    return guarded([&] { engine->engine->run(); }, &engine->last_error);
}

celeg_status celeg_engine_run_steps(celeg_engine* engine, int64_t limit, int64_t* steps) {
    if (!engine) return CELEG_INVALID_ARGUMENT;
    return guarded([&] {
        const long long done = engine->engine->run_steps(limit);
        if (steps) *steps = done;
    }, &engine->last_error);
}

celeg_status celeg_engine_has_work(celeg_engine* engine, int32_t* has_work) {
    if (!engine || !has_work) return CELEG_INVALID_ARGUMENT;
    *has_work = engine->engine->has_work() ? 1 : 0;
    return CELEG_OK;
}

static celeg_status with_request(celeg_engine* engine, const std::function<void()>& body) {
    if (!engine) return CELEG_INVALID_ARGUMENT;
    const celeg_status s = guarded(body, &engine->last_error);
    return s == CELEG_INVALID_ARGUMENT && g_error.rfind("unknown request id", 0) == 0 ? CELEG_NOT_FOUND : s;
}

celeg_status celeg_engine_poll(celeg_engine* engine, int64_t request_id, int32_t* tokens, int32_t capacity,
                               int32_t* n_tokens, int32_t* status) {
    return with_request(engine, [&] {
        Request& req = engine->engine->scheduler().request(request_id);
        int n = 0;
        while (n < capacity && tokens && !req.pending.empty()) {
            tokens[n++] = req.pending.front();
            req.pending.pop_front();
        }
        if (n_tokens) *n_tokens = n;
        if (status) *status = static_cast<int>(req.status);
    });
}

celeg_status celeg_engine_status(celeg_engine* engine, int64_t request_id, int32_t* status) {
    return with_request(engine, [&] {
        const RequestStatus s = engine->engine->status(request_id);
        if (status) *status = static_cast<int>(s);
    });
}

celeg_status celeg_engine_cancel(celeg_engine* engine, int64_t request_id) {
    return with_request(engine, [&] { engine->engine->cancel(request_id); });
}

celeg_status celeg_engine_release(celeg_engine* engine, int64_t request_id) {
    return with_request(engine, [&] {
        if (!engine->engine->release(request_id)) throw ConfigError("request " + std::to_string(request_id) + " has not ended: cancel it first");
    });
}

const char* celeg_engine_request_error(celeg_engine* engine, int64_t request_id) {
    if (!engine) return "";
    std::string message;
    guarded([&] { message = engine->engine->scheduler().request(request_id).error; });
    return text(message);
}

const char* celeg_engine_last_error(celeg_engine* engine) { return engine ? engine->last_error.c_str() : ""; }

const char* celeg_engine_metrics(celeg_engine* engine) {
    if (!engine) return text("{}");
    return text(engine->engine->metrics().dump());
}

const char* celeg_engine_request_metrics(celeg_engine* engine, int64_t request_id) {
    if (!engine) return nullptr;
    std::string out;
    if (guarded([&] { out = engine->engine->request_metrics(request_id).dump(); }, &engine->last_error) != CELEG_OK) return nullptr;
    return text(out);
}

celeg_status celeg_engine_last_logits(celeg_engine* engine, float* out, size_t capacity, int32_t* rows, int32_t* vocab) {
    if (!engine) return CELEG_INVALID_ARGUMENT;
    return guarded([&] {
        int r = 0, v = 0;
        const std::vector<float> host = engine->engine->last_logits(r, v);
        if (rows) *rows = r;
        if (vocab) *vocab = v;
        if (out) std::memcpy(out, host.data(), std::min(capacity, host.size()) * sizeof(float));
    }, &engine->last_error);
}

celeg_model* celeg_engine_model(celeg_engine* engine) { return engine ? &engine->view : nullptr; }

// ---------------------------------------------------------------------------- the step function alone
celeg_status celeg_model_create(const char* model_dir, const celeg_engine_options* options, celeg_model** out) {
    if (!model_dir || !out) {
        g_error = "celeg_model_create: model_dir and out must not be null";
        return CELEG_INVALID_ARGUMENT;
    }
    *out = nullptr;
    return guarded([&] {
        const celeg_engine_options o = options_from(options, celeg_engine_options_init);
        auto m = std::make_unique<celeg_model>();
        m->owned = load_model(model_dir, load_options(o));
        m->lm = m->owned.get();
        *out = m.release();
    });
}

void celeg_model_destroy(celeg_model* model) {
    if (model && model->owned) delete model;      // a view into an engine is the engine's
}

const char* celeg_model_describe(celeg_model* model) {
    if (!model) return nullptr;
    std::string out;
    if (guarded([&] {
            LoadedModel& lm = *model->lm;
            Json j = Json::object();
            j.set("config", lm.config).set("spec", lm.model->spec.to_json())
                .set("cache_layout", lm.cache->layout.to_json()).set("vocab_size", lm.model->spec.vocab_size)
                .set("logit_width", lm.model->logit_width()).set("max_context", lm.cache->max_context)
                .set("page_tokens", lm.cache->page_tokens).set("max_requests", lm.cache->max_requests)
                .set("max_batched_tokens", lm.runner->max_batched_tokens).set("graph_safe", lm.model->graph_safe())
                .set("dtype", dtype_name(lm.rt->dtype)).set("weights", lm.model->weight_count())
                .set("kv_bytes_per_token", lm.cache->layout.kv_bytes_per_token(dtype_size(lm.rt->dtype)))
                .set("eos_token_ids", Json::array_of(lm.model->spec.eos_token_ids))
                .set("gemm_backend", lm.model->spec.hidden_size <= lm.rt->tiled_max_width ? "tiles" : "library")
                .set("tiled_max_width", lm.rt->tiled_max_width)
                .set("unused_tensors", Json::array_of(lm.unused_tensors));
            out = j.dump();
        }) != CELEG_OK)
        return nullptr;
    return text(out);
}

celeg_status celeg_model_open_slot(celeg_model* model, int32_t* slot) {
    if (!model || !slot) return CELEG_INVALID_ARGUMENT;
    return guarded([&] { *slot = model->lm->cache->open(); });
}

celeg_status celeg_model_close_slot(celeg_model* model, int32_t slot) {
    if (!model) return CELEG_INVALID_ARGUMENT;
    return guarded([&] { model->lm->cache->close(slot); });
}

celeg_status celeg_model_prepare(celeg_model* model, int32_t slot, int32_t start, int32_t n, int32_t* ok) {
    if (!model) return CELEG_INVALID_ARGUMENT;
    return guarded([&] {
        const bool got = model->lm->cache->prepare(slot, start, n);
        if (ok) *ok = got ? 1 : 0;
    });
}

celeg_status celeg_model_check_cache(celeg_model* model) {
    if (!model) return CELEG_INVALID_ARGUMENT;
    return guarded([&] { model->lm->cache->check(); });
}

const char* celeg_model_cache_state(celeg_model* model) {
    if (!model) return nullptr;
    CacheManager& c = *model->lm->cache;
    Json held = Json::object();
    for (int slot : c.open_slots()) {
        Json groups = Json::array();
        for (const auto& g : c.pages_held(slot)) groups.push(Json::array_of(g));
        held.set(std::to_string(slot), groups);
    }
    return text(Json::object().set("free_slots", c.n_free_slots()).set("free_pages", Json::array_of(c.free_pages()))
                    .set("open_slots", Json::array_of(c.open_slots())).set("pages_held", held)
                    .set("memory", c.memory_bytes()).dump());
}

celeg_status celeg_model_step(celeg_model* model, int32_t n_entries, const int32_t* slot, const int32_t* start_pos,
                              const int32_t* n_tokens, const int32_t* tokens, const int32_t* n_want, const int32_t* want,
                              float* logits, size_t capacity) {
    if (!model || n_entries < 0 || (n_entries > 0 && (!slot || !start_pos || !n_tokens || !tokens || !n_want))) {
        g_error = "celeg_model_step: null argument";
        return CELEG_INVALID_ARGUMENT;
    }
    return guarded([&] {
        std::vector<StepEntry> entries(static_cast<size_t>(n_entries));
        size_t t = 0, w = 0, wanted = 0;
        for (int i = 0; i < n_entries; ++i) {
            StepEntry& e = entries[static_cast<size_t>(i)];
            e.slot = slot[i];
            e.start_pos = start_pos[i];
            if (n_tokens[i] < 0 || n_want[i] < 0 || (n_want[i] > 0 && !want)) throw StepError("step: negative count");
            e.tokens.assign(tokens + t, tokens + t + n_tokens[i]);
            e.want.assign(want + w, want + w + n_want[i]);
            t += static_cast<size_t>(n_tokens[i]);
            w += static_cast<size_t>(n_want[i]);
            wanted += static_cast<size_t>(n_want[i]);
        }
        LoadedModel& lm = *model->lm;
        // (checked before the step runs: a step that has run has advanced its requests)
        if (wanted && !logits) throw StepError("step: logits are wanted and there is no buffer for them");
        if (wanted * static_cast<size_t>(lm.model->logit_width()) > capacity) throw StepError("step: the logits buffer is too small");
        const Tensor out = lm.runner->step(entries);
        const size_t width = static_cast<size_t>(out.shape[1]);
        if (wanted * width > capacity) throw StepError("step: the logits buffer is too small");
        const size_t bytes = wanted * width * 4;
        if (wanted && bytes <= (size_t(8) << 20)) {
            // one asynchronous copy into pinned memory behind the step, one wait
            if (model->logits_stage.bytes() < bytes) model->logits_stage = PinnedBuffer(std::max(bytes, size_t(1) << 20));
            CELEG_HIP(hipMemcpy2DAsync(model->logits_stage.ptr(), width * 4, out.data, static_cast<size_t>(out.row_stride()) * 4,
                                       width * 4, wanted, hipMemcpyDeviceToHost, lm.stream));
            CELEG_HIP(hipStreamSynchronize(lm.stream));
            std::memcpy(logits, model->logits_stage.ptr(), bytes);
            return;
        }
        CELEG_HIP(hipStreamSynchronize(lm.stream));
        if (wanted)
            CELEG_HIP(hipMemcpy2D(logits, width * 4, out.data, static_cast<size_t>(out.row_stride()) * 4, width * 4, wanted,
                                  hipMemcpyDeviceToHost));
    });
}

// ---------------------------------------------------------------------------- one request at a time
static ModelSession& session_of(celeg_model* model) {
    if (!model->owned) throw ConfigError("the prefill / decode calls need a model of its own, not an engine's");
    if (!model->session) {
        auto s = std::make_unique<ModelSession>();
        LoadedModel& lm = *model->lm;
        s->sampler = std::make_unique<Sampler>(*lm.rt, lm.model->logit_width(), lm.cache->max_requests);
        model->session = std::move(s);
    }
    return *model->session;
}

celeg_status celeg_model_set_generation(celeg_model* model, const celeg_generation_options* options) {
    if (!model) return CELEG_INVALID_ARGUMENT;
    return guarded([&] {
        const celeg_generation_options o = options_from(options, celeg_generation_options_init);
        GenerationConfig c = generation_of(o);
        c.validate();
        session_of(model).generation = c;        // from the next prefill on
    });
}

celeg_status celeg_model_prefill(celeg_model* model, const int32_t* tokens, size_t count) {
    if (!model || !tokens || count == 0) {
        g_error = "celeg_model_prefill: model and tokens must not be null, and at least one token is needed";
        return CELEG_INVALID_ARGUMENT;
    }
    return guarded([&] {
        ModelSession& s = session_of(model);
        LoadedModel& lm = *model->lm;
        if (count > static_cast<size_t>(lm.cache->max_context)) throw ConfigError("prefill exceeds max_context");
        s.ready = false;
        if (s.slot >= 0) {                       // an earlier sequence: what it held goes back
            s.sampler->end(s.slot);
            lm.cache->close(s.slot);
            s.slot = -1;
        }
        s.slot = lm.cache->open();
        if (s.slot < 0) throw StepError("prefill: every slot of the cache is taken");
        s.position = 0;
        s.sampler->begin(s.slot, s.generation);
        const auto begun = std::chrono::steady_clock::now();
        const size_t portion = static_cast<size_t>(lm.runner->max_batched_tokens);
        for (size_t done = 0; done < count; done += portion) {
            const size_t n = std::min(portion, count - done);
            if (!lm.cache->prepare(s.slot, static_cast<int>(done), static_cast<int>(n)))
                throw StepError("prefill: the cache has too few pages for the prompt");
            StepEntry e;
            e.slot = s.slot;
            e.start_pos = static_cast<int>(done);
            e.tokens.assign(tokens + done, tokens + done + n);
            if (done + n == count) e.want = {static_cast<int>(n) - 1};
            s.logits = lm.runner->step({e});
            if (s.sampler->uses_seen()) s.sampler->mark_seen(lm.runner->last_batch());
            s.position = static_cast<int>(done + n);
        }
        CELEG_HIP(hipStreamSynchronize(lm.stream));
        s.prefill_ms = std::chrono::duration<double, std::milli>(std::chrono::steady_clock::now() - begun).count();
        s.prefill_tokens = count;
        s.decode_ms = 0.0;
        s.decode_tokens = 0;
        s.ready = true;
    });
}

celeg_status celeg_model_decode(celeg_model* model, int32_t* token) {
    if (!model || !token) return CELEG_INVALID_ARGUMENT;
    return guarded([&] {
        ModelSession& s = session_of(model);
        LoadedModel& lm = *model->lm;
        if (!s.ready) throw StepError("decode requires a successful prefill");
        if (s.position >= lm.cache->max_context) throw StepError("context limit reached");
        const auto begun = std::chrono::steady_clock::now();
        const int chosen = s.sampler->sample(s.logits, {s.slot}).at(0);
        s.ready = false;                         // until the token has been fed
        if (!lm.cache->prepare(s.slot, s.position, 1)) throw StepError("decode: the cache has no page left");
        StepEntry e;
        e.slot = s.slot;
        e.start_pos = s.position;
        e.tokens = {chosen};
        e.want = {0};
        s.logits = lm.runner->step({e});
        CELEG_HIP(hipStreamSynchronize(lm.stream));
        ++s.position;
        ++s.decode_tokens;
        s.decode_ms += std::chrono::duration<double, std::milli>(std::chrono::steady_clock::now() - begun).count();
        s.ready = true;
        *token = chosen;
    });
}

celeg_status celeg_model_copy_logits(celeg_model* model, float* output, size_t capacity, size_t* required) {
    if (!model || !required) return CELEG_INVALID_ARGUMENT;
    return guarded([&] {
        ModelSession& s = session_of(model);
        if (!s.ready) throw StepError("copy_logits requires a successful prefill");
        const size_t width = static_cast<size_t>(s.logits.shape[1]);
        *required = width;
        if (!output || capacity < width) throw StepError("logit output buffer is too small");
        CELEG_HIP(hipStreamSynchronize(model->lm->stream));
        CELEG_HIP(hipMemcpy(output, s.logits.data, width * sizeof(float), hipMemcpyDeviceToHost));
    });
}

celeg_status celeg_model_get_metrics(celeg_model* model, celeg_metrics* metrics) {
    if (!model || !metrics || metrics->struct_size < sizeof(*metrics)) return CELEG_INVALID_ARGUMENT;
    return guarded([&] {
        const ModelSession& s = session_of(model);
        metrics->prefill_ms = s.prefill_ms;
        metrics->prefill_tokens = s.prefill_tokens;
        metrics->decode_ms = s.decode_ms;
        metrics->decode_tokens = s.decode_tokens;
    });
}

}  // extern "C"

namespace {
struct Knob {
    const char* name;
    std::function<int(LoadedModel&)> get;
    std::function<void(LoadedModel&, int)> set;
};
const std::vector<Knob>& knobs() {
#define OPS_INT(field) {#field, [](LoadedModel& m) { return static_cast<int>(m.rt->ops.field); }, [](LoadedModel& m, int v) { m.rt->ops.field = v; }}
#define OPS_BOOL(field) {#field, [](LoadedModel& m) { return m.rt->ops.field ? 1 : 0; }, [](LoadedModel& m, int v) { m.rt->ops.field = v != 0; }}
    static const std::vector<Knob> table = {
        {"use_graphs", [](LoadedModel& m) { return m.runner->use_graphs ? 1 : 0; }, [](LoadedModel& m, int v) { m.runner->use_graphs = v != 0; }},
        {"portion_graph_min_tokens", [](LoadedModel& m) { return m.runner->portion_graph_min_tokens; },
         [](LoadedModel& m, int v) { m.runner->portion_graph_min_tokens = v; }},
        {"use_fused", [](LoadedModel& m) { return m.rt->use_fused ? 1 : 0; }, [](LoadedModel& m, int v) { m.rt->use_fused = v != 0; }},
        {"defer_prologue", [](LoadedModel& m) { return m.rt->defer_prologue ? 1 : 0; }, [](LoadedModel& m, int v) { m.rt->defer_prologue = v != 0; }},
        // (use_tiled_products: 1 = always, 0 = never; tiled_max_width is the rule itself)
        {"use_tiled_products", [](LoadedModel& m) { return m.model->spec.hidden_size <= m.rt->tiled_max_width ? 1 : 0; },
         [](LoadedModel& m, int v) { m.rt->tiled_max_width = v ? (1LL << 40) : 0; }},
        {"tiled_max_width", [](LoadedModel& m) { return static_cast<int>(std::min<long long>(m.rt->tiled_max_width, 1 << 30)); },
         [](LoadedModel& m, int v) { m.rt->tiled_max_width = v; }},
        {"fused_max_rows", [](LoadedModel& m) { return m.rt->fused_max_rows; }, [](LoadedModel& m, int v) { m.rt->fused_max_rows = v; }},
        OPS_INT(attention_decode_whole), OPS_BOOL(use_blaslt), OPS_INT(attention_rows_per_tile), OPS_INT(attention_rows_form),
        OPS_BOOL(attention_general), OPS_BOOL(use_rope_table), OPS_BOOL(use_argmax_parts), OPS_BOOL(use_head_argmax), OPS_BOOL(decode_parts_fill), OPS_BOOL(use_sliced),
        OPS_BOOL(use_rows_kernel), OPS_BOOL(use_tiles), OPS_BOOL(use_qkv_tail), OPS_BOOL(use_fresh_decode), OPS_INT(rows_kernel_min_rows), OPS_INT(tiles_min_rows),
        OPS_INT(fused_linear_shape),
        {"decode_parts_few", [](LoadedModel& m) { return m.rt->ops.decode_part_thresholds[0]; }, [](LoadedModel& m, int v) { m.rt->ops.decode_part_thresholds[0] = v; }},
        {"decode_parts_some", [](LoadedModel& m) { return m.rt->ops.decode_part_thresholds[1]; }, [](LoadedModel& m, int v) { m.rt->ops.decode_part_thresholds[1] = v; }},
    };
#undef OPS_INT
#undef OPS_BOOL
    return table;
}
}  // namespace

extern "C" {

celeg_status celeg_model_set_knob(celeg_model* model, const char* name, int32_t value) {
    if (!model || !name) return CELEG_INVALID_ARGUMENT;
    for (const Knob& k : knobs())
        if (std::strcmp(k.name, name) == 0) {
            k.set(*model->lm, value);
            return CELEG_OK;
        }
    g_error = std::string("unknown knob '") + name + "'";
    return CELEG_INVALID_ARGUMENT;
}

const char* celeg_model_knobs(celeg_model* model) {
    if (!model) return nullptr;
    Json out = Json::object();
    for (const Knob& k : knobs()) out.set(k.name, k.get(*model->lm));
    ModelRunner& r = *model->lm->runner;
    out.set("steps_run", r.steps_run).set("graph_replays", r.graph_replays).set("captures", r.captures);
    out.set("paths", model->lm->rt->ops.paths_json());
    return text(out.dump());
}

const char* celeg_model_phase_times(celeg_model* model) {
    if (!model) return nullptr;
    Runtime& rt = *model->lm->rt;
    return text(rt.phases ? rt.phases->report().dump() : std::string("null"));
}

celeg_status celeg_model_time_phases(celeg_model* model, int32_t on) {
    if (!model) return CELEG_INVALID_ARGUMENT;
    return guarded([&] {
        Runtime& rt = *model->lm->rt;
        if (on && !rt.phases) rt.phases = std::make_unique<PhaseTimer>(model->lm->stream);
        if (!on) rt.phases.reset();
    });
}

void* celeg_model_stream(celeg_model* model) { return model ? model->lm->stream : nullptr; }

celeg_status celeg_model_synchronize(celeg_model* model) {
    if (!model) return CELEG_INVALID_ARGUMENT;
    return guarded([&] { CELEG_HIP(hipStreamSynchronize(model->lm->stream)); });
}

// ---------------------------------------------------------------------------- descriptions
const char* celeg_describe_folder(const char* model_dir) {
    if (!model_dir) return nullptr;
    std::string out;
    if (guarded([&] {
            Json j = describe_json(describe_model_folder(model_dir));
            // how every tensor is stored, and how a bfloat16 and a 32-bit engine hold it
            Checkpoint ckpt(model_dir);
            Json held = Json::object();
            for (const Json& e : j["expected_tensors"].items()) {
                const std::string name = e["name"].as_string();
                bool there = false;
                for (const auto& n : ckpt.names()) there = there || n == name;
                if (!there) continue;
                const TensorInfo& info = ckpt.info(name);
                held.set(name, Json::object().set("stored", info.dtype)
                                   .set("bfloat16", dtype_name(stored_as(info, e["kind"].as_string(), DType::BF16)))
                                   .set("float32", dtype_name(stored_as(info, e["kind"].as_string(), DType::F32))));
            }
            j.set("held_as", held);
            // tensors that no part asks for (no error by themselves; loading warns about them)
            std::set<std::string> wanted;
            for (const Json& e : j["expected_tensors"].items()) wanted.insert(e["name"].as_string());
            std::vector<std::string> unused;
            for (const auto& n : ckpt.names())
                if (!wanted.count(n)) unused.push_back(n);
            std::sort(unused.begin(), unused.end());
            j.set("unused_tensors", Json::array_of(unused));
            out = j.dump();
        }) != CELEG_OK)
        return nullptr;
    return text(out);
}

const char* celeg_describe_config(const char* config_json, const char* shapes_json) {
    if (!config_json) return nullptr;
    std::string out;
    if (guarded([&] {
            Json config;
            try {
                config = Json::parse(config_json);
            } catch (const JsonError& e) {
                throw ConfigError(std::string("config.json cannot be read: ") + e.what());
            }
            TensorShapes shapes;
            bool have_shapes = false;
            if (shapes_json && std::strcmp(shapes_json, "null") != 0) {
                const Json s = Json::parse(shapes_json);
                have_shapes = s.is_object();
                if (have_shapes)
                    for (const auto& m : s.members()) {
                        std::vector<long long> dims;
                        for (const Json& d : m.second.items()) dims.push_back(d.as_int());
                        shapes[m.first] = dims;
                    }
            }
            out = describe_json(describe_config(config, have_shapes ? &shapes : nullptr)).dump();
        }) != CELEG_OK)
        return nullptr;
    return text(out);
}

celeg_status celeg_check_folder(const char* model_dir) { return celeg_check_folder_strict(model_dir, 0); }

celeg_status celeg_check_folder_strict(const char* model_dir, int32_t strict) {
    if (!model_dir) return CELEG_INVALID_ARGUMENT;
    return guarded([&] {
        const Described d = describe_model_folder(model_dir);
        Model model(d.spec);
        Checkpoint ckpt(model_dir);
        check_tensors(ckpt, model.expected_tensors(), strict != 0);
    });
}

const char* celeg_registered(const char* what) {
    if (!what) return nullptr;
    const std::string w = what;
    return text(Json::array_of(w == "architectures" ? registered_architectures() : registered_parts(w)).dump());
}

}  // extern "C"

// ---------------------------------------------------------------------------- parts from outside
namespace {

celeg_tensor_view view_of(const Tensor& t) {
    celeg_tensor_view v{};
    v.data = t.data;
    v.dtype = static_cast<int32_t>(t.dtype);
    v.ndim = t.ndim;
    for (int i = 0; i < 4; ++i) {
        v.shape[i] = t.shape[i];
        v.stride[i] = t.stride[i];
    }
    return v;
}

celeg_step_view view_of(const StepBatch& b) {
    celeg_step_view s{};
    s.n_tokens = b.n_tokens;
    s.n_seqs = b.n_seqs;
    s.n_logit_rows = b.n_logit_rows;
    s.decode_only = b.decode_only ? 1 : 0;
    s.single_rows = b.single_rows;
    s.token_ids = b.token_ids;
    s.positions = b.positions;
    s.token_seq = b.token_seq;
    s.token_slot = b.token_slot;
    s.cu_seqlens = b.cu_seqlens;
    s.seq_slot = b.seq_slot;
    s.seq_start = b.seq_start;
    s.logit_rows = b.logit_rows;
    s.host_seq_slot = b.host_seq_slot.data();
    s.host_seq_start = b.host_seq_start.data();
    s.host_cu_seqlens = b.host_cu_seqlens.data();
    return s;
}

// what a part's functions say of it, parsed once
struct OutsideDescription {
    WeightSpecs weights;
    std::optional<KVNeed> kv_need;
    std::vector<StateNeed> states;
    bool graph_safe = false;
    long long out_width = 0;
    std::vector<float> inv_freq;
    int rotary_dim = 0, pairing = 0;
};

class Outside {
public:
    Outside(const celeg_part_functions& f, const std::string& kind) : f_(f), kind_(kind) {
        if (!f_.describe || !f_.forward) throw SpecError("part '" + kind + "': describe and forward are required");
        const char* raw = f_.describe(f_.self);
        if (!raw) throw SpecError("part '" + kind + "': describe() returned nothing");
        const Json j = Json::parse(raw);
        if (j["weights"].is_object())
            for (const auto& m : j["weights"].members()) {
                WeightSpec ws;
                for (const Json& d : m.second["shape"].items()) ws.shape.push_back(d.as_int());
                ws.kind = m.second.get_string("kind", "matrix");
                ws.init = m.second.get_string("init", "normal");
                d_.weights.emplace_back(m.first, ws);
            }
        if (j["kv_need"].is_object()) {
            KVNeed need;
            need.kv_heads = static_cast<int>(j["kv_need"].get_int("kv_heads", 0));
            need.head_dim = static_cast<int>(j["kv_need"].get_int("head_dim", 0));
            need.v_head_dim = static_cast<int>(j["kv_need"].get_int("v_head_dim", 0));
            if (need.v_head_dim == need.head_dim) need.v_head_dim = 0;
            if (!j["kv_need"]["window"].is_null()) need.window = static_cast<int>(j["kv_need"]["window"].as_int());
            d_.kv_need = need;
        }
        if (j["states"].is_array())
            for (const Json& s : j["states"].items()) {
                StateNeed need;
                need.name = s.get_string("name", "state");
                for (const Json& d : s["shape"].items()) need.shape.push_back(d.as_int());
                const std::string dt = s.get_string("dtype", "float32");
                need.dtype = dt == "int32" ? DType::I32 : dt == "uint8" ? DType::U8 : parse_dtype(dt);
                d_.states.push_back(need);
            }
        d_.graph_safe = j.get_bool("graph_safe", false);
        d_.out_width = j.get_int("out_width", 0);
        if (j["inv_freq"].is_array())
            for (const Json& v : j["inv_freq"].items()) d_.inv_freq.push_back(static_cast<float>(v.as_double()));
        d_.rotary_dim = static_cast<int>(j.get_int("rotary_dim", 0));
        const std::string pairing = j.get_string("pairing", "halves");
        if (pairing != "halves" && pairing != "neighbours")
            throw SpecError("part '" + kind + "': pairing is 'halves' or 'neighbours', not '" + pairing + "'");
        d_.pairing = pairing == "neighbours" ? 1 : 0;
    }
    ~Outside() {
        if (f_.destroy) f_.destroy(f_.self);
    }
    Outside(const Outside&) = delete;
    const OutsideDescription& description() const { return d_; }
    void load(const PartTensors& tensors) {
        if (!f_.load) return;
        std::vector<const char*> roles;
        std::vector<celeg_tensor_view> views;
        for (const auto& t : tensors) {
            roles.push_back(t.first.c_str());
            views.push_back(view_of(t.second->view));
        }
        kept_ = tensors;     // the part works on these buffers for as long as it lives
        const int code = f_.load(f_.self, static_cast<int32_t>(roles.size()), roles.data(), views.data());
        if (code) throw SpecError("part '" + kind_ + "': load() failed with code " + std::to_string(code));
    }
    void forward(celeg_forward_args& args, Runtime& rt) {
        args.stream = rt.stream;
        args.dtype = static_cast<int32_t>(rt.dtype);
        const int code = f_.forward(f_.self, &args);
        if (code) throw KernelError("part '" + kind_ + "': forward() failed with code " + std::to_string(code));
    }

private:
    celeg_part_functions f_;
    std::string kind_;
    OutsideDescription d_;
    PartTensors kept_;
};

struct CacheViews {
    celeg_cache_view view{};
    std::vector<const char*> names;
    std::vector<celeg_tensor_view> states;
    explicit CacheViews(const LayerCache& cache) {
        if (cache.kv) {
            const KVView& kv = *cache.kv;
            view.has_kv = 1;
            view.writes_kv = cache.writes_kv ? 1 : 0;
            view.k = kv.k;
            view.v = kv.v;
            view.kv_dtype = static_cast<int32_t>(kv.dtype);
            view.layer = kv.layer;
            view.n_layers = kv.n_layers;
            view.page_tokens = kv.page_tokens;
            view.kv_heads = kv.kv_heads;
            view.head_dim = kv.head_dim;
            view.v_head_dim = kv.v_head_dim;
            view.n_pages = kv.n_pages;
            view.table_stride = kv.table_stride;
            view.table = kv.table;
        }
        for (const auto& s : cache.states) {
            names.push_back(s.first.c_str());
            states.push_back(view_of(s.second));
        }
        view.n_states = static_cast<int32_t>(names.size());
        view.state_names = names.data();
        view.states = states.data();
    }
};

class OutsideMixer final : public Mixer {
public:
    OutsideMixer(const PartSpec& s, const celeg_part_functions& f) : Mixer(s), part_(f, s.kind) {}
    bool graph_safe() const override { return part_.description().graph_safe; }
    WeightSpecs weight_specs() const override { return part_.description().weights; }
    std::optional<KVNeed> kv_need() const override { return part_.description().kv_need; }
    std::vector<StateNeed> state_needs() const override { return part_.description().states; }
    void load(const PartTensors& t, Runtime&) override { part_.load(t); }
    Tensor forward(const Tensor& x, const StepBatch& batch, const LayerCache& cache, Runtime& rt) override {
        const long long width = part_.description().out_width ? part_.description().out_width : x.shape[1];
        Tensor out = rt.ws.buf("outside_mixer_out", rt.dtype, {x.shape[0], width});
        CacheViews views(cache);
        celeg_forward_args args{};
        args.x = view_of(x);
        args.out = view_of(out);
        args.step = view_of(batch);
        args.cache = views.view;
        part_.forward(args, rt);
        return out;
    }

private:
    Outside part_;
};

class OutsideFeedForward final : public FeedForward {
public:
    OutsideFeedForward(const PartSpec& s, const celeg_part_functions& f) : FeedForward(s), part_(f, s.kind) {}
    bool graph_safe() const override { return part_.description().graph_safe; }
    WeightSpecs weight_specs() const override { return part_.description().weights; }
    void load(const PartTensors& t, Runtime&) override { part_.load(t); }
    Tensor forward(const Tensor& x, const StepBatch& batch, Runtime& rt) override {
        const long long width = part_.description().out_width ? part_.description().out_width : x.shape[1];
        Tensor out = rt.ws.buf("outside_ffn_out", rt.dtype, {x.shape[0], width});
        celeg_forward_args args{};
        args.x = view_of(x);
        args.out = view_of(out);
        args.step = view_of(batch);
        part_.forward(args, rt);
        return out;
    }

private:
    Outside part_;
};

class OutsideNorm final : public Norm {
public:
    OutsideNorm(const PartSpec& s, const celeg_part_functions& f) : Norm(s), part_(f, s.kind) {}
    bool graph_safe() const override { return part_.description().graph_safe; }
    WeightSpecs weight_specs() const override { return part_.description().weights; }
    void load(const PartTensors& t, Runtime&) override { part_.load(t); }
    void forward(const Tensor& x, const Tensor& out, Runtime& rt, const Tensor* delta, const int* rows) override {
        celeg_forward_args args{};
        args.x = view_of(x);
        args.out = view_of(out);
        if (delta) args.delta = view_of(*delta);
        args.rows = rows;
        part_.forward(args, rt);
    }

private:
    Outside part_;
};

class OutsidePosition final : public PositionEncoding {
public:
    OutsidePosition(const PartSpec& s, const celeg_part_functions& f) : PositionEncoding(s), part_(f, s.kind) {}
    bool graph_safe() const override { return true; }     // its tables are made once, on the host
    Tables tables(Runtime&) override {
        const OutsideDescription& d = part_.description();
        if (d.inv_freq.empty()) return Tables{};
        if (static_cast<int>(d.inv_freq.size()) * 2 != d.rotary_dim)
            throw SpecError("position '" + spec.kind + "': rotary_dim must be twice the number of frequencies");
        if (!table_) table_ = from_host_floats(d.inv_freq, DType::F32, {static_cast<long long>(d.inv_freq.size())});
        return Tables{table_->view, d.rotary_dim, d.pairing};
    }

private:
    Outside part_;
    std::shared_ptr<DeviceTensor> table_;
};

class OutsideEmbedding final : public Embedding {
public:
    OutsideEmbedding(const PartSpec& s, const celeg_part_functions& f) : Embedding(s), part_(f, s.kind) {}
    bool graph_safe() const override { return part_.description().graph_safe; }
    WeightSpecs weight_specs() const override { return part_.description().weights; }
    void load(const PartTensors& t, Runtime&) override { part_.load(t); }
    void forward(const int* token_ids, const Tensor& out, Runtime& rt, const StepBatch* batch) override {
        celeg_forward_args args{};
        args.out = view_of(out);
        args.token_ids = token_ids;
        if (batch) args.step = view_of(*batch);
        part_.forward(args, rt);
    }

private:
    Outside part_;
};

class OutsideHead final : public Head {
public:
    OutsideHead(const PartSpec& s, const celeg_part_functions& f) : Head(s), part_(f, s.kind) {}
    bool graph_safe() const override { return part_.description().graph_safe; }
    int vocab() const override { return static_cast<int>(part_.description().out_width); }
    WeightSpecs weight_specs() const override { return part_.description().weights; }
    void load(const PartTensors& t, Runtime&) override { part_.load(t); }
    void forward(const Tensor& x, const Tensor& out, Runtime& rt, const Embedding*) override {
        celeg_forward_args args{};
        args.x = view_of(x);
        args.out = view_of(out);
        part_.forward(args, rt);
    }

private:
    Outside part_;
};

}  // namespace

extern "C" {

celeg_status celeg_register_part(const char* role, const char* kind, celeg_part_factory factory, void* user) {
    if (!role || !kind || !factory) return CELEG_INVALID_ARGUMENT;
    return guarded([&] {
        const std::string r = role, k = kind;
        register_part(r, k, [r, k, factory, user](const PartSpec& spec) -> std::unique_ptr<Part> {
            celeg_part_functions f{};
            const int code = factory(spec.to_json().dump().c_str(), user, &f);
            if (code) throw SpecError(r + " '" + k + "': its factory failed with code " + std::to_string(code));
            if (r == "mixer") return std::make_unique<OutsideMixer>(spec, f);
            if (r == "ffn") return std::make_unique<OutsideFeedForward>(spec, f);
            if (r == "norm") return std::make_unique<OutsideNorm>(spec, f);
            if (r == "position") return std::make_unique<OutsidePosition>(spec, f);
            if (r == "embedding") return std::make_unique<OutsideEmbedding>(spec, f);
            if (r == "head") return std::make_unique<OutsideHead>(spec, f);
            throw SpecError("unknown role '" + r + "'");
        });
    });
}

celeg_status celeg_register_architecture(const char* name, celeg_architecture_describe describe, void* user) {
    if (!name || !describe) return CELEG_INVALID_ARGUMENT;
    return guarded([&] {
        Architecture arch;
        arch.name = name;
        const std::string n = name;
        // the outside function gives configuration and description in one call: the typed
        // configuration carries the description along to build_spec
        arch.read_config = [n, describe, user](const Json& config, const TensorShapes* shapes) {
            Json shape_json = Json();
            if (shapes) {
                shape_json = Json::object();
                for (const auto& s : *shapes) shape_json.set(s.first, Json::array_of(s.second));
            }
            const char* raw = describe(config.dump().c_str(), shape_json.dump().c_str(), user);
            if (!raw) throw ConfigError("architecture '" + n + "' refused the configuration");
            Json both;
            try {
                both = Json::parse(raw);
            } catch (const JsonError& e) {
                throw ConfigError("architecture '" + n + "' returned text that is not JSON: " + e.what());
            }
            if (both["error"].is_string()) throw ConfigError(both["error"].as_string());
            if (!both["spec"].is_object()) throw ConfigError("architecture '" + n + "' returned no \"spec\"");
            Json typed = both["config"].is_object() ? both["config"] : Json::object();
            typed.set("__spec__", both["spec"]);
            return typed;
        };
        arch.build_spec = [](const Json& typed) { return ModelSpec::from_json(typed["__spec__"]); };
        register_architecture(arch);
    });
}

}  // extern "C"
