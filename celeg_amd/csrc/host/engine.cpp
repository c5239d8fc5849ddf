#include "engine.hpp"

#include <algorithm>

namespace celeg {

Engine::Engine(const std::string& model_dir, const EngineOptions& options) {
    loaded_ = load_model(model_dir, options.load);
    SchedulerOptions so;
    so.max_active_requests = options.load.max_requests;
    so.max_batched_tokens = options.load.max_batched_tokens;
    so.prefill_chunk_tokens = options.prefill_chunk_tokens;
    so.policy = options.policy;
    so.portion_granule = options.portion_granule;
    scheduler_ = std::make_unique<Scheduler>(*loaded_->cache, so, loaded_->cache->max_context, loaded_->model->spec.eos_token_ids);
    sampler_ = std::make_unique<Sampler>(*loaded_->rt, loaded_->model->logit_width(), loaded_->cache->max_requests);
    run_ahead_ = options.run_ahead;
    if (run_ahead_) loaded_->runner->set_token_source(sampler_->last_tokens());
}

Engine::Engine(std::unique_ptr<LoadedModel> loaded, const SchedulerOptions& options, bool run_ahead)
    : loaded_(std::move(loaded)), run_ahead_(run_ahead) {
    if (options.max_batched_tokens > loaded_->runner->max_batched_tokens)
        throw ConfigError("max_batched_tokens exceeds what the step function was sized for");
    if (options.max_active_requests > loaded_->cache->max_requests)
        throw ConfigError("max_active_requests exceeds the cache manager's slots");
    scheduler_ = std::make_unique<Scheduler>(*loaded_->cache, options, loaded_->cache->max_context, loaded_->model->spec.eos_token_ids);
    sampler_ = std::make_unique<Sampler>(*loaded_->rt, loaded_->model->logit_width(), loaded_->cache->max_requests);
    if (run_ahead_) loaded_->runner->set_token_source(sampler_->last_tokens());
}

long long Engine::submit(const std::vector<int>& prompt, const RequestOptions& options) {
    const int vocab = loaded_->model->spec.vocab_size;
    for (int t : prompt)
        if (t < 0 || t >= vocab)
            throw ConfigError("token id " + std::to_string(t) + " out of range [0, " + std::to_string(vocab) + ")");
    for (int t : options.generation.forced_prefix)
        if (t < 0 || t >= vocab)
            throw ConfigError("forced_prefix: token id " + std::to_string(t) + " out of range [0, " + std::to_string(vocab) + ")");
    return scheduler_->submit(prompt, options);
}

RequestStatus Engine::poll(long long id, std::vector<int>& tokens, std::string& error) {
    Request& req = scheduler_->request(id);
    tokens.assign(req.pending.begin(), req.pending.end());
    req.pending.clear();
    error = req.error;
    return req.status;
}

void Engine::sync_slots() {
    std::vector<int> released;
    std::vector<std::pair<int, Request*>> bound;
    scheduler_->drain_slot_events(released, bound);
    for (int slot : released) sampler_->end(slot);
    for (const auto& b : bound) {
        Request& req = *b.second;
        if (!req.rng) req.rng = std::make_shared<XorShift64Star>(req.options.generation.seed);
        sampler_->begin(b.first, req.options.generation, req.rng, req.generated.size());
    }
}

void Engine::contain(const std::vector<PlannedEntry>& plan, const std::string& message) {
    ++failed_steps_;
    scheduler_->fail(plan, message);
    sync_slots();
}

int Engine::step() {
    std::vector<PlannedEntry> plan = scheduler_->plan();
    sync_slots();
    if (plan.empty()) return 0;
    Launched launched;
    if (!launch(plan, false, launched)) return 0;
    return complete(launched);
}

// A step in two halves, so that run() can launch the next step before it reads this one's tokens.
bool Engine::launch(const std::vector<PlannedEntry>& plan, bool device_tokens, Launched& out) {
    out.start = std::chrono::steady_clock::now();
    out.plan = plan;
    try {
        std::vector<StepEntry> entries;
        std::vector<int> slots;
        for (const PlannedEntry& e : plan) {
            StepEntry se;
            se.slot = e.request->slot;
            se.start_pos = e.start;
            se.tokens = device_tokens ? std::vector<int>{TOKEN_FROM_DEVICE} : e.request->tokens(e.start, e.count);
            if (e.samples) {
                se.want = {e.count - 1};
                slots.push_back(e.request->slot);
            }
            entries.push_back(std::move(se));
        }
        Tensor logits = loaded_->runner->step(entries);
        last_logits_ = logits;
        steps_ahead_ += device_tokens ? 1 : 0;
        // what kind of step it was: single tokens only, portions only, or both side by side
        bool singles = false, portions = false;
        for (const PlannedEntry& e : plan) (e.count == 1 ? singles : portions) = true;
        (singles && portions ? mixed_steps_ : singles ? decode_steps_ : portion_steps_) += 1;
        // tokens that count as seen by their request: the sampler's kernels mark what they choose,
        // so a step that only feeds such tokens back (every entry the one new token of a
        // decoding request) has nothing to mark; prompts, and what a request that was put back
        // feeds again, are marked here
        bool feeds_prompt = false;
        for (const PlannedEntry& e : plan)
            feeds_prompt = feeds_prompt || e.count != 1 || e.request->status != RequestStatus::Decoding;
        if (feeds_prompt && sampler_->uses_seen()) sampler_->mark_seen(loaded_->runner->last_batch());
        if (!slots.empty()) sampler_->launch(logits, slots);
        out.sampled_rows = !slots.empty();
        return true;
    } catch (const std::exception& e) {
        contain(plan, e.what());
        return false;
    }
}

int Engine::complete(Launched& launched) {
    try {
        std::vector<int> sampled = launched.sampled_rows ? sampler_->fetch() : std::vector<int>();
        // a request that ended while this step was already under way: its row is dropped
        size_t next = 0;
        std::vector<PlannedEntry> entries;
        std::vector<int> tokens;
        int fed = 0;
        for (const PlannedEntry& e : launched.plan) {
            const int token = e.samples ? sampled.at(next++) : -1;
            if (is_done(e.request->status)) continue;
            entries.push_back(e);
            fed += e.count;
            if (e.samples) tokens.push_back(token);
        }
        scheduler_->accept(entries, tokens);
        sync_slots();
        ++steps_;
        step_seconds_ += std::chrono::duration<double>(std::chrono::steady_clock::now() - launched.start).count();
        return fed;
    } catch (const std::exception& e) {
        contain(launched.plan, e.what());
        return 0;
    }
}

// The step after `plan`, decided before plan's tokens are known: possible when every active
// request is decoding (nothing waits, nothing is being prefilled), for the requests that this
// step's token cannot end by count or context.  A request that the token does end (an end token)
// rides along for one row that is dropped afterwards; what it writes lies in its own pages and
// state, which are only handed on by later steps on the same stream.
bool Engine::plan_ahead(const std::vector<PlannedEntry>& plan, std::vector<PlannedEntry>& ahead) {
    ahead.clear();
    Scheduler& sched = *scheduler_;
    if (!run_ahead_ || !loaded_->runner->token_source() || !sched.queue().empty() || plan.size() != sched.active().size())
        return false;
    for (const PlannedEntry& e : plan) {
        const Request& req = *e.request;
        if (e.count != 1 || !e.samples || req.status != RequestStatus::Decoding || req.cancel_requested) return false;
        if (static_cast<int>(req.generated.size()) + 1 >= req.options.max_new_tokens || e.start + 2 >= sched.max_context) continue;
        ahead.push_back(PlannedEntry{e.request, e.start + 1, 1, true});
    }
    if (ahead.empty()) return false;
    CacheManager& cache = *loaded_->cache;
    std::vector<int> need(static_cast<size_t>(cache.n_groups()), 0);
    for (const PlannedEntry& e : ahead) {
        const std::vector<int> n = cache.pages_needed(e.request->slot, e.start, 1);
        for (size_t g = 0; g < n.size(); ++g) need[g] += n[g];
    }
    const std::vector<int> free = cache.free_pages();
    for (size_t g = 0; g < need.size(); ++g)
        if (need[g] > free[g]) return false;     // let the ordinary step decide what to do without pages
    for (const PlannedEntry& e : ahead)
        if (!cache.prepare(e.request->slot, e.start, 1)) return false;
    return true;
}

long long Engine::run_steps(long long limit) {
    bool have = false;
    Launched launched;
    long long done = 0, begun = 0;
    int idle = 0;
    while (have || (has_work() && (limit < 0 || begun < limit))) {
        if (!have) {
            std::vector<PlannedEntry> plan = scheduler_->plan();
            sync_slots();
            if (plan.empty()) {
                // (the scheduler ends or fails what cannot advance, so this does not repeat; a
                // loop that spins on nothing must still end)
                if (++idle > 1000) throw StepError("the scheduler has work but plans no step");
                continue;
            }
            idle = 0;
            ++begun;
            if (!launch(plan, false, launched)) continue;
            have = true;
        }
        std::vector<PlannedEntry> ahead;
        Launched following;
        const bool has_following = (limit < 0 || begun < limit) && plan_ahead(launched.plan, ahead) && launch(ahead, true, following);
        if (has_following) ++begun;
        complete(launched);
        ++done;
        have = has_following;
        if (has_following) launched = std::move(following);
    }
    return done;
}

Json Engine::metrics() const {
    const ModelRunner& r = *loaded_->runner;
    Json out = Json::object();
    out.set("steps", steps_).set("steps_ahead", steps_ahead_).set("failed_steps", failed_steps_)
        .set("decode_steps", decode_steps_).set("portion_steps", portion_steps_).set("mixed_steps", mixed_steps_)
        .set("step_seconds", step_seconds_).set("graph_replays", r.graph_replays).set("captures", r.captures)
        .set("capture_seconds", r.capture_seconds).set("steps_run", r.steps_run)
        .set("scheduler", scheduler_->stats()).set("cache", loaded_->cache->memory_bytes())
        .set("workspace_bytes", static_cast<long long>(loaded_->rt->ws.bytes()));
    return out;
}

Json Engine::request_metrics(long long id) {
    const Request& req = scheduler_->request(id);
    return Json::object().set("id", req.id).set("status", status_name(req.status))
        .set("prompt_tokens", static_cast<long long>(req.prompt.size()))
        .set("generated_tokens", static_cast<long long>(req.generated.size()))
        .set("ttft_seconds", req.ttft_seconds >= 0 ? Json(req.ttft_seconds) : Json())
        .set("itl_mean_seconds", req.itl_count ? Json(req.itl_sum_seconds / req.itl_count) : Json())
        .set("itl_max_seconds", req.itl_count ? Json(req.itl_max_seconds) : Json())
        .set("preemptions", req.preemptions).set("error", req.error);
}

std::vector<float> Engine::last_logits(int& rows, int& vocab) {
    rows = vocab = 0;
    if (!last_logits_.defined()) return {};
    rows = static_cast<int>(last_logits_.shape[0]);
    vocab = static_cast<int>(last_logits_.shape[1]);
    std::vector<float> host(static_cast<size_t>(rows) * vocab);
    if (host.empty()) return host;
    CELEG_HIP(hipStreamSynchronize(loaded_->stream));
    CELEG_HIP(hipMemcpy2D(host.data(), static_cast<size_t>(vocab) * 4, last_logits_.data,
                          static_cast<size_t>(last_logits_.row_stride()) * 4, static_cast<size_t>(vocab) * 4,
                          static_cast<size_t>(rows), hipMemcpyDeviceToHost));
    return host;
}

}  // namespace celeg
