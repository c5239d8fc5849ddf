#include "scheduler.hpp"

#include <algorithm>

namespace celeg {

const char* status_name(RequestStatus s) {
    switch (s) {
        case RequestStatus::Queued: return "queued";
        case RequestStatus::Prefill: return "prefill";
        case RequestStatus::Decoding: return "decoding";
        case RequestStatus::Finished: return "finished";
        case RequestStatus::Cancelled: return "cancelled";
        default: return "failed";
    }
}

void SchedulerOptions::validate() const {
    if (max_active_requests <= 0 || max_batched_tokens <= 0 || prefill_chunk_tokens <= 0 || portion_granule <= 0)
        throw ConfigError("scheduler options must be positive");
    if (policy != "max_utilization" && policy != "guaranteed_no_evict")
        throw ConfigError("policy must be max_utilization or guaranteed_no_evict");
}

std::vector<int> Request::tokens(int begin, int count) const {
    std::vector<int> out;
    const int p = static_cast<int>(prompt.size());
    for (int i = begin; i < begin + count; ++i)
        out.push_back(i < p ? prompt[static_cast<size_t>(i)] : generated[static_cast<size_t>(i - p)]);
    return out;
}

Scheduler::Scheduler(CacheManager& c, SchedulerOptions o, int max_ctx, std::vector<int> default_eos)
    : cache(c), options(std::move(o)), max_context(max_ctx), default_eos_(std::move(default_eos)) {
    options.validate();
}

// ---------------------------------------------------------------------------- submission
long long Scheduler::submit(const std::vector<int>& prompt, const RequestOptions& opts) {
    if (prompt.empty()) throw ConfigError("request prompt is empty");
    if (static_cast<int>(prompt.size()) > max_context) throw ConfigError("request prompt exceeds max_context");
    if (opts.max_new_tokens <= 0) throw ConfigError("max_new_tokens must be positive");
    if (static_cast<long long>(prompt.size()) + opts.max_new_tokens > max_context)
        throw ConfigError("prompt plus max_new_tokens exceeds max_context");
    opts.generation.validate();
    auto req = std::make_unique<Request>();
    req->id = next_id_++;
    req->prompt = prompt;
    req->options = opts;
    req->eos = opts.eos_token_ids ? *opts.eos_token_ids : default_eos_;
    req->submitted = std::chrono::steady_clock::now();
    Request* raw = req.get();
    requests_[raw->id] = std::move(req);
    queue_.push_back(raw);
    return raw->id;
}

Request& Scheduler::request(long long id) {
    auto it = requests_.find(id);
    if (it == requests_.end()) throw ConfigError("unknown request id " + std::to_string(id));
    return *it->second;
}

void Scheduler::cancel(long long request_id) {
    Request& req = request(request_id);
    if (!is_done(req.status)) req.cancel_requested = true;
}

bool Scheduler::release_request(long long request_id) {
    Request& req = request(request_id);
    if (!is_done(req.status)) return false;
    // (a request that has ended is in no list any more; a slot event of this very step may
    // still name it)
    new_slots_.erase(std::remove_if(new_slots_.begin(), new_slots_.end(),
                                    [&](const std::pair<int, Request*>& b) { return b.second == &req; }),
                     new_slots_.end());
    requests_.erase(request_id);
    return true;
}

// ---------------------------------------------------------------------------- planning
Request* Scheduler::best_queued() const {
    Request* best = nullptr;
    for (Request* r : queue_)
        if (!best || r->options.priority > best->options.priority ||
            (r->options.priority == best->options.priority && r->id < best->id))
            best = r;
    return best;
}

void Scheduler::release(Request& req, RequestStatus status, const std::string& error) {
    if (req.slot >= 0) {
        cache.close(req.slot);
        released_slots_.push_back(req.slot);
        req.slot = -1;
    }
    active_.erase(std::remove(active_.begin(), active_.end(), &req), active_.end());
    queue_.erase(std::remove(queue_.begin(), queue_.end(), &req), queue_.end());
    req.status = status;
    req.error = error;
}

// The largest n <= want such that the pages for positions [start, start+n) can be had now
// (0 if not even one token can).
int Scheduler::affordable(const Request& req, int start, int want) const {
    const int P = cache.page_tokens;
    int n = want;
    const std::vector<int> free = cache.free_pages();
    while (n > 0) {
        const std::vector<int> need = cache.pages_needed(req.slot, start, n);
        bool ok = true;
        for (size_t g = 0; g < need.size(); ++g) ok = ok && need[g] <= free[g];
        if (ok) return n;
        // shrink to the end of the previous page
        const int end = start + n;
        n = ((end - 1) / P) * P - start;
    }
    return 0;
}

void Scheduler::admit(int budget) {
    while (!queue_.empty() && static_cast<int>(active_.size()) < options.max_active_requests &&
           cache.n_free_slots() > 0 && budget > 0) {
        Request* req = best_queued();
        const int slot = cache.open();
        if (slot < 0) return;
        req->slot = slot;
        const int total = req->sequence_length();
        bool ok;
        if (options.policy == "guaranteed_no_evict") {
            ok = cache.prepare(slot, 0, static_cast<int>(req->prompt.size()) + req->options.max_new_tokens);
        } else {
            const int first = std::min({total, options.prefill_chunk_tokens, budget});
            ok = affordable(*req, 0, first) > 0;
        }
        if (!ok) {
            cache.close(slot);
            req->slot = -1;
            if (active_.empty()) {
                // nothing is running and it still does not fit: it never will
                release(*req, RequestStatus::Failed, "request needs more cache pages than the pool holds");
                continue;
            }
            return;            // stays queued; admission stops here
        }
        queue_.erase(std::remove(queue_.begin(), queue_.end(), req), queue_.end());
        req->status = RequestStatus::Prefill;
        req->fed = 0;
        req->order = admitted_++;
        active_.push_back(req);
        new_slots_.emplace_back(slot, req);
        budget -= std::min(total, options.prefill_chunk_tokens);
    }
}

std::vector<PlannedEntry> Scheduler::plan() {
    for (auto& r : requests_)
        if (r.second->cancel_requested && !is_done(r.second->status)) release(*r.second, RequestStatus::Cancelled);
    for (;;) {
        std::vector<PlannedEntry> entries = plan_once();
        if (!entries.empty() || active_.empty()) return entries;
        preempt_youngest();
    }
}

std::vector<PlannedEntry> Scheduler::plan_once() {
    std::vector<PlannedEntry> entries;
    int budget = options.max_batched_tokens;
    const std::vector<Request*> running = active_;
    for (Request* req : running) {
        if (!(req->sequence_length() - req->fed == 1 && req->status == RequestStatus::Decoding)) continue;
        if (budget <= 0) break;
        if (cache.prepare(req->slot, req->fed, 1)) {
            entries.push_back(PlannedEntry{req, req->fed, 1, true});
            --budget;
        } else {
            ++stalled_decodes_;
        }
    }
    admit(budget);
    for (Request* req : active_) {
        if (req->status != RequestStatus::Prefill || budget <= 0) continue;
        const int remaining = req->sequence_length() - req->fed;
        int count = std::min({remaining, options.prefill_chunk_tokens, budget});
        if (count == budget && count < std::min(remaining, options.prefill_chunk_tokens)) {
            const int rounded = count - count % options.portion_granule;
            if (rounded > 0 || !entries.empty()) count = rounded;
        }
        count = affordable(*req, req->fed, count);
        if (count <= 0) continue;
        if (!cache.prepare(req->slot, req->fed, count)) continue;
        entries.push_back(PlannedEntry{req, req->fed, count, req->fed + count == req->sequence_length()});
        budget -= count;
    }
    return entries;
}

void Scheduler::preempt_youngest() {
    Request* victim = *std::max_element(active_.begin(), active_.end(),
                                        [](const Request* a, const Request* b) { return a->order < b->order; });
    if (active_.size() == 1) {
        release(*victim, RequestStatus::Failed, "request needs more cache pages than the pool holds");
        return;
    }
    cache.close(victim->slot);
    released_slots_.push_back(victim->slot);
    victim->slot = -1;
    victim->fed = 0;
    victim->status = RequestStatus::Queued;
    ++victim->preemptions;
    ++preemptions_;
    active_.erase(std::remove(active_.begin(), active_.end(), victim), active_.end());
    queue_.insert(queue_.begin(), victim);
}

void Scheduler::drain_slot_events(std::vector<int>& released, std::vector<std::pair<int, Request*>>& bound) {
    released.swap(released_slots_);
    bound.swap(new_slots_);
    released_slots_.clear();
    new_slots_.clear();
}

// ---------------------------------------------------------------------------- after the step
void Scheduler::accept(const std::vector<PlannedEntry>& entries, const std::vector<int>& sampled) {
    ++steps_;
    size_t next = 0;
    const auto now = std::chrono::steady_clock::now();
    const long long decoded_before = decode_tokens_, prefilled_before = prefill_tokens_;
    for (const PlannedEntry& e : entries) {
        Request& req = *e.request;
        if (e.count == 1 && req.status == RequestStatus::Decoding) ++decode_tokens_;
        else prefill_tokens_ += e.count;
    }
    if (decode_tokens_ > decoded_before && prefill_tokens_ > prefilled_before) ++mixed_steps_;
    for (const PlannedEntry& e : entries) {
        Request& req = *e.request;
        req.fed = e.start + e.count;
        if (!e.samples) continue;
        if (next >= sampled.size()) throw StepError("accept: fewer sampled tokens than sampling entries");
        const int token = sampled[next++];
        if (req.generated.empty() && req.ttft_seconds < 0) {
            req.ttft_seconds = std::chrono::duration<double>(now - req.submitted).count();
        } else if (!req.generated.empty()) {
            const double gap = std::chrono::duration<double>(now - req.last_token).count();
            req.itl_sum_seconds += gap;
            req.itl_max_seconds = std::max(req.itl_max_seconds, gap);
            ++req.itl_count;
        }
        req.last_token = now;
        req.generated.push_back(token);
        req.pending.push_back(token);
        req.status = RequestStatus::Decoding;
        const bool ended = std::find(req.eos.begin(), req.eos.end(), token) != req.eos.end();
        if (ended || static_cast<int>(req.generated.size()) >= req.options.max_new_tokens || req.sequence_length() >= max_context)
            release(req, RequestStatus::Finished);
    }
}

void Scheduler::fail(const std::vector<PlannedEntry>& entries, const std::string& message) {
    for (const PlannedEntry& e : entries)
        if (!is_done(e.request->status)) release(*e.request, RequestStatus::Failed, message);
}

Json Scheduler::stats() const {
    return Json::object().set("steps", steps_).set("preemptions", preemptions_).set("stalled_decodes", stalled_decodes_)
        .set("prefill_tokens", prefill_tokens_).set("decode_tokens", decode_tokens_).set("mixed_steps", mixed_steps_);
}

}  // namespace celeg
