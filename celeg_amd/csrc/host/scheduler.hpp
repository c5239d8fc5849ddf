// The scheduler: admits requests, cuts prompts into portions under a token budget, lets every
// decoding request take one token per step, finishes and frees.
//
// What it mirrors of the reference: submission checks
// (src/backend/cuda/runtime/request_lifecycle.cpp:10-32), the queue order priority descending
// then id ascending (src/runtime/concurrency/batch_planner.cpp:14-50), admission that stops at
// the first request whose pages cannot be had (the request stays queued,
// request_lifecycle.cpp:103-198), the token budget max_batched_tokens - #decoding and portions
// of at most prefill_chunk_tokens (src/backend/cuda/runtime/prefill_scheduler.cpp:4-186), the
// two reservation policies (decode_scheduler.cpp:23-66), finishing on an end token (which is
// emitted) or on max_new_tokens (decode_scheduler.cpp:68-99), and the states Queued, Prefill,
// Decoding, Finished, Cancelled, Failed (include/celeg/runtime/concurrency/policy.hpp:10-25).
//
// What differs: portions and decode tokens go into ONE step; logits are sampled after the step
// that produced them, so a request that finishes is not fed again.
//
// When pages run out: a queued request waits; a decoding request whose next token needs a page
// that is not free is left out of the step and tried again later (the reference does the same);
// a prompt portion is cut to what the free pages hold.  If no running request can take a single
// token, the youngest running request is preempted: it gives back its pages and slot and goes
// back to the head of the queue, to be recomputed from its prompt plus what it has generated
// (its output so far is kept).  A request that cannot fit the pool even alone fails.
//
// A request is one growing sequence, prompt + generated; `fed` counts how many of its tokens are
// in the cache.  A step feeds seq[fed:fed+n]; when that reaches the end of the sequence the last
// row's logits are sampled.  Decoding is the case n = 1.
#pragma once
#include <chrono>
#include <deque>
#include <map>
#include <memory>
#include <optional>
#include <string>
#include <vector>

#include "cache.hpp"
#include "sampler.hpp"

namespace celeg {

enum class RequestStatus : int { Queued = 0, Prefill = 1, Decoding = 2, Finished = 3, Cancelled = 4, Failed = 5 };
inline bool is_done(RequestStatus s) { return s == RequestStatus::Finished || s == RequestStatus::Cancelled || s == RequestStatus::Failed; }
const char* status_name(RequestStatus s);

// Defaults as include/celeg/runtime/request_types.hpp:16-26, except that the end tokens default
// to the model's own (unset here).
struct RequestOptions {
    int max_new_tokens = 128;
    std::optional<std::vector<int>> eos_token_ids;
    int priority = 0;
    GenerationConfig generation;
};

// Defaults as include/celeg/backend/cuda/concurrency.hpp:18-32.
struct SchedulerOptions {
    int max_active_requests = 8;
    int max_batched_tokens = 512;
    int prefill_chunk_tokens = 256;
    std::string policy = "max_utilization";      // or "guaranteed_no_evict"
    // 1: a portion that the step's budget cuts short is cut exactly at the budget, as the
    // reference does (src/backend/cuda/runtime/prefill_scheduler.cpp:4-186).  More: such a portion
    // (not one that the prompt's end or the portion size cuts) is shortened further to a multiple
    // of this, or left for the next step, so that the steps of a steady load repeat a few shapes.
    int portion_granule = 1;
    void validate() const;
};

struct Request {
    long long id = 0;
    std::vector<int> prompt;
    RequestOptions options;
    std::vector<int> eos;
    RequestStatus status = RequestStatus::Queued;
    int slot = -1;
    int fed = 0;
    std::vector<int> generated;
    std::deque<int> pending;       // generated, not yet polled
    std::string error;
    bool cancel_requested = false;
    int preemptions = 0;
    long long order = 0;           // admission order, for "youngest"
    std::shared_ptr<XorShift64Star> rng;    // survives preemption
    // latencies, as the reference records them per token (decode_scheduler.cpp:68-99):
    // submission to first token, and between tokens
    std::chrono::steady_clock::time_point submitted, last_token;
    double ttft_seconds = -1.0, itl_sum_seconds = 0.0, itl_max_seconds = 0.0;
    int itl_count = 0;

    int sequence_length() const { return static_cast<int>(prompt.size() + generated.size()); }
    std::vector<int> tokens(int begin, int count) const;
};

struct PlannedEntry {
    Request* request = nullptr;
    int start = 0, count = 0;
    bool samples = false;     // the portion reaches the end of the sequence: sample from its last row
};

class Scheduler {
public:
    Scheduler(CacheManager& cache, SchedulerOptions options, int max_context, std::vector<int> default_eos);
    long long submit(const std::vector<int>& prompt, const RequestOptions& options);
    void cancel(long long request_id);
    // Forgets a request that has ended (finished, cancelled or failed): its record, tokens that
    // were not polled and its metrics go.  False, and nothing happens, while it is queued or
    // running (the reference's release, src/backend/cuda/runtime/request_lifecycle.cpp:47-55).
    bool release_request(long long request_id);
    bool has_work() const { return !queue_.empty() || !active_.empty(); }
    // decide this step's entries; pages for them are taken here
    std::vector<PlannedEntry> plan();
    // sampled: one token for every entry with `samples`, in order
    void accept(const std::vector<PlannedEntry>& entries, const std::vector<int>& sampled);
    // a step that failed: its requests become Failed with the message and give back what they hold
    void fail(const std::vector<PlannedEntry>& entries, const std::string& message);
    Request& request(long long id);
    // (slots released, (slot, request) pairs newly bound) since the last call, in that order of
    // effect: the caller drops and starts per-slot sampling state with them
    void drain_slot_events(std::vector<int>& released, std::vector<std::pair<int, Request*>>& bound);
    Json stats() const;

    CacheManager& cache;
    const SchedulerOptions options;
    const int max_context;
    const std::vector<Request*>& queue() const { return queue_; }
    const std::vector<Request*>& active() const { return active_; }

private:
    Request* best_queued() const;
    void release(Request& req, RequestStatus status, const std::string& error = "");
    int affordable(const Request& req, int start, int want) const;
    void admit(int budget);
    std::vector<PlannedEntry> plan_once();
    void preempt_youngest();

    std::vector<int> default_eos_;
    std::map<long long, std::unique_ptr<Request>> requests_;
    std::vector<Request*> queue_, active_;
    long long next_id_ = 0, admitted_ = 0;
    std::vector<std::pair<int, Request*>> new_slots_;
    std::vector<int> released_slots_;
    long long steps_ = 0, preemptions_ = 0, stalled_decodes_ = 0, prefill_tokens_ = 0, decode_tokens_ = 0, mixed_steps_ = 0;
};

}  // namespace celeg
