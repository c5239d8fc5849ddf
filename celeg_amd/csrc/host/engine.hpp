// The engine: submit / step / poll / cancel, and generate.
//
// Shaped after the reference's concurrent engine and its C API
// (include/celeg/backend/cuda/concurrency.hpp:36-70; include/celeg/api.h:19-183): one step()
// admits, runs ONE batch through the step function, samples on the returned logits and frees
// what finished.  An exception while a step is launched or completed marks the step's requests
// Failed with the message, gives back their pages and slots and leaves the engine usable
// (src/backend/cuda/runtime/request_lifecycle.cpp:200-218).
#pragma once
#include <memory>
#include <string>
#include <vector>

#include "model.hpp"
#include "sampler.hpp"
#include "scheduler.hpp"

namespace celeg {

struct EngineOptions {
    LoadOptions load;
    int prefill_chunk_tokens = 1024;
    std::string policy = "max_utilization";
    int portion_granule = 1;
    bool run_ahead = true;
};

class Engine {
public:
    // (Steps of 2,048 tokens and portions of 1,024 by default: on an MI355X a step of a few
    // hundred rows leaves most of the chip idle.  SchedulerOptions keeps the reference's 512 / 256,
    // include/celeg/backend/cuda/concurrency.hpp:18-32.)
    Engine(const std::string& model_dir, const EngineOptions& options);
    Engine(std::unique_ptr<LoadedModel> loaded, const SchedulerOptions& options, bool run_ahead);

    long long submit(const std::vector<int>& prompt, const RequestOptions& options);
    void cancel(long long id) { scheduler_->cancel(id); }
    bool release(long long id) { return scheduler_->release_request(id); }
    RequestStatus status(long long id) { return scheduler_->request(id).status; }
    // drains the tokens generated since the last poll (src/backend/cuda/runtime/request_lifecycle.cpp:57-73)
    RequestStatus poll(long long id, std::vector<int>& tokens, std::string& error);
    bool has_work() const { return scheduler_->has_work(); }
    // runs one batch; returns the number of tokens it fed (0 if there was nothing)
    int step();
    // runs until no request is queued or active (limit < 0) or for at most `limit` steps, launching
    // decode steps one ahead of their tokens; returns the number of steps
    long long run_steps(long long limit);
    void run() { run_steps(-1); }
    Json metrics() const;
    Json request_metrics(long long id);
    // 32-bit logits of the last step on the host, [rows, vocab] (for --dump-logits)
    std::vector<float> last_logits(int& rows, int& vocab);

    LoadedModel& loaded() { return *loaded_; }
    Scheduler& scheduler() { return *scheduler_; }
    Sampler& sampler() { return *sampler_; }

private:
    struct Launched {
        std::vector<PlannedEntry> plan;
        bool sampled_rows = false;
        std::chrono::steady_clock::time_point start;
    };
    void sync_slots();
    bool launch(const std::vector<PlannedEntry>& plan, bool device_tokens, Launched& out);
    int complete(Launched& launched);
    bool plan_ahead(const std::vector<PlannedEntry>& plan, std::vector<PlannedEntry>& ahead);
    void contain(const std::vector<PlannedEntry>& plan, const std::string& message);

    std::unique_ptr<LoadedModel> loaded_;
    std::unique_ptr<Scheduler> scheduler_;
    std::unique_ptr<Sampler> sampler_;
    bool run_ahead_ = true;
    Tensor last_logits_;
    long long steps_ = 0, steps_ahead_ = 0, failed_steps_ = 0;
    long long decode_steps_ = 0, portion_steps_ = 0, mixed_steps_ = 0;      // launched steps by kind
    double step_seconds_ = 0.0;
};

}  // namespace celeg
