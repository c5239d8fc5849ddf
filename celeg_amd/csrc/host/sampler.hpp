// Generation options and the sampler that turns rows of logits into tokens.
//
// Names, meanings, defaults and limits are the reference's GenerationConfig
// (include/celeg/model/runtime_types.hpp:98-108; validation
// src/model/execution/runtime_types.cpp:20-37): greedy when temperature <= 0 or top_k == 1;
// top_k in [1, 128]; top_p in (0, 1]; repetition_penalty >= 1; a non-zero seed.  Each request
// owns one xorshift64* state (src/backend/cpu/sampler.cpp:10-22), kept on the host and seeded
// with its seed, so a request's draws do not depend on its batch mates.  The selection itself
// runs on the GPU, one workgroup per row.
#pragma once
#include <cstdint>
#include <deque>
#include <map>
#include <memory>
#include <vector>

#include "ops.hpp"

namespace celeg {

constexpr int MAX_TOP_K = 128;

struct GenerationConfig {
    float temperature = 0.1f;
    int top_k = 50;
    float top_p = 1.0f;
    float repetition_penalty = 1.05f;
    uint64_t seed = 1;
    // given out as the first generated tokens instead of sampled ones, without a draw from the
    // generator (include/celeg/model/runtime_types.hpp:93-104; src/backend/cpu/sampler.cpp:31-34)
    std::vector<int> forced_prefix;
    bool greedy() const { return temperature <= 0.0f || top_k == 1; }
    void validate() const;     // throws ConfigError
};

// s ^= s>>12; s ^= s<<25; s ^= s>>27; bits = s * 2685821657736338717;
// unit = float(((bits >> 11) + 0.5) / 2^53)  (src/backend/cpu/sampler.cpp:10-22)
class XorShift64Star {
public:
    explicit XorShift64Star(uint64_t seed);
    float next_unit();
    uint64_t state;
};

// Per-slot sampling state (generator, seen tokens) and the device call.
class Sampler {
public:
    Sampler(Runtime& rt, int vocab, int max_requests);
    ~Sampler();
    Sampler(const Sampler&) = delete;
    // Bind a request to `slot`.  rng continues an existing generator (a request that was
    // preempted and comes back); null: a fresh one is seeded.  `generated`: how many tokens the
    // request has been given already (as many of its forced prefix are used up).
    void begin(int slot, const GenerationConfig& config, std::shared_ptr<XorShift64Star> rng = nullptr, size_t generated = 0);
    void end(int slot);
    bool uses_seen() const;
    // every token a step feeds (prompt portions and decoded tokens) counts as seen by its request
    void mark_seen(const StepBatch& batch);
    // Starts the sampling of one token per row without waiting for it; fetch returns the tokens
    // of the oldest launch not fetched yet (at most two may be open).
    void launch(const Tensor& logits, const std::vector<int>& slots);
    std::vector<int> fetch();
    std::vector<int> sample(const Tensor& logits, const std::vector<int>& slots) {
        if (slots.empty()) return {};
        launch(logits, slots);
        return fetch();
    }
    // int32 [slots + 1] on the device: the token every slot sampled last
    int* last_tokens() const { return last_tokens_.as<int>(); }

private:
    Runtime& rt_;
    int vocab_, cap_;
    std::map<int, GenerationConfig> configs_;
    std::map<int, std::shared_ptr<XorShift64Star>> rng_;
    std::map<int, size_t> forced_used_;      // of the slot's forced prefix
    DeviceBuffer seen_;            // [max_requests, vocab] bytes, made on need
    PinnedBuffer params_[2];       // 4 floats a row, then 3 ints a row
    DeviceBuffer params_dev_, last_tokens_;
    std::vector<uint32_t> uploaded_;
    PinnedBuffer tokens_host_[2];
    hipEvent_t events_[2] = {nullptr, nullptr};
    std::deque<std::pair<int, int>> pending_;      // launched and not fetched yet: (turn, rows)
    int turn_ = 0;
};

}  // namespace celeg
