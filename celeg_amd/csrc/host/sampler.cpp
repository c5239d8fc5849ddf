#include "sampler.hpp"

#include <cmath>
#include <cstring>

namespace celeg {

void GenerationConfig::validate() const {
    if (!std::isfinite(temperature) || temperature < 0.0f) throw ConfigError("temperature must be finite and non-negative");
    if (top_k <= 0 || top_k > MAX_TOP_K) throw ConfigError("top_k must be between 1 and " + std::to_string(MAX_TOP_K));
    if (!std::isfinite(top_p) || top_p <= 0.0f || top_p > 1.0f) throw ConfigError("top_p must be in (0, 1]");
    if (!std::isfinite(repetition_penalty) || repetition_penalty < 1.0f)
        throw ConfigError("repetition_penalty must be finite and at least 1");
    if (seed == 0) throw ConfigError("seed must be non-zero");
    for (int t : forced_prefix)
        if (t < 0) throw ConfigError("forced_prefix holds a negative token id");
}

XorShift64Star::XorShift64Star(uint64_t seed) : state(seed) {
    if (seed == 0) throw ConfigError("seed must be non-zero");
}

float XorShift64Star::next_unit() {
    uint64_t s = state;
    s ^= s >> 12;
    s ^= s << 25;
    s ^= s >> 27;
    state = s;
    const uint64_t bits = s * 2685821657736338717ULL;
    return static_cast<float>((static_cast<double>(bits >> 11) + 0.5) * (1.0 / 9007199254740992.0));
}

Sampler::Sampler(Runtime& rt, int vocab, int max_requests) : rt_(rt), vocab_(vocab), cap_(max_requests) {
    const size_t cap = static_cast<size_t>(cap_);
    // one staging buffer and one device buffer for a step's parameters: 4 floats a row, then 3
    // ints a row (two staging buffers take turns, like the buffers the tokens come back through)
    for (auto& p : params_) {
        p = PinnedBuffer(cap * 7 * 4);
        std::memset(p.ptr(), 0, cap * 7 * 4);
    }
    params_dev_ = DeviceBuffer(cap * 7 * 4, true);
    last_tokens_ = DeviceBuffer((cap + 1) * 4, true);
    // sampled tokens come back through two pinned buffers that take turns, so that one step's
    // tokens can still be on their way while the next step is launched
    for (auto& t : tokens_host_) t = PinnedBuffer(cap * 4);
    for (auto& e : events_) CELEG_HIP(hipEventCreateWithFlags(&e, hipEventDisableTiming));
}

Sampler::~Sampler() {
    for (auto e : events_)
        if (e) (void)hipEventDestroy(e);
}

void Sampler::begin(int slot, const GenerationConfig& config, std::shared_ptr<XorShift64Star> rng, size_t generated) {
    config.validate();
    for (int t : config.forced_prefix)
        if (t >= vocab_) throw ConfigError("forced_prefix: token id " + std::to_string(t) + " out of range [0, " + std::to_string(vocab_) + ")");
    configs_[slot] = config;
    forced_used_[slot] = std::min(generated, config.forced_prefix.size());
    rng_[slot] = rng ? std::move(rng) : std::make_shared<XorShift64Star>(config.seed);
    if (config.repetition_penalty > 1.0f && !seen_.ptr()) {
        seen_ = DeviceBuffer(static_cast<size_t>(cap_) * vocab_, true);
    } else if (seen_.ptr()) {
        CELEG_HIP(hipMemsetAsync(seen_.as<uint8_t>() + static_cast<size_t>(slot) * vocab_, 0, static_cast<size_t>(vocab_), rt_.stream));
    }
}

void Sampler::end(int slot) {
    configs_.erase(slot);
    rng_.erase(slot);
    forced_used_.erase(slot);
}

bool Sampler::uses_seen() const {
    if (!seen_.ptr()) return false;
    for (const auto& c : configs_)
        if (c.second.repetition_penalty > 1.0f) return true;
    return false;
}

void Sampler::mark_seen(const StepBatch& batch) {
    if (uses_seen())
        rt_.ops.mark_seen(seen_.as<uint8_t>(), static_cast<size_t>(vocab_), cap_, vocab_, batch.token_ids, batch.token_slot, batch.n_tokens);
}

void Sampler::launch(const Tensor& logits, const std::vector<int>& slots) {
    const int R = static_cast<int>(slots.size());
    if (logits.shape[0] != R || logits.shape[1] != vocab_) throw StepError("sample: one row of logits per slot is needed");
    if (R > cap_) throw StepError("sample: more rows than requests");
    if (pending_.size() >= 2) throw StepError("sample: two launches are open; fetch one first");
    const int turn = turn_;        // its previous launch has been fetched: its buffers are free
    turn_ ^= 1;
    const size_t cap = static_cast<size_t>(cap_);
    float* f = params_[turn].as<float>();
    int* iv = reinterpret_cast<int*>(f + cap * 4);
    bool all_greedy = true, penalised = false;
    for (int r = 0; r < R; ++r) {
        auto cit = configs_.find(slots[static_cast<size_t>(r)]);
        if (cit == configs_.end()) throw StepError("sample: slot " + std::to_string(slots[static_cast<size_t>(r)]) + " has no request");
        const GenerationConfig& c = cit->second;
        f[4 * r] = c.temperature;
        f[4 * r + 1] = c.top_p;
        f[4 * r + 2] = c.repetition_penalty;
        size_t& forced_used = forced_used_[slots[static_cast<size_t>(r)]];
        const bool forced = forced_used < c.forced_prefix.size();
        f[4 * r + 3] = (c.greedy() || forced) ? 0.0f : rng_[slots[static_cast<size_t>(r)]]->next_unit();
        // a forced token travels in the place of top_k as -(token + 1): the kernel gives it out
        // (and marks it as seen, and leaves it for the next step) instead of choosing one
        iv[3 * r] = forced ? -(c.forced_prefix[forced_used++] + 1) : c.top_k;
        iv[3 * r + 1] = (c.repetition_penalty > 1.0f && seen_.ptr()) ? slots[static_cast<size_t>(r)] : -1;
        iv[3 * r + 2] = slots[static_cast<size_t>(r)];
        all_greedy = all_greedy && c.greedy() && !forced;
        penalised = penalised || iv[3 * r + 1] >= 0;
    }
    // greedy rows have nothing that changes from step to step: ship only what differs from what
    // the device holds
    std::vector<uint32_t> used(static_cast<size_t>(7 * R));
    std::memcpy(used.data(), f, static_cast<size_t>(4 * R) * 4);
    std::memcpy(used.data() + 4 * R, iv, static_cast<size_t>(3 * R) * 4);
    if (used != uploaded_) {
        CELEG_HIP(hipMemcpyAsync(params_dev_.ptr(), params_[turn].ptr(), cap * 7 * 4, hipMemcpyHostToDevice, rt_.stream));
        uploaded_ = used;
    }
    const float* fdev = params_dev_.as<float>();
    const int* idev = reinterpret_cast<const int*>(fdev + cap * 4);
    // the kernels write the tokens straight into the turn's pinned buffer (memory of the host that
    // the device can address): no copy behind them, the event tells when they are there
    rt_.ops.sample(logits, fdev, idev, seen_.as<uint8_t>(), static_cast<size_t>(vocab_), tokens_host_[turn].as<int>(),
                   last_tokens_.as<int>(), all_greedy, rt_.ws, &rt_.head_best, penalised);
    CELEG_HIP(hipEventRecord(events_[turn], rt_.stream));
    pending_.emplace_back(turn, R);
}

std::vector<int> Sampler::fetch() {
    if (pending_.empty()) return {};
    const auto [turn, R] = pending_.front();
    pending_.pop_front();
    CELEG_HIP(hipEventSynchronize(events_[turn]));
    const int* host = tokens_host_[turn].as<int>();
    return std::vector<int>(host, host + R);
}

}  // namespace celeg
