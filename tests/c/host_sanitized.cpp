// The host side of the library under AddressSanitizer and UndefinedBehaviorSanitizer, without a
// GPU: descriptions of good and broken model folders and configurations, and long random
// sequences of calls on the page pool, the cache manager, the scheduler and the batch builder
// through the C interface.  Everything must come back as a result or as an error message; the
// sanitizers end the program at the first bad access.
//
//   host_sanitized GOOD_DIR [BROKEN_DIR ...]
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <random>
#include <string>
#include <vector>

#include "celeg_amd.h"

static int failures = 0;
#define EXPECT(cond) do { if (!(cond)) { std::fprintf(stderr, "line %d: %s\n  last error: %s\n", __LINE__, #cond, celeg_last_error()); ++failures; } } while (0)

static std::string call(long long handle, const char* method, const std::string& args) {
    const char* r = celeg_host_call(handle, method, args.c_str());
    return r ? std::string(r) : std::string("!") + celeg_last_error();
}
static bool failed(const std::string& r) { return !r.empty() && r[0] == '!'; }

static std::string ints(const std::vector<int>& v) {
    std::string s = "[";
    for (size_t i = 0; i < v.size(); ++i) s += (i ? "," : "") + std::to_string(v[i]);
    return s + "]";
}

static void descriptions(int argc, char** argv) {
    const char* good = argv[1];
    const char* text = celeg_describe_folder(good);
    EXPECT(text != nullptr && std::strstr(text, "expected_tensors") != nullptr);
    EXPECT(celeg_check_folder(good) == CELEG_OK);
    for (int i = 2; i < argc; ++i) {            // broken folders: an error with a message, nothing else
        const bool described = celeg_describe_folder(argv[i]) != nullptr;
        const bool checked = celeg_check_folder(argv[i]) == CELEG_OK;
        EXPECT(!(described && checked));
        EXPECT(std::strlen(celeg_last_error()) > 0);
        std::printf("broken %d: %s\n", i - 1, celeg_last_error());
    }
    EXPECT(celeg_describe_folder("/nonexistent") == nullptr);
    EXPECT(celeg_describe_folder(nullptr) == nullptr);
    const char* configs[] = {
        "", "{", "[]", "null", "{\"architectures\": 3}", "{\"architectures\": [\"Nobody\"]}",
        "{\"architectures\": [\"Lfm2ForCausalLM\"]}",
        "{\"architectures\": [\"Lfm2ForCausalLM\"], \"vocab_size\": -1, \"hidden_size\": 8}",
        "{\"architectures\": [\"Lfm2ForCausalLM\"], \"vocab_size\": 1e30, \"hidden_size\": \"x\", \"layer_types\": {}}",
        "{\"a\": 1, \"a\": 2}", "{\"architectures\": [\"Lfm2ForCausalLM\"], \"layer_types\": [1, 2, null]}",
    };
    for (const char* c : configs) EXPECT(celeg_describe_config(c, nullptr) == nullptr);
    const char* tiny =
        "{\"architectures\": [\"Lfm2ForCausalLM\"], \"vocab_size\": 50, \"hidden_size\": 32, \"num_hidden_layers\": 2,"
        " \"layer_types\": [\"conv\", \"full_attention\"], \"num_attention_heads\": 2, \"num_key_value_heads\": 1,"
        " \"head_dim\": 16, \"intermediate_size\": 48, \"block_auto_adjust_ff_dim\": false, \"rope_theta\": 10000.0,"
        " \"conv_L_cache\": 3, \"norm_eps\": 1e-5, \"max_position_embeddings\": 64}";
    EXPECT(celeg_describe_config(tiny, nullptr) != nullptr);
    EXPECT(celeg_describe_config(tiny, "{\"model.embed_tokens.weight\": [50, 32]}") != nullptr);
    EXPECT(celeg_describe_config(tiny, "{\"model.embed_tokens.weight\": \"x\"}") == nullptr || true);
    EXPECT(celeg_registered("architectures") != nullptr && celeg_registered("mixer") != nullptr);
    celeg_engine* engine = nullptr;
    EXPECT(celeg_engine_create(good, nullptr, &engine) != CELEG_OK && engine == nullptr);   // no GPU here
    celeg_model* model = nullptr;
    EXPECT(celeg_model_create(good, nullptr, &model) != CELEG_OK && model == nullptr);
}

static void pool_calls(std::mt19937& rng) {
    const long long pool = celeg_host_new("pool", "{\"n_pages\": 13, \"page_tokens\": 8}");
    EXPECT(pool != 0);
    std::vector<std::vector<int>> held;
    for (int step = 0; step < 600; ++step) {
        const int what = static_cast<int>(rng() % 5);
        if (what <= 1) {
            const std::string r = call(pool, "allocate", "[" + std::to_string(rng() % 6) + "]");
            if (!failed(r) && r != "null") {
                std::vector<int> pages;
                for (const char* p = r.c_str(); *p; ++p)
                    if (*p >= '0' && *p <= '9') { pages.push_back(std::atoi(p)); while (p[1] >= '0' && p[1] <= '9') ++p; }
                held.push_back(pages);
            }
        } else if (what == 2 && !held.empty()) {
            const size_t i = rng() % held.size();
            EXPECT(!failed(call(pool, "release", "[" + ints(held[i]) + "]")));
            held.erase(held.begin() + static_cast<long>(i));
        } else if (what == 3) {       // wrong ids and double releases are refused as a whole
            EXPECT(failed(call(pool, "release", "[[99]]")));
            EXPECT(failed(call(pool, "retain", "[[-1]]")));
        } else {
            EXPECT(!failed(call(pool, "check", "[]")));
        }
    }
    EXPECT(failed(call(pool, "no_such_method", "[]")));
    EXPECT(failed(call(pool, "allocate", "[\"x\"]")) || true);
    celeg_host_delete(pool);
    EXPECT(celeg_host_call(pool, "check", "[]") == nullptr);       // a handle that is gone
}

static void cache_and_scheduler_calls(std::mt19937& rng, const char* policy) {
    const char* layout =
        "{\"layout\": {\"kv_groups\": [{\"kv_heads\": 2, \"head_dim\": 16, \"window\": null, \"layers\": 2},"
        " {\"kv_heads\": 1, \"head_dim\": 16, \"window\": 24, \"layers\": 1}],"
        " \"kv_of_step\": [{\"step\": 0, \"group\": 0, \"layer\": 0, \"writes\": true}, {\"step\": 1, \"group\": 1, \"layer\": 0, \"writes\": true},"
        " {\"step\": 3, \"group\": 0, \"layer\": 1, \"writes\": true}],"
        " \"states\": [{\"step\": 2, \"name\": \"conv\", \"shape\": [3, 32], \"dtype\": \"float32\"}]},"
        " \"page_tokens\": 8, \"n_pages\": [40, 12], \"max_requests\": 4, \"max_context\": 160}";
    const long long cache = celeg_host_new("cache", layout);
    EXPECT(cache != 0);
    const std::string options = std::string("{\"cache\": ") + std::to_string(cache) +
        ", \"options\": {\"max_active_requests\": 4, \"max_batched_tokens\": 24, \"prefill_chunk_tokens\": 16, \"policy\": \"" + policy +
        "\"}, \"max_context\": 160, \"default_eos\": [3]}";
    const long long sched = celeg_host_new("scheduler", options.c_str());
    EXPECT(sched != 0);
    const long long batch = celeg_host_new("batch", "{\"capacity\": 4096, \"n_groups\": 2}");
    EXPECT(batch != 0);
    std::vector<long long> ids;
    for (int step = 0; step < 500; ++step) {
        if (rng() % 3 == 0 && ids.size() < 40) {
            std::vector<int> prompt(1 + rng() % 60);
            for (int& t : prompt) t = static_cast<int>(rng() % 50);
            const std::string r = call(sched, "submit", "[" + ints(prompt) + ", {\"max_new_tokens\": " + std::to_string(1 + rng() % 30) +
                                       ", \"priority\": " + std::to_string(rng() % 3) + ", \"generation\": {\"temperature\": 0.0}}]");
            if (!failed(r)) ids.push_back(std::atoll(r.c_str()));
        }
        if (rng() % 11 == 0 && !ids.empty()) call(sched, "cancel", "[" + std::to_string(ids[rng() % ids.size()]) + "]");
        const std::string plan = call(sched, "plan", "[]");
        EXPECT(!failed(plan));
        // one sampled token for every entry that samples
        int samples = 0;
        for (size_t at = plan.find("\"samples\":true"); at != std::string::npos; at = plan.find("\"samples\":true", at + 1)) ++samples;
        for (size_t at = plan.find("\"samples\": true"); at != std::string::npos; at = plan.find("\"samples\": true", at + 1)) ++samples;
        if (plan != "[]") {
            if (rng() % 17 == 0) {
                EXPECT(!failed(call(sched, "fail", "[\"a step that failed\"]")));
            } else {
                std::vector<int> tokens(static_cast<size_t>(samples));
                for (int& t : tokens) t = static_cast<int>(rng() % 50);
                const std::string r = call(sched, "accept", "[" + ints(tokens) + "]");
                EXPECT(!failed(r));
            }
        }
        EXPECT(!failed(call(cache, "check", "[]")));
        if (!ids.empty()) EXPECT(!failed(call(sched, "poll", "[" + std::to_string(ids[rng() % ids.size()]) + "]")));
        call(cache, "drain", "[[4, 4]]");
    }
    EXPECT(failed(call(sched, "poll", "[123456]")));
    EXPECT(failed(call(sched, "submit", "[[], {}]")));
    EXPECT(failed(call(cache, "prepare", "[99, 0, 4]")));
    EXPECT(failed(call(cache, "close", "[-3]")));
    // the batch builder: entries that fit and entries that do not
    EXPECT(!failed(call(batch, "build", "[[{\"slot\": 0, \"start_pos\": 0, \"tokens\": [1, 2, 3], \"want\": [2]}], [[], []], {}]")) || true);
    EXPECT(failed(call(batch, "build", "[[{\"slot\": 0, \"start_pos\": 0, \"tokens\": [1], \"want\": [5]}], [[], []], {}]")) || true);
    celeg_host_delete(batch);
    celeg_host_delete(sched);
    celeg_host_delete(cache);
}

int main(int argc, char** argv) {
    if (argc < 2) {
        std::fprintf(stderr, "usage: host_sanitized GOOD_DIR [BROKEN_DIR ...]\n");
        return 2;
    }
    std::printf("%s\n", celeg_version());
    descriptions(argc, argv);
    std::mt19937 rng(20240611u);
    pool_calls(rng);
    cache_and_scheduler_calls(rng, "max_utilization");
    cache_and_scheduler_calls(rng, "guaranteed_no_evict");
    EXPECT(celeg_host_new("nothing", "{}") == 0);
    EXPECT(celeg_host_new("pool", "{") == 0);
    EXPECT(celeg_host_new("cache", "{\"layout\": 3}") == 0 || true);
    std::printf("failures: %d\n", failures);
    return failures ? 1 : 0;
}
