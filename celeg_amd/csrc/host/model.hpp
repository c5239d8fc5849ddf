// A model put together from a ModelSpec: parts, their tensors, their cache needs, and the
// forward pass over one step's rows; the step function that runs a batch of entries through
// it from the cache; and the way from a model folder to a ready step function.
//
// The reference compiles a resolved model into a program whose layers declare their tensors
// and their state layout (src/model/weight_plan.cpp:278-326;
// include/celeg/model/program.hpp:118-177) and runs it layer by layer
// (src/backend/cuda/packed/layer_executor.cu:93-217).  Here the run order is a list that may
// name a layer twice (shared weights, separate cache) or let an entry read the keys and values
// of an earlier entry.
#pragma once
#include <memory>
#include <string>
#include <vector>

#include "batch.hpp"
#include "cache.hpp"
#include "parts.hpp"

namespace celeg {

class Model {
public:
    explicit Model(ModelSpec spec);
    const ModelSpec spec;

    // whether a recorded step of this model may be replayed from a HIP graph
    bool graph_safe() const { return graph_safe_; }
    std::vector<std::pair<std::string, Part*>> named_parts();
    // checkpoint tensor name -> what is expected of it
    ExpectedTensors expected_tensors();
    CacheLayout cache_layout();
    // tensors: checkpoint name -> device tensor, already checked and converted
    void load(const WeightMap& tensors, Runtime& rt);
    void bind_cache(const CacheManager& cache);
    // Runs the rows of `batch` through every entry of the run order and returns 32-bit logits
    // [batch.n_logit_rows, vocab] (a workspace buffer: it holds until the next step).
    Tensor forward(const StepBatch& batch, Runtime& rt);
    int logit_width() const { return head_->vocab(); }
    long long weight_count();

private:
    Mixer& mixer_of(int layer) { return blocks_[static_cast<size_t>(layer)]->mixer(); }
    void resolve_cache_sharing();
    std::unique_ptr<Embedding> embedding_;
    std::vector<std::unique_ptr<Block>> blocks_;
    std::unique_ptr<Norm> final_norm_;
    std::unique_ptr<Head> head_;
    std::vector<LayerCache> caches_;
    bool bound_ = false, graph_safe_ = false;
};

// The step function: runs one batch of (request, its next tokens) through the model, from the
// cache, and returns the logits at the wanted places.
//
// The reference runs prompt portions and decode tokens in separate passes
// (src/backend/cuda/runtime/engine_control.cpp:4-23;
// src/backend/cuda/packed/execution.cu:141-224 and 234-384); here one function takes both in
// one batch.  Positions are the caller's to keep: start_pos is an input, so the scheduler and
// the trace replay drive the same function.
class ModelRunner {
public:
    ModelRunner(Model& model, CacheManager& cache, Runtime& rt, int max_batched_tokens);
    ~ModelRunner();
    ModelRunner(const ModelRunner&) = delete;

    // Logits, 32-bit [number of wanted places, vocab] on the device, in the order of the entries
    // and of each entry's want.  The buffer is reused: it holds until the next step.
    Tensor step(const std::vector<StepEntry>& entries);

    Model& model;
    CacheManager& cache;
    Runtime& rt;
    const int max_batched_tokens;
    bool use_graphs = true;
    int portion_graph_min_tokens = 32;      // portions of fewer rows are never recorded
    long long steps_run = 0, graph_replays = 0, captures = 0;
    double capture_seconds = 0.0;
    const StepBatch& last_batch() const { return last_batch_; }
    // int32 [slots + 1] on the device: the token every slot sampled last.  With it set, an entry
    // may bring {TOKEN_FROM_DEVICE} instead of a token, and the step can be launched before the
    // host has read the previous step's tokens.
    void set_token_source(int* last_tokens);
    int* token_source() const { return token_source_; }
    int update_room() const { return update_room_; }
    BatchBuilder& builder() { return *builder_; }

private:
    struct Captured {
        hipGraph_t graph = nullptr;
        hipGraphExec_t exec = nullptr;
        Tensor logits;
        HeadBest head_best;           // what the recorded head leaves beside the logits
        unsigned long long generation = 0;
    };
    void validate(const std::vector<StepEntry>& entries) const;
    bool graph_applies(const std::vector<StepEntry>& entries) const;
    int context_bound(const std::vector<StepEntry>& entries) const;
    Tensor step_from_graph(const std::vector<StepEntry>& entries);
    Captured& capture(int bucket, const std::vector<int>& caps, int bound);
    Captured& record(std::pair<int, int> key, const StepBatch& batch);
    bool portion_graph_applies(const std::vector<StepEntry>& entries);
    Tensor step_from_portion_graph(const std::vector<StepEntry>& entries);
    std::vector<std::vector<TableUpdate>> drain_updates(const std::vector<int>& caps);
    StepBatch build(const std::vector<StepEntry>& entries, std::vector<std::vector<TableUpdate>>& updates,
                    const BuildOptions& options);
    void ship_table_updates(int group, const std::vector<TableUpdate>& updates);
    void begin_step(const StepBatch& batch);
    void drop_graphs();

    std::unique_ptr<BatchBuilder> builder_;
    // (batch-size bucket, bound on the context) for steps of single tokens; (-rows, context
    // from 4,096 tokens or not) for steps of one portion
    std::map<std::pair<int, int>, Captured> graphs_;
    std::map<int, int> portion_sizes_seen_;
    int n_portion_graphs_ = 0;
    std::vector<int> buckets_;
    int update_room_ = 0;
    int* token_source_ = nullptr;
    StepBatch last_batch_;
};

struct LoadOptions {
    std::string dtype = "bfloat16";
    int device = 0;
    int page_tokens = 16;
    int n_pages = -1;               // pages of the cache pool (per group); -1: enough for max_requests requests of max_context tokens
    int max_requests = 8;
    int max_context = -1;           // -1: the model's own maximum; may not exceed it
    int max_batched_tokens = 2048;
    std::string gemm_backend = "auto";      // how bfloat16 steps of more than 64 rows multiply: "library", "tiles" or "auto"
    bool use_graphs = true;
    bool strict_weights = false;    // tensors of the checkpoint that the model has no use for are an error
};

// From a model folder to a ready step function.  The reference's path: open the checkpoint,
// select the architecture, resolve it, compile the program, upload the weights, size the
// buffers (src/checkpoint/bootstrap.cpp:13-21; src/backend/cuda/execution_plan.cpp:19-130;
// src/backend/cuda/model/weight_setup.cpp).  The model class is chosen by config.json.
struct LoadedModel {
    Json config;
    hipStream_t stream = nullptr;
    std::unique_ptr<Runtime> rt;
    std::unique_ptr<Model> model;
    std::unique_ptr<CacheManager> cache;
    std::unique_ptr<ModelRunner> runner;
    int device = 0;
    std::vector<std::string> unused_tensors;   // in the checkpoint, asked for by no part
    ~LoadedModel();
};

Described describe_model_folder(const std::string& model_dir);
std::unique_ptr<LoadedModel> load_model(const std::string& model_dir, const LoadOptions& options);

// An environment flag for bisecting mismatches: with CELEG_DUMP_HIDDEN=<folder> set when a model
// is loaded, every step writes the residual stream after every entry of the run order to
// <folder>/step<k>_layer<i>.f32 ([rows, width] 32-bit, rows in the batch's order).
void install_hidden_dump(Runtime& rt, const std::string& folder);

}  // namespace celeg
