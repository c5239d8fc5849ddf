// The kernels as host calls: shapes, dtypes, strides and limits are checked here, then the
// extern "C" entry points are called with raw device pointers and the runtime's stream (so a
// stream that is recording a graph records them too).  There is no fallback: a size a kernel
// was not written for is a KernelError that says why.
//
// Matrix products in bfloat16 of more than 64 rows go to hipBLASLt (blaslt.cpp), as the
// reference sends its products to cuBLAS (src/backend/cuda/runtime/gemm_dispatcher.cpp);
// products in 32-bit go to this library's own kernel, which uses no reduced-precision matrix
// mode.
#pragma once
#include <functional>
#include <map>
#include <memory>
#include <string>

#include "batch.hpp"
#include "blaslt.hpp"
#include "cache.hpp"
#include "device.hpp"
#include "weights.hpp"

namespace celeg {

enum class Epilogue : int { Store = 0, StoreF32 = 1, Residual = 2, Swiglu = 3, Conv = 4 };

// What follows a q/k/v product of many rows inside its kernel (heads of 64 columns): the norm of
// query and key heads, their rotation by the rows' positions, and the write of keys and values
// into the pages of the rows' requests; the query heads alone reach `out`.
struct QkvTail {
    int heads = 0, kv_heads = 0, head_dim = 0;
    const Tensor* q_weight = nullptr;      // [head_dim] 32-bit, or null: no norm
    const Tensor* k_weight = nullptr;
    float eps = 0.f;
    const Tensor* inv_freq = nullptr;      // [head_dim / 2], or null: no rotation
    const StepBatch* batch = nullptr;
    const KVView* kv = nullptr;
};

// A decode-only step's own keys and values as the q/k/v product left them, for an attention
// that normalises and turns q and the new keys itself and writes keys and values into the pages.
struct FreshKV {
    const Tensor* k = nullptr;             // [rows, kv_heads * head_dim]
    const Tensor* v = nullptr;
    const Tensor* q_weight = nullptr;      // [head_dim] 32-bit, or null: no norm
    const Tensor* k_weight = nullptr;
    float eps = 0.f;
    const Tensor* inv_freq = nullptr;      // [head_dim / 2], or null: no rotation
};

// The convolution epilogue's operands: one new token per request.
struct ConvOperands {
    Tensor taps;          // [N, L] 32-bit
    Tensor bias;          // optional [N]
    Tensor state;         // [slots, L, N] 32-bit, the slots a fixed number of elements apart
    const int* seq_slot = nullptr;   // [M]
};

struct FusedArgs {
    Epilogue epilogue = Epilogue::Store;
    Tensor norm_weight;           // the older form: the 32-bit stream normalised on the fly
    float eps = 0.f;
    Tensor stats;                 // partial sums of squares of the rows of the stream [rows, >= stat_blocks]
    int stat_blocks = 0;
    const int* rows = nullptr;    // picks rows of a
    int n_rows = -1;              // number of output rows (with rows: how many are picked)
    Tensor bias;
    Tensor stats_out;             // residual: partial sums of squares of the new rows
    const ConvOperands* conv = nullptr;
    Tensor out_bf16;              // residual: the bfloat16 copy of the stream
    bool packed = false;          // w is [K/32, rows, 32] (pack_weight)
    // 32-bit store of an output head: beside the logits, the best (logit, index) of every share of
    // columns [row_best_rows, row_best_ld >= parts]; Ops::last_best_parts then says how many parts
    // of every row were written
    unsigned long long* row_best = nullptr;
    int row_best_ld = 0, row_best_rows = 0;
};

// What an output head left beside its logits for greedy rows: the best (logit, index) of every
// share of a row's columns [rows, ld >= parts], for the first `rows` rows of `logits`.
struct HeadBest {
    const void* logits = nullptr;
    const unsigned long long* best = nullptr;
    int ld = 0, parts = 0, rows = 0;
    int cols = 0;        // columns a part stands for: part p is the best of columns p * cols .. + cols - 1
};

// What a step begins with, when the runner leaves it to the step's first kernel: the block-table
// updates of the (one) cache group and the rows whose token is on the device.
struct StepPrologue {
    int* table = nullptr;
    int stride = 0, n_slots = 0;
    const int* updates = nullptr;
    int capacity = 0;
    int* token_ids = nullptr;
    const int* token_slot = nullptr;
    const int* last_tokens = nullptr;
    int n = 0;
    bool pending = false;
};

// Which kernel a call was handed to (counted per Ops at the time of the launch, also while a
// graph records; a replay counts nothing): what tests and tools ask to see that a size took the
// path it was meant to take.
enum class Path : int {
    AttentionDecode = 0, AttentionDecodeFresh, AttentionRows, AttentionGeneral, LinearF32, LinearLibrary, LinearStandIn,
    FusedSliced, FusedRows, FusedStaged, Tiled, TiledQkv, ArgmaxMerged, Count
};
const char* path_name(Path p);

class Ops {
public:
    explicit Ops(hipStream_t stream) : stream(stream) {}
    hipStream_t stream;
    long long path_count[static_cast<int>(Path::Count)] = {};
    void took(Path p) { ++path_count[static_cast<int>(p)]; }
    Json paths_json() const;
    // knobs (tests and tuning)
    int attention_decode_whole = -1;     // -1: chosen from the batch; 0 split-key kernels; 1 one workgroup per request and key/value head
    bool use_blaslt = true;
    int attention_rows_per_tile = 0, attention_rows_form = 0;
    int decode_part_thresholds[2] = {64, 256};
    bool decode_parts_fill = true;       // parts of 16 rounds where they are one workgroup a compute unit
    int decode_split_rounds(long long groups, int rounds) const;
    bool decode_whole(long long groups, int rounds) const;
    bool attention_general = false;      // always the general attention kernel
    bool use_rope_table = true, use_argmax_parts = true, use_sliced = true, use_rows_kernel = true, use_tiles = true;
    bool use_qkv_tail = true;          // q/k/v products of many rows take norm, rotation and cache write along
    bool use_fresh_decode = true;      // decode-only steps: the attention prepares and writes the new keys and values
    bool use_head_argmax = true;       // greedy rows without a penalty: the token from what the head left beside the logits
    int rows_kernel_min_rows = 9, tiles_min_rows = 65, fused_linear_shape = 0;
    int last_stat_blocks = 0, last_best_parts = 0, last_best_cols = 0;

    // row-wise
    void embed(const Tensor& table, const int* token_ids, const Tensor& out);
    void rmsnorm(const Tensor& x, const Tensor& weight, float eps, const Tensor& out, const Tensor* delta = nullptr,
                 const int* rows = nullptr);
    void swiglu(const Tensor& gate_up, const Tensor& out);
    void add_bias(const Tensor& x, const Tensor& bias);
    void cast(const Tensor& src, const Tensor& dst);
    void apply_table_updates(int* table, int stride, int rows, const int* updates, int capacity);
    void step_prologue(int* table, int stride, int rows, const int* updates, int capacity, int* token_ids,
                       const int* token_slot, const int* last_tokens, int n);
    void resolve_tokens(int* token_ids, const int* token_slot, const int* last_tokens, int n);
    // products
    void linear(const Tensor& x, const Tensor& w, const Tensor& out, const Tensor* bias, Workspace& ws);
    // cache-backed
    void short_conv(const Tensor& bcx, const Tensor& weight, const Tensor* bias, const Tensor& state, const Tensor& out,
                    const StepBatch& batch);
    void qk_norm_rope_store(const Tensor& q, const Tensor* k, const Tensor* v, const Tensor* q_weight,
                            const Tensor* k_weight, float eps, const Tensor* inv_freq, int rotary_dim, int pairing, int heads,
                            int kv_heads, int head_dim, const StepBatch& batch, const KVView& kv);
    void paged_attention(const Tensor& q, const Tensor& out, int heads, int kv_heads, int head_dim, float scale,
                         int window, const StepBatch& batch, const KVView& kv, Workspace& ws, const FreshKV* fresh = nullptr);
    // whether a decode-only step's attention can prepare and write the step's own keys and values itself
    bool attention_fresh_ok(int heads, int head_dim, const Tensor* inv_freq, int rotary_dim, int pairing, const StepBatch& batch,
                            const KVView& kv, DType dtype) const;
    // sampling
    void sample(const Tensor& logits, const float* fparams, const int* iparams, uint8_t* seen,
                size_t seen_stride, int* out_tokens, int* last_tokens, bool all_greedy, Workspace& ws,
                const HeadBest* head_best = nullptr, bool penalised = false);
    // the most parts a row of an output head of n columns can have (for the caller's buffer): one
    // per 16 columns, or per 4 where the columns are few (narrow tiles, or less than a tile a workgroup)
    static int head_best_parts(long long n) { return static_cast<int>(std::max((n + 15) / 16, std::min<long long>((n + 3) / 4, 4096))); }
    void mark_seen(uint8_t* seen, size_t stride, int n_slots, int vocab, const int* token_ids, const int* token_slot, int n);
    // fused skinny products
    bool fused_linear_ok(int rows, std::initializer_list<long long> inner) const;
    bool rows_kernel_ok(int rows, std::initializer_list<long long> inner) const;
    int residual_stat_blocks(int rows, int n, int k) const;
    void stream_prepare(const Tensor& h, const Tensor& xb, const Tensor& stats);
    // (with `prologue`: the step's block-table updates and token ids from the device in the same launch)
    void embed_stream(const Tensor& table, const int* token_ids, const Tensor& out, const Tensor& xb, const Tensor& stats,
                      const StepPrologue* prologue = nullptr);
    void embed_stats(const Tensor& table, const int* token_ids, const Tensor& out, const Tensor& stats);
    void fused_linear(const Tensor& a, const Tensor& w, const Tensor& out, const FusedArgs& args);
    // fused products of many rows
    bool tiled_linear_ok(int rows, int n, std::initializer_list<long long> inner) const;
    int tiled_stat_blocks(int rows, int n, int k) const;
    void tiled_linear(const Tensor& a, const Tensor& w, const Tensor& out, Epilogue epilogue, float eps,
                      const Tensor* stats, int stat_blocks, const Tensor* bias, const Tensor* stats_out,
                      const Tensor* out_bf16, const QkvTail* qkv = nullptr);
    // whether the q/k/v product of many rows can take what follows it (norm, rotation, cache write) along
    bool tiled_qkv_ok(int head_dim, const Tensor* inv_freq, int rotary_dim, int pairing, const KVView& kv) const;
    // weights re-laid at load time: w [rows, K] scaled by a norm's weight (or not) and, if
    // `packed`, laid as [K/32, rows, 32]
    std::shared_ptr<DeviceTensor> fold_weight(const Tensor& w, const Tensor* scale, bool packed);
    // The tables of cosines and sines are kept by the address of their frequencies, which a model's
    // position encoding owns for as long as the dispatcher lives.  A caller whose frequency tensors
    // come and go (an address may then name other frequencies later) says so here: the tables made
    // for this address are set aside (not freed: a recorded graph may still read them) and made anew.
    void forget_rope_tables(const void* inv_freq);

private:
    std::unique_ptr<BlasLt> blaslt_;
    DeviceBuffer argmax_state_;
    std::map<std::pair<const void*, int>, std::shared_ptr<DeviceTensor>> rope_tables_;
    std::vector<std::shared_ptr<DeviceTensor>> retired_rope_tables_;
    const float* rope_table(const Tensor& inv_freq, int n_positions);
    void attention_decode(const Tensor& q, const Tensor& out, int heads, int kv_heads, int head_dim, float scale,
                          int window, const StepBatch& batch, const KVView& kv, int T, Workspace& ws, const FreshKV* fresh = nullptr);
    void library_product(const Tensor& x, const Tensor& w, const Tensor& out, Workspace& ws);
};

// What every part computes with: the stream, the activation dtype, the kernels, a workspace of
// reusable buffers, and what the parts of the fused path tell each other about the residual
// stream between kernels.
struct Runtime {
    Runtime(DType dtype, hipStream_t stream) : dtype(dtype), stream(stream), ops(stream) {}
    DType dtype;
    hipStream_t stream;
    Ops ops;
    Workspace ws;
    bool use_fused = true;
    // Steps of more than 64 bfloat16 rows: products that read a stream of up to this width go
    // through the tiled products with the norm, SwiGLU and residual sum folded in, wider ones
    // through the library's products with separate norm and activation kernels.  The default is
    // what was measured on whole prefills of 2,048 tokens: at a width of 1,024 the tiled path
    // takes 2.33 ms against 2.72 ms, at 2,048 the library's products run at 1.2 PFLOP/s and win
    // (5.5 against 6.2 ms and 9.3 against 11.0 ms for 16 and 30 layers).  0: always the library;
    // a large number: always the tiles.
    long long tiled_max_width = 1024;
    int fused_max_rows = -1;            // -1: by the kernels' own limits
    // how many partial sums of squares of the stream's rows are valid (0: none), and whether
    // the stream's bfloat16 copy is; whoever writes the stream another way resets them
    int stream_stat_blocks = 0;
    bool stream_has_bf16 = false;
    // the step's prologue, left by the runner for the embedding's kernel to take along
    // (defer_prologue); whoever cannot take it along calls flush_prologue() before its own work
    bool defer_prologue = true;
    // what the step's output head left for greedy rows (none: logits == nullptr); every forward
    // pass and every replay of a recorded one sets it anew
    HeadBest head_best;
    StepPrologue prologue;
    void flush_prologue() {
        if (!prologue.pending) return;
        prologue.pending = false;
        ops.step_prologue(prologue.table, prologue.stride, prologue.n_slots, prologue.updates, prologue.capacity,
                          prologue.token_ids, prologue.token_slot, prologue.last_tokens, prologue.n);
    }
    // weights re-laid for the fused path, made once per (weight, norm weight) pair
    std::map<std::pair<const void*, const void*>, std::shared_ptr<DeviceTensor>> folded_weights, folded_plain_weights;
    std::map<const void*, std::shared_ptr<DeviceTensor>> packed_weights;
    // a hook for bisecting mismatches: called after every entry of the run order with the
    // residual stream (the pending addition, if any, not yet made)
    std::function<void(int step, const Tensor& h, const Tensor* delta)> after_layer;
    // set: every step is timed phase by phase (and none is replayed from a recorded graph)
    std::unique_ptr<PhaseTimer> phases;
    void mark(const std::string& phase) {
        if (phases) phases->mark(phase);
    }
};

}  // namespace celeg
