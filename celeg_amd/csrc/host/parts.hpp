// Interfaces of the parts a model is put together from, and their registries.
//
// A part is built from a PartSpec (kind, sizes and constants, tensor names).  It never learns
// which model it is in: it declares the tensors it wants and the cache it needs, receives them,
// and maps rows to rows.
//
// Kinds of part and what each must provide:
//  * every part: weight_specs() (role -> WeightSpec) and load(tensors, rt);
//  * norm: forward(x, out, rt, delta, rows): normalises rows of the 32-bit residual stream,
//    optionally after adding delta to it in place, optionally only the rows listed in rows;
//  * mixer: kv_need() (keys and values that grow with the sequence, in pages) and state_needs()
//    (state of fixed size per request), and forward(x, batch, cache, rt) that gives the same
//    rows however the sequence was cut into steps;
//  * feed-forward: forward(x, batch, rt);
//  * position encoding: tables(rt), what the mixer's kernels need to turn a row's position into
//    its encoding;
//  * embedding and head: forward.
// Optional, for the few-rows path: forward_fused, which takes the norm in front of the part and
// the addition behind it into the part's own products and writes the stream itself.
#pragma once
#include <functional>
#include <map>
#include <memory>
#include <optional>
#include <string>
#include <vector>

#include "cache.hpp"
#include "ops.hpp"
#include "spec.hpp"
#include "weights.hpp"

namespace celeg {

using PartTensors = std::map<std::string, std::shared_ptr<DeviceTensor>>;   // role -> tensor
using WeightSpecs = std::vector<std::pair<std::string, WeightSpec>>;        // role -> what is wanted

class Part {
public:
    explicit Part(PartSpec s) : spec(std::move(s)) {}
    virtual ~Part() = default;
    const PartSpec spec;
    // True if forward only enqueues device work whose arguments do not depend on the step's
    // contents (every per-step number is read from the batch's device arrays), so that a
    // recorded step can be replayed from a HIP graph.  A part that plans on the host must leave
    // this false; a model with such a part is never replayed from a graph.
    virtual bool graph_safe() const { return false; }
    virtual WeightSpecs weight_specs() const { return {}; }
    virtual void load(const PartTensors& tensors, Runtime& rt) {}
    // parts nested inside this one (an attention's position encoding), for graph safety
    virtual std::vector<const Part*> children() const { return {}; }
};

class Norm : public Part {
public:
    using Part::Part;
    // out = norm(x [+ delta]).  With delta and no rows the sum is written back to x (the
    // residual stream); with rows only those rows are read and x is left alone.
    virtual void forward(const Tensor& x, const Tensor& out, Runtime& rt, const Tensor* delta, const int* rows) = 0;
    // An RMS norm's weight and eps if this is one whose work the fused products can take over
    // (the stream's bfloat16 copy times weights with the norm weight folded in, scaled by the
    // rows' 1/rms); nullptr otherwise.
    struct Foldable { Tensor weight; float eps; };
    virtual const Foldable* foldable() const { return nullptr; }
};

class PositionEncoding : public Part {
public:
    using Part::Part;
    // inv_freq undefined: no rotation.  Pair i of the first rotary_dim values of a head turns by
    // position * inv_freq[i]; pairing 0: the pair is (i, i + rotary_dim/2), 1: (2i, 2i + 1).
    struct Tables { Tensor inv_freq; int rotary_dim = 0; int pairing = 0; };
    virtual Tables tables(Runtime& rt) = 0;
};

class Mixer : public Part {
public:
    using Part::Part;
    virtual std::optional<KVNeed> kv_need() const { return std::nullopt; }
    virtual std::vector<StateNeed> state_needs() const { return {}; }
    // Called when a run-order entry makes this mixer read the keys and values another entry
    // wrote; a mixer that cannot do that refuses.
    virtual void set_reads_foreign_kv() { throw SpecError("mixer '" + spec.kind + "' cannot read another layer's cache"); }
    // x: normalised rows [T, width] in the run's dtype; returns the branch output [T, width]
    // (a workspace buffer, good until the part's next call)
    virtual Tensor forward(const Tensor& x, const StepBatch& batch, const LayerCache& cache, Runtime& rt) = 0;
    // h += mixer(norm(h)); false (nothing done) if this step cannot take the fused path
    virtual bool forward_fused(const Tensor& h, const Norm::Foldable& norm, const StepBatch& batch,
                               const LayerCache& cache, Runtime& rt) { return false; }
};

class FeedForward : public Part {
public:
    using Part::Part;
    virtual Tensor forward(const Tensor& x, const StepBatch& batch, Runtime& rt) = 0;
    virtual bool forward_fused(const Tensor& h, const Norm::Foldable& norm, const StepBatch& batch, Runtime& rt) { return false; }
};

class Embedding : public Part {
public:
    using Part::Part;
    virtual void forward(const int* token_ids, const Tensor& out, Runtime& rt, const StepBatch* batch) = 0;
    virtual Tensor table() const { return Tensor(); }     // what a tied head multiplies with
    // true: forward looks at rt.prologue itself (its kernel takes the step's prologue along, or
    // it calls rt.flush_prologue() first); false: the model runs the prologue before forward
    virtual bool takes_step_prologue() const { return false; }
};

class Head : public Part {
public:
    using Part::Part;
    virtual int vocab() const = 0;
    virtual void forward(const Tensor& x, const Tensor& out, Runtime& rt, const Embedding* embedding) = 0;
    virtual bool forward_fused(const Tensor& h, const Norm::Foldable& norm, const StepBatch& batch, const Tensor& out,
                               Runtime& rt, const Embedding* embedding) { return false; }
};

// The arrangement of a layer's parts.  forward takes h [T, width] 32-bit and delta, an addition
// to h not made yet (undefined: none), and returns the addition its last part leaves for the
// next norm (undefined: none).
class Block {
public:
    virtual ~Block() = default;
    virtual std::vector<std::pair<std::string, Part*>> parts() = 0;
    virtual Mixer& mixer() = 0;
    virtual Tensor forward(const Tensor& h, const Tensor& delta, const StepBatch& batch, const LayerCache& cache, Runtime& rt) = 0;
};

// ---------------------------------------------------------------------------- registries
using PartFactory = std::function<std::unique_ptr<Part>(const PartSpec&)>;
using BlockFactory = std::function<std::unique_ptr<Block>(const LayerSpec&)>;

// role: norm, mixer, ffn, position, embedding, head
void register_part(const std::string& role, const std::string& kind, PartFactory factory, bool replace = false);
void register_block(const std::string& arrangement, BlockFactory factory, bool replace = false);
std::unique_ptr<Part> build_part(const std::string& role, const PartSpec& spec);
std::unique_ptr<Block> build_block(const LayerSpec& layer);
std::vector<std::string> registered_parts(const std::string& role);

template <typename T>
std::unique_ptr<T> build_as(const std::string& role, const PartSpec& spec) {
    std::unique_ptr<Part> p = build_part(role, spec);
    T* typed = dynamic_cast<T*>(p.get());
    if (!typed) throw SpecError("part '" + spec.kind + "' is not a " + role);
    p.release();
    return std::unique_ptr<T>(typed);
}

// ---------------------------------------------------------------------------- the fused path's helpers
// A step of up to 64 rows is bound by the number of dependent kernels, so the parts fold their
// neighbours into their matrix products: the norm in front of a product is applied to the rows
// of the 32-bit residual stream as they are read, and a product that ends a sub-block adds its
// result into the stream itself.  Whoever writes the stream this way also leaves partial sums of
// squares of its rows ("stream statistics"), which the next norm reads instead of walking the
// rows again.  Runtime::stream_stat_blocks says how many partial sums are valid (0: none);
// anything else that writes the stream resets it to 0.
namespace fused {
constexpr int STAT_COLUMNS = 64;               // most rows of a fused step of few rows
constexpr int FUSED_MAX_ROWS = 64;             // where every inner size is a multiple of 32
constexpr int FUSED_MAX_ROWS_OLD_KERNEL = 32;  // else; above it the library's product is the faster one
constexpr int TILED_MAX_STAT_BLOCKS = 128;
constexpr int SLICED_MAX_ROWS = 16, SLICED_MAX_STAT_BLOCKS = 512, SLICED_MAX_COLUMNS = 16384;

bool tiled_step(const Runtime& rt, int rows, long long width);
bool fused_rows_ok(const Runtime& rt, const StepBatch& batch, std::initializer_list<long long> inner);
Tensor stream_stats(Runtime& rt, long long width, int rows = 0);
Tensor operand_rows(Runtime& rt, const std::string& name, int rows, long long width, std::initializer_list<long long> producer_inner);
Tensor stream_bf16(Runtime& rt, int rows, long long width);
bool sliced(const Runtime& rt, int rows, long long inner);

struct LinearExtras {
    const int* rows = nullptr;
    int n_rows = -1;
    Tensor bias;
    const ConvOperands* conv = nullptr;
    const QkvTail* qkv = nullptr;          // steps of many rows: what follows a q/k/v product, inside its kernel
    unsigned long long* row_best = nullptr;   // an output head's 32-bit store: see FusedArgs
    int row_best_ld = 0, row_best_rows = 0;
};
// whether norm_linear would take a q/k/v tail for a step of this many rows
bool qkv_tail_ok(const Runtime& rt, int rows, long long width);
// out = epilogue(norm(h) w^T), the norm applied while the rows of h are read
void norm_linear(Runtime& rt, const Tensor& h, const Norm::Foldable& norm, const Tensor& w, const Tensor& out,
                 Epilogue epilogue, const LinearExtras& extras = {});
// h += a w^T, leaving the partial sums of squares of the new rows (and, for few rows, the
// stream's bfloat16 copy)
void linear_into_stream(Runtime& rt, const Tensor& a, const Tensor& w, const Tensor& h, const Tensor* bias = nullptr);
}  // namespace fused

}  // namespace celeg
