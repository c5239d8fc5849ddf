// One step's batch: the rows, and the per-row and per-request numbers kernels need.
//
// A step takes a list of entries, one per request: the request's next tokens (a portion of
// its prompt, or one decoded token) and the places among them whose logits are wanted.  The
// tokens of all entries are laid side by side into T rows.  The reference builds the same
// arrays for its packed passes, separately for a prefill pass and a decode pass
// (src/backend/cuda/packed/batch_planner.cu:38-87); here one batch holds both kinds.
//
// All integer metadata travels to the device in ONE copy of one packed buffer.
#pragma once
#include <hip/hip_runtime_api.h>

#include <string>
#include <utility>
#include <vector>

#include "device.hpp"

namespace celeg {

constexpr int TOKEN_FROM_DEVICE = -1;   // a single-token entry whose token the device supplies

struct StepEntry {
    int slot = 0;                 // the request's slot in the cache manager
    int start_pos = 0;            // position of tokens[0] in the request's sequence
    std::vector<int> tokens;      // {TOKEN_FROM_DEVICE}: the token the request sampled last, taken on the device
    std::vector<int> want;        // indices into tokens whose logits are wanted
};

// (slot, logical page, physical page)
struct TableUpdate {
    int slot, logical, page;
};

// Device views (int32) into the packed buffer, plus host-side facts.
// token_ids[T], positions[T], token_seq[T] (which sequence a row belongs to), token_slot[T]
// (that entry's cache slot), cu_seqlens[S+1] (row offsets of the sequences), seq_slot[S],
// seq_start[S] (position of the sequence's first row), the sequences being the entries with
// those of a single token moved to the front, logit_rows[R] (rows whose logits are wanted),
// table_updates[g] ([1 + 3*cap]: a count, then (slot, logical page, physical page) triples)
// per cache group.
struct StepBatch {
    int n_tokens = 0, n_seqs = 0, n_logit_rows = 0, n_real_seqs = 0;
    int max_seg_len = 0, max_context_len = 0;
    int context_bound = 0;      // set by whoever records the step for replay: the longest context the recording must serve
    bool decode_only = false;
    int single_rows = 0;        // rows [0, single_rows) are entries of one token each
    std::vector<int> entry_order;          // which entry each sequence of the layout is
    int *token_ids = nullptr, *positions = nullptr, *token_seq = nullptr, *token_slot = nullptr;
    int *cu_seqlens = nullptr, *seq_slot = nullptr, *seq_start = nullptr, *logit_rows = nullptr;
    std::vector<int*> table_updates;
    std::vector<int> table_update_caps;
    // host copies, for parts that plan on the host
    std::vector<int> host_seg_lens, host_seq_slot, host_seq_start, host_cu_seqlens, host_want_rows;

    int context_hint() const { return context_bound ? context_bound : max_context_len; }
};

struct PackedField {
    std::string name;
    size_t offset, count;
};
// Offsets (in int32 elements) of every array in the packed buffer; each array starts at a
// multiple of 4 elements.  The layout depends only on the counts, so a recorded graph of a
// fixed (T, S, R, caps) always finds its arrays in place.  Returns the total.
size_t packed_layout(int T, int S, int R, const std::vector<int>& update_caps, std::vector<PackedField>& fields);

struct BuildOptions {
    int pad_to = -1;             // batches of single rows: the fixed number of rows of a recorded graph
    int null_slot = 0;
    const std::vector<int>* update_caps = nullptr;
};

// Packs entries on the host and ships them with one copy.  Two pinned staging buffers take
// turns, each guarded by an event, so a step's arrays are never overwritten while their copy
// is still in flight.
class BatchBuilder {
public:
    // on_device false: no GPU is touched; the "device" arrays are ordinary host memory (what
    // host-only tests of the layout read back)
    BatchBuilder(size_t capacity_ints, int n_groups, bool on_device, hipStream_t stream);
    ~BatchBuilder();
    BatchBuilder(const BatchBuilder&) = delete;
    StepBatch build(const std::vector<StepEntry>& entries, const std::vector<std::vector<TableUpdate>>& updates,
                    const BuildOptions& options);
    size_t capacity;
    int* device_buffer() const { return device_; }

private:
    int n_groups_;
    bool on_device_;
    hipStream_t stream_;
    PinnedBuffer stage_[2];
    hipEvent_t events_[2] = {nullptr, nullptr};
    bool pending_[2] = {false, false};
    int turn_ = 0;
    DeviceBuffer device_owner_;
    std::vector<int> host_device_;     // stands in for the device buffer when there is no GPU
    int* device_ = nullptr;
};

}  // namespace celeg
