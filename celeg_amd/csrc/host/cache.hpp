// The cache manager: pages of keys and values, block tables, and state slots.
//
// Layers are put into *groups* by what they need (KVNeed: heads, head size, all keys or a
// window of them).  Every group has its own page pool, its own K and V storage and its own
// block table per request; one page id of a group covers all the layers of that group.  The
// reference has one such group, for attention (include/celeg/runtime/cache/page_layout.hpp:14-142;
// src/backend/cuda/memory/paged_kv.cu:10-130), and keeps the short convolution's state per
// lane (include/celeg/detail/model/layer_state.hpp:180-187); here state of fixed size per
// request lives in *slots*: one row of one buffer per request, zeroed when the request
// starts, with a region for every layer that declared a need.
//
// Storage of a group: K [pages + 1, layers, kv_heads, page_tokens, head_dim] and V
// [pages + 1, layers, kv_heads, v_head_dim, page_tokens] (transposed inside a page: the layout
// the matrix-core attention kernel reads without shuffling).  The extra last page is never
// handed out: rows that pad a batch to a fixed size write there.  Likewise the last slot
// (null_slot) is never given to a request.
//
// Pages are given back when a request closes, and, in a window group, as soon as every
// position of a page lies before the window of the next token.
#pragma once
#include <map>
#include <optional>
#include <string>
#include <vector>

#include "batch.hpp"
#include "device.hpp"

namespace celeg {

// The page pool: which pages are free, who holds which.  Behaviour follows the reference's
// PagedBlockPool (src/runtime/concurrency/policy.cpp:21-120, pinned by
// tests/concurrent_policy_test.cpp:8-50): a LIFO free stack that hands out page 0 first, a
// count of holders per page, all-or-nothing allocation, `retain` that checks every id before
// it changes anything, and a transactional `release` that throws on an invalid or double release.
class PagePool {
public:
    PagePool(int n_pages, int page_tokens);
    int n_pages() const { return n_pages_; }
    int page_tokens() const { return page_tokens_; }
    int n_free() const { return static_cast<int>(free_.size()); }
    int n_used() const { return n_pages_ - n_free(); }
    int pages_for(long long n_tokens) const;
    // `count` pages, or false (and nothing taken) if fewer are free
    bool allocate(int count, std::vector<int>& out);
    bool allocate_tokens(long long n_tokens, std::vector<int>& out) { return allocate(pages_for(n_tokens), out); }
    void retain(const std::vector<int>& pages);
    void release(const std::vector<int>& pages);
    int holders(int page) const { return holders_.at(static_cast<size_t>(page)); }
    void check() const;    // every page is either free exactly once or held

private:
    int n_pages_, page_tokens_;
    std::vector<int> free_, holders_;
};

// Keys and values of every position, or of a trailing window of positions.  Values may have
// another width than keys (v_head_dim; 0: the keys').
struct KVNeed {
    int kv_heads = 0, head_dim = 0;
    std::optional<int> window;
    int v_head_dim = 0;
    int value_dim() const { return v_head_dim > 0 ? v_head_dim : head_dim; }
    bool operator==(const KVNeed& o) const {
        return kv_heads == o.kv_heads && head_dim == o.head_dim && window == o.window && value_dim() == o.value_dim();
    }
};

// State of fixed size per request, zero when the request starts.
struct StateNeed {
    std::string name;
    std::vector<long long> shape;
    DType dtype = DType::F32;
};

// What a model's run order needs.  kv_of_step[i] = (group, layer in group, writes) for the
// entries of the run order whose mixer uses keys and values; states lists (run-order entry, need).
struct CacheLayout {
    struct KvUse { int group, layer; bool writes; };
    std::vector<KVNeed> kv_groups;
    std::vector<int> group_layers;
    std::map<int, KvUse> kv_of_step;
    std::vector<std::pair<int, StateNeed>> states;
    long long kv_bytes_per_token(size_t itemsize) const;
    Json to_json() const;
    static CacheLayout from_json(const Json& j);
};

// What a mixer's kernels need to reach one layer's keys and values.
struct KVView {
    void* k = nullptr;
    void* v = nullptr;
    DType dtype = DType::F32;
    int layer = 0, n_layers = 0;
    int* table = nullptr;
    int table_stride = 0, table_rows = 0;
    int page_tokens = 0, kv_heads = 0, head_dim = 0, group = 0, n_pages = 0;
    int v_head_dim = 0;           // width of a value (the keys' unless the mixer asked for another)
};

// The cache of one entry of the run order.
struct LayerCache {
    std::optional<KVView> kv;
    bool writes_kv = false;
    std::map<std::string, Tensor> states;     // [slots + 1, shape...], the slots a row of bytes apart
};

class CacheManager {
public:
    // on_device false: the bookkeeping alone (pages, tables, slots), no GPU memory
    CacheManager(CacheLayout layout, int page_tokens, std::vector<int> n_pages, int max_requests, int max_context,
                 DType dtype, bool on_device, hipStream_t stream);

    const CacheLayout layout;
    const int page_tokens, max_requests, max_context, null_slot, max_pages_per_request;
    const DType dtype;
    size_t slot_bytes = 0;

    int n_groups() const { return static_cast<int>(groups_.size()); }
    int n_free_slots() const { return static_cast<int>(free_slots_.size()); }
    std::vector<int> open_slots() const;
    // a slot for a new request, its state zeroed; -1 if every slot is taken
    int open();
    void close(int slot);        // give back everything the request holds
    std::vector<int> pages_needed(int slot, int start_pos, int n_new) const;
    // Make the request's pages cover positions [start_pos, start_pos + n_new), after giving
    // back the pages that no later token can see (window groups).  False, with no page taken,
    // if some pool has too few free pages.
    bool prepare(int slot, int start_pos, int n_new);
    bool covers(int slot, int start_pos, int n_new) const;
    std::vector<std::vector<int>> pages_held(int slot) const;
    std::vector<int> free_pages() const;
    // Pages added to the block tables since the last call, per group, in order, at most one per
    // table entry.  The step function ships them to the device with the step's other metadata.
    // Entries of pages that were given back are not cleared on the device: no kernel reads a
    // table beyond the positions of its rows (the host copy does show -1 there).
    std::vector<std::vector<TableUpdate>> drain_table_updates();
    // put drained updates back (the step they were to travel with was refused); a newer
    // update of the same table entry wins
    void requeue_table_updates(const std::vector<std::vector<TableUpdate>>& updates);
    LayerCache layer_cache(int step) const;
    void check() const;          // no page lost, none held twice; slots free or open, never both
    Json memory_bytes() const;
    // where, inside a slot's row of bytes, the state `name` of run-order entry `step` lies
    size_t state_offset(int step, const std::string& name) const { return regions_.at({step, name}).offset; }
    int* device_table(int group) const { return groups_[static_cast<size_t>(group)].table.as<int>(); }
    int table_host(int group, int slot, int logical) const;
    int trash_page(int group) const { return groups_[static_cast<size_t>(group)].trash_page; }
    const PagePool& pool(int group) const { return groups_[static_cast<size_t>(group)].pool; }

private:
    struct Group {
        KVNeed need;
        int n_layers = 0;
        PagePool pool;
        DeviceBuffer k, v, table;
        int trash_page = 0;
        std::vector<int> table_host;                  // [slots + 1, max_pages_per_request]
        std::vector<std::vector<int>> pages;          // per slot: physical page of each logical page (-1 once given back)
        std::vector<int> first_live;
        std::vector<std::pair<std::pair<int, int>, int>> updates;   // ((slot, logical), page) in order
        std::map<std::pair<int, int>, size_t> update_index;
        Group(KVNeed n, int layers, int pages_, int page_tokens) : need(n), n_layers(layers), pool(pages_, page_tokens) {}
        void add_update(int slot, int logical, int page);
    };
    struct Region { size_t offset; StateNeed need; };
    void release_passed(Group& g, int slot, int next_pos);
    std::vector<Group> groups_;
    std::map<std::pair<int, std::string>, Region> regions_;
    DeviceBuffer state_buffer_;
    bool on_device_;
    hipStream_t stream_;
    std::vector<int> free_slots_;
    std::map<int, int> open_;       // slot -> tokens covered by pages so far
};

}  // namespace celeg
