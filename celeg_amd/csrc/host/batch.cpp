#include "batch.hpp"

#include <algorithm>
#include <numeric>

namespace celeg {

size_t packed_layout(int T, int S, int R, const std::vector<int>& update_caps, std::vector<PackedField>& fields) {
    fields.clear();
    size_t offset = 0;
    auto add = [&](const std::string& name, size_t count) {
        fields.push_back({name, offset, count});
        offset += (count + 3) / 4 * 4;
    };
    add("token_ids", static_cast<size_t>(T));
    add("positions", static_cast<size_t>(T));
    add("token_seq", static_cast<size_t>(T));
    add("token_slot", static_cast<size_t>(T));
    add("cu_seqlens", static_cast<size_t>(S) + 1);
    add("seq_slot", static_cast<size_t>(S));
    add("seq_start", static_cast<size_t>(S));
    add("logit_rows", static_cast<size_t>(R));
    for (size_t g = 0; g < update_caps.size(); ++g)
        add("updates" + std::to_string(g), 1 + 3 * static_cast<size_t>(update_caps[g]));
    return offset;
}

BatchBuilder::BatchBuilder(size_t capacity_ints, int n_groups, bool on_device, hipStream_t stream)
    : capacity(capacity_ints), n_groups_(n_groups), on_device_(on_device), stream_(stream) {
    for (auto& s : stage_) s = PinnedBuffer(capacity_ints * sizeof(int));
    if (on_device_) {
        device_owner_ = DeviceBuffer(capacity_ints * sizeof(int), true);
        device_ = device_owner_.as<int>();
        for (auto& e : events_) CELEG_HIP(hipEventCreateWithFlags(&e, hipEventDisableTiming));
    } else {
        host_device_.assign(capacity_ints, 0);
        device_ = host_device_.data();
    }
}

BatchBuilder::~BatchBuilder() {
    for (auto e : events_)
        if (e) (void)hipEventDestroy(e);
}

StepBatch BatchBuilder::build(const std::vector<StepEntry>& entries,
                              const std::vector<std::vector<TableUpdate>>& updates, const BuildOptions& opt) {
    const int S_real = static_cast<int>(entries.size());
    std::vector<int> seg_lens(entries.size());
    bool decode_only = true;
    long long total_rows = 0;
    for (size_t i = 0; i < entries.size(); ++i) {
        seg_lens[i] = static_cast<int>(entries[i].tokens.size());
        decode_only = decode_only && seg_lens[i] == 1;
        total_rows += seg_lens[i];
    }
    if (opt.pad_to >= 0 && (!decode_only || opt.pad_to < S_real))
        throw StepError("only batches of single rows can be padded, and only upwards");
    const int n_single = static_cast<int>(std::count(seg_lens.begin(), seg_lens.end(), 1));
    const int T_real = decode_only ? S_real : static_cast<int>(total_rows);
    const int S = opt.pad_to >= 0 ? opt.pad_to : S_real;
    const int T = opt.pad_to >= 0 ? opt.pad_to : T_real;
    // Rows are laid out with the entries of a single token first (their order kept), so that
    // kernels made for single rows can take them as one range also beside portions of prompts;
    // logits still come back in the order of the entries.
    std::vector<int> order(entries.size());
    std::iota(order.begin(), order.end(), 0);
    if (!decode_only)
        std::stable_sort(order.begin(), order.end(), [&](int a, int b) { return (seg_lens[a] != 1) < (seg_lens[b] != 1); });
    std::vector<int> want_rows;
    if (opt.pad_to >= 0) {
        want_rows.resize(static_cast<size_t>(T));
        std::iota(want_rows.begin(), want_rows.end(), 0);
    } else {
        std::vector<int> first_row(entries.size(), 0);
        int row = 0;
        for (int i : order) {
            first_row[static_cast<size_t>(i)] = row;
            row += seg_lens[static_cast<size_t>(i)];
        }
        for (size_t i = 0; i < entries.size(); ++i)
            for (int w : entries[i].want) {
                if (w < 0 || w >= seg_lens[i])
                    throw StepError("wanted place " + std::to_string(w) + " is outside the entry's " +
                                    std::to_string(seg_lens[i]) + " tokens");
                want_rows.push_back(first_row[i] + w);
            }
    }
    const int R = static_cast<int>(want_rows.size());
    std::vector<int> caps;
    if (opt.update_caps) {
        caps = *opt.update_caps;
    } else {
        for (const auto& u : updates) caps.push_back(static_cast<int>(u.size()));
    }
    if (caps.size() != updates.size() || static_cast<int>(updates.size()) != n_groups_)
        throw StepError("one list of block-table updates per cache group is needed");
    for (size_t g = 0; g < updates.size(); ++g)
        if (static_cast<int>(updates[g].size()) > caps[g])
            throw StepError("more block-table updates than the step has room for");
    std::vector<PackedField> fields;
    const size_t total = packed_layout(T, S, R, caps, fields);
    if (total > capacity)
        throw StepError("step metadata (" + std::to_string(total) + " ints) exceeds the staging buffer (" +
                        std::to_string(capacity) + " ints)");
    const int turn = turn_;
    turn_ ^= 1;
    if (pending_[turn]) {
        CELEG_HIP(hipEventSynchronize(events_[turn]));
        pending_[turn] = false;
    }
    int* stage = stage_[turn].as<int>();
    auto arr = [&](size_t f) { return stage + fields[f].offset; };
    int *token_ids = arr(0), *positions = arr(1), *token_seq = arr(2), *token_slot = arr(3);
    int *cu = arr(4), *seq_slot = arr(5), *seq_start = arr(6), *logit_rows = arr(7);
    if (decode_only) {
        for (int i = 0; i < S_real; ++i) {
            token_ids[i] = entries[static_cast<size_t>(i)].tokens[0];
            positions[i] = entries[static_cast<size_t>(i)].start_pos;
            token_slot[i] = entries[static_cast<size_t>(i)].slot;
        }
        for (int i = S_real; i < T; ++i) {
            token_ids[i] = 0;
            positions[i] = 0;
            token_slot[i] = opt.null_slot;
        }
        for (int i = 0; i < T; ++i) {
            token_seq[i] = i;
            seq_slot[i] = token_slot[i];
            seq_start[i] = positions[i];
        }
        for (int i = 0; i <= S; ++i) cu[i] = i;
    } else {
        int row = 0, seq = 0;
        cu[0] = 0;
        for (int j : order) {
            const StepEntry& e = entries[static_cast<size_t>(j)];
            const int n = seg_lens[static_cast<size_t>(j)];
            for (int t = 0; t < n; ++t) {
                token_ids[row + t] = e.tokens[static_cast<size_t>(t)];
                positions[row + t] = e.start_pos + t;
                token_seq[row + t] = seq;
                token_slot[row + t] = e.slot;
            }
            seq_slot[seq] = e.slot;
            seq_start[seq] = e.start_pos;
            row += n;
            cu[++seq] = row;
        }
    }
    std::copy(want_rows.begin(), want_rows.end(), logit_rows);
    for (size_t g = 0; g < updates.size(); ++g) {
        int* a = arr(8 + g);
        a[0] = static_cast<int>(updates[g].size());
        for (size_t i = 0; i < updates[g].size(); ++i) {
            a[1 + 3 * i] = updates[g][i].slot;
            a[2 + 3 * i] = updates[g][i].logical;
            a[3 + 3 * i] = updates[g][i].page;
        }
    }
    if (on_device_) {
        CELEG_HIP(hipMemcpyAsync(device_, stage, total * sizeof(int), hipMemcpyHostToDevice, stream_));
        CELEG_HIP(hipEventRecord(events_[turn], stream_));
        pending_[turn] = true;
    } else {
        std::copy(stage, stage + total, device_);
    }

    StepBatch b;
    b.n_tokens = T;
    b.n_seqs = S;
    b.n_logit_rows = R;
    b.n_real_seqs = S_real;
    b.decode_only = decode_only;
    b.single_rows = decode_only ? S : n_single;
    b.entry_order = order;
    for (size_t i = 0; i < entries.size(); ++i) {
        b.max_seg_len = std::max(b.max_seg_len, seg_lens[i]);
        b.max_context_len = std::max(b.max_context_len, entries[i].start_pos + seg_lens[i]);
    }
    auto dev = [&](size_t f) { return device_ + fields[f].offset; };
    b.token_ids = dev(0);
    b.positions = dev(1);
    b.token_seq = dev(2);
    b.token_slot = dev(3);
    b.cu_seqlens = dev(4);
    b.seq_slot = dev(5);
    b.seq_start = dev(6);
    b.logit_rows = dev(7);
    for (size_t g = 0; g < updates.size(); ++g) b.table_updates.push_back(dev(8 + g));
    b.table_update_caps = caps;
    for (int j : order) b.host_seg_lens.push_back(seg_lens[static_cast<size_t>(j)]);
    b.host_seg_lens.resize(static_cast<size_t>(S), 1);
    b.host_seq_slot.assign(seq_slot, seq_slot + S);
    b.host_seq_start.assign(seq_start, seq_start + S);
    b.host_cu_seqlens.assign(cu, cu + S + 1);
    b.host_want_rows = want_rows;
    return b;
}

}  // namespace celeg
