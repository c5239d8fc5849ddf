#include "cache.hpp"

#include <algorithm>
#include <set>

namespace celeg {

// ---------------------------------------------------------------------------- pages
PagePool::PagePool(int n_pages, int page_tokens) : n_pages_(n_pages), page_tokens_(page_tokens) {
    if (n_pages < 0 || page_tokens <= 0)
        throw PageError("page pool: n_pages must be >= 0 and page_tokens positive");
    for (int p = n_pages - 1; p >= 0; --p) free_.push_back(p);     // pop_back() gives page 0 first
    holders_.assign(static_cast<size_t>(n_pages), 0);
}

int PagePool::pages_for(long long n_tokens) const {
    if (n_tokens < 0) throw PageError("token count must not be negative");
    return static_cast<int>((n_tokens + page_tokens_ - 1) / page_tokens_);
}

bool PagePool::allocate(int count, std::vector<int>& out) {
    if (count < 0) throw PageError("page count must not be negative");
    out.clear();
    if (count > n_free()) return false;
    for (int i = 0; i < count; ++i) {
        out.push_back(free_.back());
        free_.pop_back();
        holders_[static_cast<size_t>(out.back())] = 1;
    }
    return true;
}

void PagePool::retain(const std::vector<int>& pages) {
    for (int p : pages)
        if (p < 0 || p >= n_pages_ || holders_[static_cast<size_t>(p)] == 0)
            throw PageError("invalid page retain: " + std::to_string(p));
    for (int p : pages) ++holders_[static_cast<size_t>(p)];
}

void PagePool::release(const std::vector<int>& pages) {
    std::map<int, int> drops;
    for (int p : pages) ++drops[p];
    for (const auto& d : drops)
        if (d.first < 0 || d.first >= n_pages_ || holders_[static_cast<size_t>(d.first)] < d.second)
            throw PageError("invalid or double page release: " + std::to_string(d.first));
    for (int p : pages)
        if (--holders_[static_cast<size_t>(p)] == 0) free_.push_back(p);
}

void PagePool::check() const {
    std::set<int> free(free_.begin(), free_.end());
    if (free.size() != free_.size()) throw PageError("a page is on the free stack twice");
    for (int p = 0; p < n_pages_; ++p) {
        const bool on_stack = free.count(p) > 0;
        if (on_stack == (holders_[static_cast<size_t>(p)] > 0))
            throw PageError("page " + std::to_string(p) + (on_stack ? " is free and held" : " is lost"));
    }
}

// ---------------------------------------------------------------------------- layout
long long CacheLayout::kv_bytes_per_token(size_t itemsize) const {
    long long total = 0;
    for (size_t g = 0; g < kv_groups.size(); ++g)
        total += static_cast<long long>(group_layers[g]) * kv_groups[g].kv_heads * (kv_groups[g].head_dim + kv_groups[g].value_dim()) *
                 static_cast<long long>(itemsize);
    return total;
}

Json CacheLayout::to_json() const {
    Json groups = Json::array();
    for (size_t g = 0; g < kv_groups.size(); ++g)
        groups.push(Json::object().set("kv_heads", kv_groups[g].kv_heads).set("head_dim", kv_groups[g].head_dim)
                        .set("v_head_dim", kv_groups[g].value_dim())
                        .set("window", kv_groups[g].window ? Json(*kv_groups[g].window) : Json())
                        .set("layers", group_layers[g]));
    Json uses = Json::array();
    for (const auto& u : kv_of_step)
        uses.push(Json::object().set("step", u.first).set("group", u.second.group).set("layer", u.second.layer)
                      .set("writes", u.second.writes));
    Json st = Json::array();
    for (const auto& s : states)
        st.push(Json::object().set("step", s.first).set("name", s.second.name)
                    .set("shape", Json::array_of(s.second.shape)).set("dtype", dtype_name(s.second.dtype)));
    return Json::object().set("kv_groups", groups).set("kv_of_step", uses).set("states", st);
}

CacheLayout CacheLayout::from_json(const Json& j) {
    CacheLayout out;
    if (j["kv_groups"].is_array())
        for (const Json& g : j["kv_groups"].items()) {
            KVNeed need;
            need.kv_heads = static_cast<int>(g.get_int("kv_heads", 0));
            need.head_dim = static_cast<int>(g.get_int("head_dim", 0));
            need.v_head_dim = static_cast<int>(g.get_int("v_head_dim", 0));
            if (need.v_head_dim == need.head_dim) need.v_head_dim = 0;
            if (!g["window"].is_null()) need.window = static_cast<int>(g["window"].as_int());
            out.kv_groups.push_back(need);
            out.group_layers.push_back(static_cast<int>(g.get_int("layers", 1)));
        }
    if (j["kv_of_step"].is_array())
        for (const Json& u : j["kv_of_step"].items())
            out.kv_of_step[static_cast<int>(u.get_int("step", 0))] =
                KvUse{static_cast<int>(u.get_int("group", 0)), static_cast<int>(u.get_int("layer", 0)), u.get_bool("writes", true)};
    if (j["states"].is_array())
        for (const Json& s : j["states"].items()) {
            StateNeed need;
            need.name = s.get_string("name", "state");
            for (const Json& d : s["shape"].items()) need.shape.push_back(d.as_int());
            const std::string dt = s.get_string("dtype", "float32");
            need.dtype = dt == "int32" ? DType::I32 : dt == "uint8" ? DType::U8 : parse_dtype(dt);
            out.states.emplace_back(static_cast<int>(s.get_int("step", 0)), need);
        }
    return out;
}

// ---------------------------------------------------------------------------- manager
void CacheManager::Group::add_update(int slot, int logical, int page) {
    const auto key = std::make_pair(slot, logical);
    auto it = update_index.find(key);
    if (it != update_index.end()) {
        updates[it->second].second = page;
    } else {
        update_index[key] = updates.size();
        updates.push_back({key, page});
    }
}

CacheManager::CacheManager(CacheLayout layout_, int page_tokens_, std::vector<int> n_pages, int max_requests_,
                           int max_context_, DType dtype_, bool on_device, hipStream_t stream)
    : layout(std::move(layout_)), page_tokens(page_tokens_), max_requests(max_requests_), max_context(max_context_),
      null_slot(max_requests_), max_pages_per_request(page_tokens_ > 0 ? (max_context_ + page_tokens_ - 1) / page_tokens_ : 0),
      dtype(dtype_), on_device_(on_device), stream_(stream) {
    if (page_tokens <= 0 || max_requests <= 0 || max_context <= 0)
        throw PageError("cache manager: page_tokens, max_requests and max_context must be positive");
    if (n_pages.size() == 1 && layout.kv_groups.size() != 1) n_pages.assign(layout.kv_groups.size(), n_pages[0]);
    if (n_pages.size() != layout.kv_groups.size()) throw PageError("cache manager: one page count per group is needed");
    const size_t itemsize = dtype_size(dtype);
    for (size_t g = 0; g < layout.kv_groups.size(); ++g) {
        const KVNeed& need = layout.kv_groups[g];
        groups_.emplace_back(need, layout.group_layers[g], n_pages[g], page_tokens);
        Group& grp = groups_.back();
        grp.trash_page = n_pages[g];
        grp.table_host.assign(static_cast<size_t>(max_requests + 1) * max_pages_per_request, -1);
        for (int i = 0; i < max_pages_per_request; ++i)
            grp.table_host[static_cast<size_t>(max_requests) * max_pages_per_request + i] = grp.trash_page;
        grp.pages.assign(static_cast<size_t>(max_requests), {});
        grp.first_live.assign(static_cast<size_t>(max_requests), 0);
        if (on_device_) {
            const size_t per_dim = static_cast<size_t>(n_pages[g] + 1) * grp.n_layers * need.kv_heads * page_tokens * itemsize;
            grp.k = DeviceBuffer(per_dim * need.head_dim, true);
            grp.v = DeviceBuffer(per_dim * need.value_dim(), true);
            grp.table = DeviceBuffer(grp.table_host.size() * sizeof(int));
            CELEG_HIP(hipMemcpy(grp.table.ptr(), grp.table_host.data(), grp.table_host.size() * sizeof(int),
                                hipMemcpyHostToDevice));
        }
    }
    // state slots: one row of bytes per request (+ the null slot)
    size_t offset = 0;
    for (const auto& s : layout.states) {
        const auto key = std::make_pair(s.first, s.second.name);
        if (regions_.count(key))
            throw PageError("run-order entry " + std::to_string(s.first) + " declares state '" + s.second.name + "' twice");
        size_t count = 1;
        for (long long d : s.second.shape) count *= static_cast<size_t>(d);
        regions_[key] = Region{offset, s.second};
        offset += (count * dtype_size(s.second.dtype) + 15) / 16 * 16;
    }
    slot_bytes = offset;
    if (on_device_) state_buffer_ = DeviceBuffer(static_cast<size_t>(max_requests + 1) * std::max<size_t>(offset, 16), true);
    for (int s = max_requests - 1; s >= 0; --s) free_slots_.push_back(s);
}

std::vector<int> CacheManager::open_slots() const {
    std::vector<int> out;
    for (const auto& o : open_) out.push_back(o.first);
    return out;
}

int CacheManager::open() {
    if (free_slots_.empty()) return -1;
    const int slot = free_slots_.back();
    free_slots_.pop_back();
    open_[slot] = 0;
    if (slot_bytes && on_device_)
        CELEG_HIP(hipMemsetAsync(static_cast<char*>(state_buffer_.ptr()) + static_cast<size_t>(slot) * slot_bytes, 0,
                                 slot_bytes, stream_));
    return slot;
}

void CacheManager::close(int slot) {
    if (!open_.count(slot)) throw PageError("slot " + std::to_string(slot) + " is not open");
    for (Group& g : groups_) {
        auto& pages = g.pages[static_cast<size_t>(slot)];
        std::vector<int> live;
        for (int p : pages)
            if (p >= 0) live.push_back(p);
        g.pool.release(live);
        for (size_t idx = 0; idx < pages.size(); ++idx)
            if (pages[idx] >= 0) g.table_host[static_cast<size_t>(slot) * max_pages_per_request + idx] = -1;
        pages.clear();
        g.first_live[static_cast<size_t>(slot)] = 0;
    }
    open_.erase(slot);
    free_slots_.push_back(slot);
}

std::vector<int> CacheManager::pages_needed(int slot, int start_pos, int n_new) const {
    const int top = (start_pos + n_new - 1) / page_tokens;
    std::vector<int> out;
    for (const Group& g : groups_)
        out.push_back(std::max(0, top + 1 - static_cast<int>(g.pages[static_cast<size_t>(slot)].size())));
    return out;
}

void CacheManager::release_passed(Group& g, int slot, int next_pos) {
    const int lowest_needed = std::max(0, next_pos - *g.need.window + 1);
    const int first_needed_page = lowest_needed / page_tokens;
    auto& pages = g.pages[static_cast<size_t>(slot)];
    const int stop = std::min(first_needed_page, static_cast<int>(pages.size()));
    for (int idx = g.first_live[static_cast<size_t>(slot)]; idx < stop; ++idx)
        if (pages[static_cast<size_t>(idx)] >= 0) {
            g.pool.release({pages[static_cast<size_t>(idx)]});
            pages[static_cast<size_t>(idx)] = -1;
            g.table_host[static_cast<size_t>(slot) * max_pages_per_request + idx] = -1;
        }
    g.first_live[static_cast<size_t>(slot)] = std::max(g.first_live[static_cast<size_t>(slot)], stop);
}

bool CacheManager::prepare(int slot, int start_pos, int n_new) {
    if (!open_.count(slot)) throw PageError("slot " + std::to_string(slot) + " is not open");
    if (n_new <= 0 || start_pos < 0) throw PageError("prepare: n_new must be positive and start_pos >= 0");
    if (start_pos + n_new > max_context)
        throw StepError("context limit reached: " + std::to_string(start_pos + n_new) + " > " + std::to_string(max_context));
    for (Group& g : groups_)
        if (g.need.window) release_passed(g, slot, start_pos);
    const std::vector<int> need = pages_needed(slot, start_pos, n_new);
    for (size_t g = 0; g < groups_.size(); ++g)
        if (need[g] > groups_[g].pool.n_free()) return false;
    for (size_t gi = 0; gi < groups_.size(); ++gi) {
        Group& g = groups_[gi];
        std::vector<int> fresh;
        g.pool.allocate(need[gi], fresh);
        for (int p : fresh) {
            auto& pages = g.pages[static_cast<size_t>(slot)];
            const int idx = static_cast<int>(pages.size());
            pages.push_back(p);
            g.table_host[static_cast<size_t>(slot) * max_pages_per_request + idx] = p;
            g.add_update(slot, idx, p);
        }
    }
    open_[slot] = std::max(open_[slot], start_pos + n_new);
    return true;
}

bool CacheManager::covers(int slot, int start_pos, int n_new) const {
    if (!open_.count(slot)) return false;
    const int top = (start_pos + n_new - 1) / page_tokens;
    for (const Group& g : groups_) {
        const auto& pages = g.pages[static_cast<size_t>(slot)];
        if (top >= static_cast<int>(pages.size())) return false;
        const int low = g.need.window ? std::max(0, start_pos - *g.need.window + 1) : 0;
        for (int idx = low / page_tokens; idx <= top; ++idx)
            if (pages[static_cast<size_t>(idx)] < 0) return false;
    }
    return true;
}

std::vector<std::vector<int>> CacheManager::pages_held(int slot) const {
    std::vector<std::vector<int>> out;
    for (const Group& g : groups_) {
        out.emplace_back();
        for (int p : g.pages.at(static_cast<size_t>(slot)))
            if (p >= 0) out.back().push_back(p);
    }
    return out;
}

std::vector<int> CacheManager::free_pages() const {
    std::vector<int> out;
    for (const Group& g : groups_) out.push_back(g.pool.n_free());
    return out;
}

std::vector<std::vector<TableUpdate>> CacheManager::drain_table_updates() {
    std::vector<std::vector<TableUpdate>> out;
    for (Group& g : groups_) {
        out.emplace_back();
        for (const auto& u : g.updates) out.back().push_back({u.first.first, u.first.second, u.second});
        g.updates.clear();
        g.update_index.clear();
    }
    return out;
}

void CacheManager::requeue_table_updates(const std::vector<std::vector<TableUpdate>>& updates) {
    for (size_t gi = 0; gi < groups_.size() && gi < updates.size(); ++gi) {
        Group& g = groups_[gi];
        const auto fresh = g.updates;
        g.updates.clear();
        g.update_index.clear();
        for (const auto& u : updates[gi]) g.add_update(u.slot, u.logical, u.page);
        for (const auto& u : fresh) g.add_update(u.first.first, u.first.second, u.second);
    }
}

LayerCache CacheManager::layer_cache(int step) const {
    LayerCache out;
    auto it = layout.kv_of_step.find(step);
    if (it != layout.kv_of_step.end()) {
        const Group& g = groups_.at(static_cast<size_t>(it->second.group));
        KVView kv;
        kv.k = g.k.ptr();
        kv.v = g.v.ptr();
        kv.dtype = dtype;
        kv.layer = it->second.layer;
        kv.n_layers = g.n_layers;
        kv.table = g.table.as<int>();
        kv.table_stride = max_pages_per_request;
        kv.table_rows = max_requests + 1;
        kv.page_tokens = page_tokens;
        kv.kv_heads = g.need.kv_heads;
        kv.head_dim = g.need.head_dim;
        kv.v_head_dim = g.need.value_dim();
        kv.group = it->second.group;
        kv.n_pages = g.pool.n_pages() + 1;
        out.kv = kv;
        out.writes_kv = it->second.writes;
    }
    for (const auto& r : regions_) {
        if (r.first.first != step) continue;
        const StateNeed& need = r.second.need;
        Tensor t;
        t.data = state_buffer_.ptr() ? static_cast<char*>(state_buffer_.ptr()) + r.second.offset : nullptr;
        t.dtype = need.dtype;
        t.ndim = static_cast<int>(need.shape.size()) + 1;
        if (t.ndim > 4) throw PageError("state '" + need.name + "' has more than three dimensions");
        t.shape[0] = max_requests + 1;
        t.stride[0] = static_cast<long long>(slot_bytes / dtype_size(need.dtype));
        long long stride = 1;
        for (int i = t.ndim - 1; i >= 1; --i) {
            t.shape[i] = need.shape[static_cast<size_t>(i - 1)];
            t.stride[i] = stride;
            stride *= t.shape[i];
        }
        out.states[need.name] = t;
    }
    return out;
}

int CacheManager::table_host(int group, int slot, int logical) const {
    return groups_.at(static_cast<size_t>(group)).table_host.at(static_cast<size_t>(slot) * max_pages_per_request + logical);
}

void CacheManager::check() const {
    for (const Group& g : groups_) {
        g.pool.check();
        std::map<int, int> seen;
        for (int slot = 0; slot < max_requests; ++slot)
            for (int p : g.pages[static_cast<size_t>(slot)]) {
                if (p < 0) continue;
                if (!open_.count(slot))
                    throw PageError("closed slot " + std::to_string(slot) + " still holds page " + std::to_string(p));
                if (seen.count(p))
                    throw PageError("page " + std::to_string(p) + " is held by slots " + std::to_string(seen[p]) + " and " +
                                    std::to_string(slot));
                seen[p] = slot;
            }
        for (int p = 0; p < g.pool.n_pages(); ++p)
            if ((g.pool.holders(p) > 0) != (seen.count(p) > 0))
                throw PageError("page " + std::to_string(p) + ": pool and block tables disagree");
    }
    std::set<int> free(free_slots_.begin(), free_slots_.end());
    if (free.size() != free_slots_.size()) throw PageError("a slot is free twice");
    for (const auto& o : open_)
        if (free.count(o.first)) throw PageError("a slot is both free and open");
    if (static_cast<int>(free_slots_.size() + open_.size()) != max_requests) throw PageError("a slot is lost");
}

Json CacheManager::memory_bytes() const {
    long long kv = 0, tables = 0;
    for (const Group& g : groups_) {
        kv += static_cast<long long>(g.k.bytes() + g.v.bytes());
        tables += static_cast<long long>(g.table_host.size() * sizeof(int));
    }
    return Json::object().set("kv_cache", kv).set("state", static_cast<long long>(state_buffer_.bytes()))
        .set("block_tables", tables);
}

}  // namespace celeg
