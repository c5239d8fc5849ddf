// The host-side objects (page pool, cache manager, scheduler, batch builder) by themselves,
// without a GPU, driven by JSON calls: what the tests of the bookkeeping use where there is no
// device, and what a tool can use to replay a scheduling decision.
//
//   celeg_host_new(kind, args)  -> handle (0 on failure)
//   celeg_host_call(handle, method, args) -> JSON result (null on failure, celeg_last_error says why,
//                                            prefixed with the kind of error: "PageError: ...")
//   celeg_host_delete(handle)
//
// kinds and their constructor arguments:
//   "pool"      {"n_pages", "page_tokens"}
//   "cache"     {"layout": cache layout JSON, "page_tokens", "n_pages": n or [n per group], "max_requests", "max_context"}
//   "scheduler" {"cache": handle, "options": {..SchedulerOptions..}, "max_context", "default_eos": [..]}
//   "batch"     {"capacity", "n_groups"}
#include <algorithm>
#include <map>
#include <mutex>

#include "../include/celeg_amd.h"
#include "batch.hpp"
#include "cache.hpp"
#include "scheduler.hpp"

using namespace celeg;

namespace {
thread_local std::string g_host_text;

struct HostObject {
    std::string kind;
    std::unique_ptr<PagePool> pool;
    std::unique_ptr<CacheManager> cache;
    std::unique_ptr<Scheduler> scheduler;
    std::unique_ptr<BatchBuilder> batch;
    std::vector<PlannedEntry> last_plan;
};
std::map<long long, std::unique_ptr<HostObject>>& objects() {
    static std::map<long long, std::unique_ptr<HostObject>> o;
    return o;
}
std::mutex g_lock;
long long g_next = 1;

std::vector<int> ints(const Json& j) {
    std::vector<int> out;
    if (j.is_array())
        for (const Json& v : j.items()) out.push_back(static_cast<int>(v.as_int()));
    return out;
}

GenerationConfig generation_from(const Json& j) {
    GenerationConfig g;
    if (!j.is_object()) return g;
    g.temperature = static_cast<float>(j.get_double("temperature", g.temperature));
    g.top_k = static_cast<int>(j.get_int("top_k", g.top_k));
    g.top_p = static_cast<float>(j.get_double("top_p", g.top_p));
    g.repetition_penalty = static_cast<float>(j.get_double("repetition_penalty", g.repetition_penalty));
    g.seed = static_cast<uint64_t>(j.get_int("seed", 1));
    const Json& forced = j["forced_prefix"];
    if (forced.is_array())
        for (const Json& t : forced.items()) g.forced_prefix.push_back(static_cast<int>(t.as_int()));
    return g;
}

Json plan_json(const std::vector<PlannedEntry>& plan) {
    Json out = Json::array();
    for (const PlannedEntry& e : plan)
        out.push(Json::object().set("id", e.request->id).set("slot", e.request->slot).set("start", e.start)
                     .set("count", e.count).set("samples", e.samples).set("tokens", Json::array_of(e.request->tokens(e.start, e.count))));
    return out;
}

Json call(HostObject& o, const std::string& method, const Json& a) {
    if (o.kind == "pool") {
        PagePool& p = *o.pool;
        if (method == "allocate" || method == "allocate_tokens") {
            std::vector<int> pages;
            const bool ok = method == "allocate" ? p.allocate(static_cast<int>(a[0].as_int()), pages) : p.allocate_tokens(a[0].as_int(), pages);
            return ok ? Json::array_of(pages) : Json();
        }
        if (method == "retain") { p.retain(ints(a[0])); return Json(true); }
        if (method == "release") { p.release(ints(a[0])); return Json(true); }
        if (method == "check") { p.check(); return Json(true); }
        if (method == "state") {
            Json holders = Json::array();
            for (int i = 0; i < p.n_pages(); ++i) holders.push(Json(p.holders(i)));
            return Json::object().set("n_free", p.n_free()).set("n_used", p.n_used()).set("holders", holders);
        }
    } else if (o.kind == "cache") {
        CacheManager& c = *o.cache;
        if (method == "open") return Json(c.open());
        if (method == "close") { c.close(static_cast<int>(a[0].as_int())); return Json(true); }
        if (method == "prepare") return Json(c.prepare(static_cast<int>(a[0].as_int()), static_cast<int>(a[1].as_int()), static_cast<int>(a[2].as_int())));
        if (method == "covers") return Json(c.covers(static_cast<int>(a[0].as_int()), static_cast<int>(a[1].as_int()), static_cast<int>(a[2].as_int())));
        if (method == "pages_needed") return Json::array_of(c.pages_needed(static_cast<int>(a[0].as_int()), static_cast<int>(a[1].as_int()), static_cast<int>(a[2].as_int())));
        if (method == "check") { c.check(); return Json(true); }
        if (method == "pages_held") {
            Json out = Json::array();
            for (const auto& g : c.pages_held(static_cast<int>(a[0].as_int()))) out.push(Json::array_of(g));
            return out;
        }
        if (method == "table") return Json(c.table_host(static_cast<int>(a[0].as_int()), static_cast<int>(a[1].as_int()), static_cast<int>(a[2].as_int())));
        if (method == "drain" || method == "requeue") {
            if (method == "requeue") {
                std::vector<std::vector<TableUpdate>> updates;
                for (const Json& g : a[0].items()) {
                    updates.emplace_back();
                    for (const Json& u : g.items())
                        updates.back().push_back({static_cast<int>(u[0].as_int()), static_cast<int>(u[1].as_int()), static_cast<int>(u[2].as_int())});
                }
                c.requeue_table_updates(updates);
                return Json(true);
            }
            Json out = Json::array();
            for (const auto& g : c.drain_table_updates()) {
                Json group = Json::array();
                for (const TableUpdate& u : g) group.push(Json::array_of(std::vector<int>{u.slot, u.logical, u.page}));
                out.push(group);
            }
            return out;
        }
        if (method == "state") {
            Json regions = Json::object();
            for (size_t i = 0; i < c.layout.states.size(); ++i) {
                const LayerCache lc = c.layer_cache(c.layout.states[i].first);
                const Tensor& t = lc.states.at(c.layout.states[i].second.name);
                regions.set(std::to_string(c.layout.states[i].first) + ":" + c.layout.states[i].second.name,
                            Json::object().set("shape", Json::array_of(std::vector<long long>(t.shape, t.shape + t.ndim)))
                                .set("slot_stride", t.stride[0]).set("dtype", dtype_name(t.dtype))
                                .set("offset", static_cast<long long>(c.state_offset(c.layout.states[i].first, c.layout.states[i].second.name))));
            }
            return Json::object().set("free_slots", c.n_free_slots()).set("free_pages", Json::array_of(c.free_pages()))
                .set("open_slots", Json::array_of(c.open_slots())).set("null_slot", c.null_slot)
                .set("slot_bytes", static_cast<long long>(c.slot_bytes)).set("max_pages_per_request", c.max_pages_per_request)
                .set("n_groups", c.n_groups()).set("state_regions", regions);
        }
    } else if (o.kind == "scheduler") {
        Scheduler& s = *o.scheduler;
        if (method == "submit") {
            RequestOptions ro;
            const Json& opts = a[1];
            ro.max_new_tokens = static_cast<int>(opts.get_int("max_new_tokens", ro.max_new_tokens));
            ro.priority = static_cast<int>(opts.get_int("priority", 0));
            if (opts["eos_token_ids"].is_array()) ro.eos_token_ids = ints(opts["eos_token_ids"]);
            ro.generation = generation_from(opts["generation"]);
            return Json(s.submit(ints(a[0]), ro));
        }
        if (method == "cancel") { s.cancel(a[0].as_int()); return Json(true); }
        if (method == "release") {
            const long long id = a[0].as_int();
            const bool ended = is_done(s.request(id).status);
            if (ended)      // the plan kept for accept / fail must not name a record that goes
                o.last_plan.erase(std::remove_if(o.last_plan.begin(), o.last_plan.end(),
                                                 [&](const PlannedEntry& e) { return e.request->id == id; }),
                                  o.last_plan.end());
            return Json(s.release_request(id));
        }
        if (method == "has_work") return Json(s.has_work());
        if (method == "plan") {
            o.last_plan = s.plan();
            return plan_json(o.last_plan);
        }
        if (method == "accept") { s.accept(o.last_plan, ints(a[0])); return Json(true); }
        if (method == "fail") { s.fail(o.last_plan, a[0].as_string()); return Json(true); }
        if (method == "poll") {
            Request& r = s.request(a[0].as_int());
            Json tokens = Json::array();
            for (int t : r.pending) tokens.push(Json(t));
            r.pending.clear();
            return Json::object().set("status", status_name(r.status)).set("tokens", tokens).set("error", r.error);
        }
        if (method == "request") {
            Request& r = s.request(a[0].as_int());
            return Json::object().set("status", status_name(r.status)).set("slot", r.slot).set("fed", r.fed)
                .set("generated", Json::array_of(r.generated)).set("preemptions", r.preemptions).set("error", r.error)
                .set("ttft_seconds", r.ttft_seconds).set("itl_count", r.itl_count);
        }
        if (method == "slot_events") {
            std::vector<int> released;
            std::vector<std::pair<int, Request*>> bound;
            s.drain_slot_events(released, bound);
            Json b = Json::array();
            for (const auto& p : bound) b.push(Json::array_of(std::vector<long long>{p.first, p.second->id}));
            return Json::object().set("released", Json::array_of(released)).set("bound", b);
        }
        if (method == "stats") {
            Json st = s.stats();
            st.set("queued", static_cast<long long>(s.queue().size())).set("active", static_cast<long long>(s.active().size()));
            return st;
        }
    } else if (o.kind == "batch") {
        if (method == "build") {
            std::vector<StepEntry> entries;
            for (const Json& e : a[0].items()) {
                StepEntry se;
                se.slot = static_cast<int>(e.get_int("slot", 0));
                se.start_pos = static_cast<int>(e.get_int("start_pos", 0));
                se.tokens = ints(e["tokens"]);
                se.want = ints(e["want"]);
                entries.push_back(se);
            }
            std::vector<std::vector<TableUpdate>> updates;
            for (const Json& g : a[1].items()) {
                updates.emplace_back();
                for (const Json& u : g.items())
                    updates.back().push_back({static_cast<int>(u[0].as_int()), static_cast<int>(u[1].as_int()), static_cast<int>(u[2].as_int())});
            }
            BuildOptions options;
            const Json& opt = a[2];
            options.pad_to = static_cast<int>(opt.get_int("pad_to", -1));
            options.null_slot = static_cast<int>(opt.get_int("null_slot", 0));
            std::vector<int> caps = ints(opt["update_caps"]);
            if (opt["update_caps"].is_array()) options.update_caps = &caps;
            const StepBatch b = o.batch->build(entries, updates, options);
            auto arr = [](const int* p, int n) { return Json::array_of(std::vector<int>(p, p + n)); };
            Json ups = Json::array();
            for (size_t g = 0; g < b.table_updates.size(); ++g) ups.push(arr(b.table_updates[g], 1 + 3 * b.table_update_caps[g]));
            std::vector<long long> offsets;
            for (const int* p : {b.token_ids, b.positions, b.token_seq, b.token_slot, b.cu_seqlens, b.seq_slot, b.seq_start, b.logit_rows})
                offsets.push_back(p - o.batch->device_buffer());
            return Json::object().set("n_tokens", b.n_tokens).set("n_seqs", b.n_seqs).set("n_logit_rows", b.n_logit_rows)
                .set("decode_only", b.decode_only).set("single_rows", b.single_rows).set("entry_order", Json::array_of(b.entry_order))
                .set("max_context_len", b.max_context_len)
                .set("token_ids", arr(b.token_ids, b.n_tokens)).set("positions", arr(b.positions, b.n_tokens))
                .set("token_seq", arr(b.token_seq, b.n_tokens)).set("token_slot", arr(b.token_slot, b.n_tokens))
                .set("cu_seqlens", arr(b.cu_seqlens, b.n_seqs + 1)).set("seq_slot", arr(b.seq_slot, b.n_seqs))
                .set("seq_start", arr(b.seq_start, b.n_seqs)).set("logit_rows", arr(b.logit_rows, b.n_logit_rows))
                .set("table_updates", ups).set("offsets", Json::array_of(offsets));
        }
    }
    throw ConfigError("unknown method '" + method + "' of a " + o.kind);
}
}  // namespace

// (api.cpp owns the thread's last error; this hook writes it)
extern "C" void celeg_set_last_error_(const char* message);

extern "C" {

long long celeg_host_new(const char* kind, const char* args_json) {
    try {
        const Json a = Json::parse(args_json ? args_json : "{}");
        auto o = std::make_unique<HostObject>();
        o->kind = kind ? kind : "";
        if (o->kind == "pool") {
            o->pool = std::make_unique<PagePool>(static_cast<int>(a.get_int("n_pages", 0)), static_cast<int>(a.get_int("page_tokens", 16)));
        } else if (o->kind == "cache") {
            std::vector<int> pages = a["n_pages"].is_array() ? ints(a["n_pages"]) : std::vector<int>{static_cast<int>(a.get_int("n_pages", 0))};
            o->cache = std::make_unique<CacheManager>(CacheLayout::from_json(a["layout"]), static_cast<int>(a.get_int("page_tokens", 16)),
                                                      pages, static_cast<int>(a.get_int("max_requests", 1)),
                                                      static_cast<int>(a.get_int("max_context", 1)), DType::F32, false, nullptr);
        } else if (o->kind == "scheduler") {
            std::lock_guard<std::mutex> guard(g_lock);
            auto it = objects().find(a.get_int("cache", 0));
            if (it == objects().end() || !it->second->cache) throw ConfigError("scheduler: 'cache' is not the handle of a cache");
            SchedulerOptions so;
            const Json& opt = a["options"];
            so.max_active_requests = static_cast<int>(opt.get_int("max_active_requests", so.max_active_requests));
            so.max_batched_tokens = static_cast<int>(opt.get_int("max_batched_tokens", so.max_batched_tokens));
            so.prefill_chunk_tokens = static_cast<int>(opt.get_int("prefill_chunk_tokens", so.prefill_chunk_tokens));
            so.policy = opt.get_string("policy", so.policy);
            so.portion_granule = static_cast<int>(opt.get_int("portion_granule", 1));
            o->scheduler = std::make_unique<Scheduler>(*it->second->cache, so, static_cast<int>(a.get_int("max_context", 1)), ints(a["default_eos"]));
        } else if (o->kind == "batch") {
            o->batch = std::make_unique<BatchBuilder>(static_cast<size_t>(a.get_int("capacity", 1 << 16)), static_cast<int>(a.get_int("n_groups", 1)), false, nullptr);
        } else {
            throw ConfigError("unknown kind of host object '" + o->kind + "'");
        }
        std::lock_guard<std::mutex> guard(g_lock);
        const long long id = g_next++;
        objects()[id] = std::move(o);
        return id;
    } catch (const PageError& e) {
        celeg_set_last_error_((std::string("PageError: ") + e.what()).c_str());
    } catch (const ConfigError& e) {
        celeg_set_last_error_((std::string("ConfigError: ") + e.what()).c_str());
    } catch (const std::exception& e) {
        celeg_set_last_error_((std::string("Error: ") + e.what()).c_str());
    }
    return 0;
}

const char* celeg_host_call(long long handle, const char* method, const char* args_json) {
    try {
        HostObject* o = nullptr;
        {
            std::lock_guard<std::mutex> guard(g_lock);
            auto it = objects().find(handle);
            if (it == objects().end()) throw ConfigError("unknown handle");
            o = it->second.get();
        }
        const Json a = Json::parse(args_json ? args_json : "[]");
        g_host_text = call(*o, method ? method : "", a).dump();
        return g_host_text.c_str();
    } catch (const PageError& e) {
        celeg_set_last_error_((std::string("PageError: ") + e.what()).c_str());
    } catch (const ConfigError& e) {
        celeg_set_last_error_((std::string("ConfigError: ") + e.what()).c_str());
    } catch (const StepError& e) {
        celeg_set_last_error_((std::string("StepError: ") + e.what()).c_str());
    } catch (const std::exception& e) {
        celeg_set_last_error_((std::string("Error: ") + e.what()).c_str());
    }
    return nullptr;
}

void celeg_host_delete(long long handle) {
    std::lock_guard<std::mutex> guard(g_lock);
    objects().erase(handle);
}

}  // extern "C"
