// The description of a model as data: which parts, with which sizes, in which order.
//
// An architecture turns its typed configuration into a ModelSpec; everything below
// (weights, cache manager, step function) reads only the spec and never asks which
// architecture it came from.  The reference keeps the same separation: a LayerSpec is a
// mixer variant plus a feed-forward variant plus norms (include/celeg/model/graph.hpp:431-438)
// and back ends consume the compiled program, never names
// (src/model/program_builder.cpp:112-164).
//
// A spec also travels as JSON (an architecture defined outside this library hands its
// spec over that way):
//   part:  {"kind": .., "params": {..}, "tensors": {role: checkpoint name}}; a parameter
//          may itself be a part (an attention's "position")
//   layer: {"mixer": part, "mixer_norm": part, "ffn": part, "ffn_norm": part,
//           "arrangement": "pre_norm"}
//   model: {"architecture", "vocab_size", "hidden_size", "max_context", "embedding": part,
//           "layers": [layer], "order": [{"layer": i, "kv_from": j or null}],
//           "final_norm": part, "head": part, "eos_token_ids": [..], "bos_token_id"}
#pragma once
#include <map>
#include <optional>
#include <stdexcept>
#include <string>
#include <vector>

#include "json.hpp"

namespace celeg {

// One message per kind of failure; the C API hands the text to the caller.
struct ConfigError : std::runtime_error { using std::runtime_error::runtime_error; };
struct SpecError : std::runtime_error { using std::runtime_error::runtime_error; };
struct KernelError : std::runtime_error { using std::runtime_error::runtime_error; };
struct PageError : std::runtime_error { using std::runtime_error::runtime_error; };
struct StepError : std::runtime_error { using std::runtime_error::runtime_error; };

struct PartSpec {
    std::string kind;
    Json params = Json::object();
    std::vector<std::pair<std::string, std::string>> tensors;   // role -> checkpoint tensor name

    const std::string* tensor(const std::string& role) const {
        for (const auto& t : tensors)
            if (t.first == role) return &t.second;
        return nullptr;
    }

    Json to_json() const {
        Json t = Json::object();
        for (const auto& p : tensors) t.set(p.first, p.second);
        return Json::object().set("kind", kind).set("params", params).set("tensors", t);
    }
    static PartSpec from_json(const Json& j, const std::string& where) {
        if (!j.is_object() || !j["kind"].is_string())
            throw SpecError(where + ": a part is an object with a \"kind\"");
        PartSpec p;
        p.kind = j["kind"].as_string();
        if (!j["params"].is_null()) {
            if (!j["params"].is_object()) throw SpecError(where + ": \"params\" must be an object");
            p.params = j["params"];
        }
        if (!j["tensors"].is_null()) {
            if (!j["tensors"].is_object()) throw SpecError(where + ": \"tensors\" must be an object");
            for (const auto& m : j["tensors"].members()) {
                if (!m.second.is_string()) throw SpecError(where + ": tensor names are strings");
                p.tensors.emplace_back(m.first, m.second.as_string());
            }
        }
        return p;
    }
    // whether a parameter value is itself a part
    static bool is_part(const Json& v) { return v.is_object() && v["kind"].is_string(); }
};

struct LayerSpec {
    PartSpec mixer, mixer_norm, ffn, ffn_norm;
    std::string arrangement = "pre_norm";
};

// One entry of the run order.  `layer` indexes ModelSpec::layers (a layer may be named more
// than once: its weights are shared, its cache is not).  `kv_from` is the index of an
// EARLIER entry of the run order whose keys and values this entry's mixer reads instead of
// writing its own.
struct RunStep {
    int layer = 0;
    std::optional<int> kv_from;
};

struct ModelSpec {
    std::string architecture;
    int vocab_size = 0, hidden_size = 0, max_context = 0;
    PartSpec embedding;
    std::vector<LayerSpec> layers;
    std::vector<RunStep> order;
    PartSpec final_norm, head;
    std::vector<int> eos_token_ids;
    std::optional<int> bos_token_id;

    void validate() const {
        if (vocab_size <= 0 || hidden_size <= 0 || max_context <= 0)
            throw SpecError("vocab_size, hidden_size and max_context must be positive");
        if (order.empty()) throw SpecError("the run order is empty");
        for (size_t i = 0; i < order.size(); ++i) {
            if (order[i].layer < 0 || order[i].layer >= static_cast<int>(layers.size()))
                throw SpecError("run order entry " + std::to_string(i) + " names layer " +
                                std::to_string(order[i].layer) + ", but the model has " +
                                std::to_string(layers.size()) + " layers");
            if (order[i].kv_from && (*order[i].kv_from < 0 || *order[i].kv_from >= static_cast<int>(i)))
                throw SpecError("run order entry " + std::to_string(i) + " reads the cache of entry " +
                                std::to_string(*order[i].kv_from) + ", which does not run before it");
        }
    }

    Json to_json() const {
        Json ls = Json::array();
        for (const auto& l : layers)
            ls.push(Json::object().set("mixer", l.mixer.to_json()).set("mixer_norm", l.mixer_norm.to_json())
                        .set("ffn", l.ffn.to_json()).set("ffn_norm", l.ffn_norm.to_json())
                        .set("arrangement", l.arrangement));
        Json ord = Json::array();
        for (const auto& s : order)
            ord.push(Json::object().set("layer", s.layer).set("kv_from", s.kv_from ? Json(*s.kv_from) : Json()));
        return Json::object().set("architecture", architecture).set("vocab_size", vocab_size)
            .set("hidden_size", hidden_size).set("max_context", max_context)
            .set("embedding", embedding.to_json()).set("layers", ls).set("order", ord)
            .set("final_norm", final_norm.to_json()).set("head", head.to_json())
            .set("eos_token_ids", Json::array_of(eos_token_ids))
            .set("bos_token_id", bos_token_id ? Json(*bos_token_id) : Json());
    }

    static ModelSpec from_json(const Json& j) {
        if (!j.is_object()) throw SpecError("a model description is an object");
        ModelSpec m;
        m.architecture = j.get_string("architecture", "");
        m.vocab_size = static_cast<int>(j.get_int("vocab_size", 0));
        m.hidden_size = static_cast<int>(j.get_int("hidden_size", 0));
        m.max_context = static_cast<int>(j.get_int("max_context", 0));
        m.embedding = PartSpec::from_json(j["embedding"], "embedding");
        if (!j["layers"].is_array()) throw SpecError("\"layers\" must be an array");
        int n = 0;
        for (const Json& l : j["layers"].items()) {
            const std::string where = "layers[" + std::to_string(n++) + "]";
            LayerSpec ls;
            ls.mixer = PartSpec::from_json(l["mixer"], where + ".mixer");
            ls.mixer_norm = PartSpec::from_json(l["mixer_norm"], where + ".mixer_norm");
            ls.ffn = PartSpec::from_json(l["ffn"], where + ".ffn");
            ls.ffn_norm = PartSpec::from_json(l["ffn_norm"], where + ".ffn_norm");
            ls.arrangement = l.get_string("arrangement", "pre_norm");
            m.layers.push_back(std::move(ls));
        }
        if (j["order"].is_array()) {
            for (const Json& s : j["order"].items()) {
                RunStep step;
                step.layer = static_cast<int>(s.is_object() ? s.get_int("layer", -1) : s.as_int());
                if (s.is_object() && !s["kv_from"].is_null()) step.kv_from = static_cast<int>(s["kv_from"].as_int());
                m.order.push_back(step);
            }
        } else {
            for (size_t i = 0; i < m.layers.size(); ++i) m.order.push_back(RunStep{static_cast<int>(i), {}});
        }
        m.final_norm = PartSpec::from_json(j["final_norm"], "final_norm");
        m.head = PartSpec::from_json(j["head"], "head");
        if (j["eos_token_ids"].is_array())
            for (const Json& e : j["eos_token_ids"].items()) m.eos_token_ids.push_back(static_cast<int>(e.as_int()));
        if (!j["bos_token_id"].is_null()) m.bos_token_id = static_cast<int>(j["bos_token_id"].as_int());
        m.validate();
        return m;
    }
};

}  // namespace celeg
