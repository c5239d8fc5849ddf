// The architecture registry, reading config.json, and the LFM2 dense configuration.
//
// The reference has no class for this architecture: it recognises the layers from tensor
// names (src/model/inference/rules.cpp:12-90 for the short convolution,
// src/model/inference/rules_attention.cpp:138-345 for attention) and reads the scalar keys
// through its metadata normaliser (src/model/inference/metadata.cpp:350-703).  Here every
// size comes from config.json; nothing about a particular checkpoint stands in code.
#include "config.hpp"

#include <cmath>
#include <fstream>
#include <mutex>
#include <set>
#include <sstream>

namespace celeg {

namespace {
std::map<std::string, Architecture>& table() {
    static std::map<std::string, Architecture> t;
    return t;
}
std::mutex& table_lock() {
    static std::mutex m;
    return m;
}
void register_builtin();
void ensure_builtin() {
    static std::once_flag once;
    std::call_once(once, register_builtin);
}
std::string list_of(const std::vector<std::string>& names) {
    std::string out = "[";
    for (size_t i = 0; i < names.size(); ++i) out += (i ? ", '" : "'") + names[i] + "'";
    return out + "]";
}
}  // namespace

void register_architecture(Architecture arch, bool replace) {
    ensure_builtin();
    std::lock_guard<std::mutex> guard(table_lock());
    std::vector<std::string> names{arch.name};
    names.insert(names.end(), arch.aliases.begin(), arch.aliases.end());
    for (const auto& n : names)
        if (table().count(n) && !replace) throw SpecError("architecture '" + n + "' is already registered");
    for (const auto& n : names) table()[n] = arch;
}

std::vector<std::string> registered_architectures() {
    ensure_builtin();
    std::lock_guard<std::mutex> guard(table_lock());
    std::vector<std::string> out;
    for (const auto& e : table()) out.push_back(e.first);
    return out;
}

std::string architecture_name(const Json& config) {
    const Json& archs = config["architectures"];
    if (archs.is_array() && archs.size() > 0 && archs[0].is_string()) return archs[0].as_string();
    if (config["model_type"].is_string()) return config["model_type"].as_string();
    throw ConfigError("config.json names no architecture: neither 'architectures' nor 'model_type' is present");
}

const Architecture& find_architecture(const Json& config) {
    ensure_builtin();
    const std::string name = architecture_name(config);
    {
        std::lock_guard<std::mutex> guard(table_lock());
        auto it = table().find(name);
        if (it != table().end()) return it->second;
    }
    throw ConfigError("no registered architecture is called '" + name + "'; registered: " +
                      list_of(registered_architectures()));
}

static bool read_text(const std::string& path, std::string& out) {
    std::ifstream in(path, std::ios::binary);
    if (!in) return false;
    std::ostringstream ss;
    ss << in.rdbuf();
    out = ss.str();
    return true;
}

Json read_config_file(const std::string& model_dir) {
    std::string text;
    const std::string path = model_dir + "/config.json";
    if (!read_text(path, text)) throw ConfigError("config.json not found in model folder " + model_dir);
    Json config;
    try {
        config = Json::parse(text);
    } catch (const JsonError& e) {
        throw ConfigError("config.json in " + model_dir + " cannot be read: " + e.what());
    }
    if (!config.is_object()) throw ConfigError("config.json in " + model_dir + " is not an object");
    std::string gen_text;
    if (read_text(model_dir + "/generation_config.json", gen_text)) {
        try {
            const Json gen = Json::parse(gen_text);
            for (const char* key : {"bos_token_id", "eos_token_id"}) {
                const Json& v = gen[key];
                if (v.is_number()) {
                    config.set(key, Json(v.as_int()));
                } else if (v.is_array()) {
                    Json ids = Json::array();
                    for (const Json& item : v.items())
                        if (item.is_number()) ids.push(Json(item.as_int()));
                    if (ids.size() > 0) config.set(key, ids);
                }
            }
        } catch (const JsonError&) {
            // unreadable: ignored, as the reference does
        }
    }
    return config;
}

Described describe_config(const Json& config, const TensorShapes* shapes) {
    const Architecture& arch = find_architecture(config);
    Described d;
    d.config = arch.read_config(config, shapes);
    d.spec = arch.build_spec(d.config);
    d.spec.validate();
    return d;
}

// ---------------------------------------------------------------------------- LFM2 dense
namespace {

std::string repr(const Json& v) { return v.dump(); }

long long typed_int(const Json& cfg, const std::string& key) {
    const Json& v = cfg[key];
    if (v.is_int()) return v.as_int();
    if (v.kind() == Json::Float && std::floor(v.as_double()) == v.as_double()) return v.as_int();
    throw ConfigError("config.json: '" + key + "' must be an integer, got " + repr(v));
}
double typed_float(const Json& cfg, const std::string& key) {
    const Json& v = cfg[key];
    if (!v.is_number()) throw ConfigError("config.json: '" + key + "' must be a number, got " + repr(v));
    return v.as_double();
}
bool typed_bool(const Json& cfg, const std::string& key) {
    const Json& v = cfg[key];
    if (!v.is_bool()) throw ConfigError("config.json: '" + key + "' must be true or false, got " + repr(v));
    return v.as_bool();
}
bool present(const Json& cfg, const std::string& key) { return !cfg[key].is_null(); }

long long require_int(const Json& cfg, const std::string& key) {
    if (!present(cfg, key)) throw ConfigError("config.json: required key '" + key + "' is missing");
    return typed_int(cfg, key);
}

// First present alias wins; two aliases that disagree are an error, as in the reference
// (src/model/inference/metadata.cpp:350-703 raises ConflictingMetadata).
template <typename T, typename Read>
bool alias(const Json& cfg, const std::vector<std::string>& keys, Read read, T& out) {
    bool found = false;
    std::string first_key;
    for (const auto& k : keys) {
        if (!present(cfg, k)) continue;
        const T v = read(cfg, k);
        if (!found) {
            out = v;
            found = true;
            first_key = k;
        } else if (!(v == out)) {
            throw ConfigError("config.json: '" + first_key + "'=" + repr(cfg[first_key]) + " and '" + k + "'=" +
                              repr(cfg[k]) + " disagree");
        }
    }
    return found;
}

const char* const LAYER_KINDS[] = {"conv", "full_attention"};
bool known_kind(const std::string& k) { return k == LAYER_KINDS[0] || k == LAYER_KINDS[1]; }

// layer_types if given; else from full_attn_idxs; else from the tensors each layer has
// (src/model/inference/rules.cpp:18-26, rules_attention.cpp:138-160).  Whatever the source,
// tensors that say otherwise are an error.
std::vector<std::string> layer_kinds(const Json& cfg, long long layers, const TensorShapes* shapes) {
    std::vector<std::string> from_tensors;     // "" where the tensors tell nothing
    if (shapes) {
        for (long long i = 0; i < layers; ++i) {
            const std::string p = "model.layers." + std::to_string(i) + ".";
            const bool conv = shapes->count(p + "conv.in_proj.weight") > 0;
            const bool attn = shapes->count(p + "self_attn.q_proj.weight") > 0;
            from_tensors.push_back(conv && !attn ? "conv" : attn && !conv ? "full_attention" : "");
        }
    }
    std::vector<std::string> kinds;
    if (present(cfg, "layer_types")) {
        const Json& v = cfg["layer_types"];
        bool ok = v.is_array();
        if (ok)
            for (const Json& k : v.items()) ok = ok && k.is_string();
        if (!ok) throw ConfigError("config.json: 'layer_types' must be a list of strings");
        for (const Json& k : v.items()) kinds.push_back(k.as_string());
    } else if (present(cfg, "full_attn_idxs")) {
        const Json& v = cfg["full_attn_idxs"];
        bool ok = v.is_array();
        if (ok)
            for (const Json& k : v.items()) ok = ok && k.is_int();
        if (!ok) throw ConfigError("config.json: 'full_attn_idxs' must be a list of integers");
        std::set<long long> idxs;
        for (const Json& k : v.items()) {
            if (k.as_int() < 0 || k.as_int() >= layers)
                throw ConfigError("config.json: 'full_attn_idxs' names a layer outside [0, " + std::to_string(layers) + ")");
            idxs.insert(k.as_int());
        }
        for (long long i = 0; i < layers; ++i) kinds.push_back(idxs.count(i) ? "full_attention" : "conv");
    } else if (shapes) {
        std::string unknown;
        for (size_t i = 0; i < from_tensors.size(); ++i)
            if (from_tensors[i].empty()) unknown += (unknown.empty() ? "" : ", ") + std::to_string(i);
        if (!unknown.empty())
            throw ConfigError("config.json has no 'layer_types' and the tensors of layer(s) [" + unknown +
                              "] tell neither a convolution nor an attention layer");
        return from_tensors;
    } else {
        throw ConfigError("config.json: required key 'layer_types' is missing");
    }
    if (shapes && static_cast<long long>(kinds.size()) == layers) {
        for (size_t i = 0; i < kinds.size(); ++i)
            if (!from_tensors[i].empty() && known_kind(kinds[i]) && kinds[i] != from_tensors[i])
                throw ConfigError("config.json: 'layer_types'[" + std::to_string(i) + "] is '" + kinds[i] +
                                  "' but the checkpoint's tensors of layer " + std::to_string(i) + " are those of '" +
                                  from_tensors[i] + "'");
    }
    return kinds;
}

// Keys and defaults follow src/model/inference/metadata.cpp: hidden_size (353),
// intermediate_size (355-357), num_hidden_layers (358-360), num_attention_heads (364-366),
// num_key_value_heads (367-369), head_dim (370), vocab_size (399), max_position_embeddings
// (404-406), norm_eps (407-409, default 1e-6 at 643), conv_L_cache (425-426), rope_theta
// (427-429: also as rope_parameters.rope_theta; required 663-666), block_auto_adjust_ff_dim
// (512-514), tying (630-632), token ids (638-642).  The original LFM2 keys full_attn_idxs
// (the attention layers; every other layer is a convolution) and block_ff_dim
// (= intermediate_size) are read too.  With the checkpoint's tensor shapes at hand, what
// config.json leaves out is filled the way the reference does: layer kinds from the tensors
// each layer has, the feed-forward width from the rows of w1 (global_facts.cpp:127-152).
Json lfm2_read_config(const Json& raw, const TensorShapes* shapes) {
    if (!raw.is_object()) throw ConfigError("config.json is not an object");
    Json cfg = raw;
    const Json& nested = raw["rope_parameters"];
    if (nested.is_object() && !nested["rope_theta"].is_null())
        cfg.set("rope_parameters.rope_theta", nested["rope_theta"]);
    const long long vocab = require_int(cfg, "vocab_size");
    const long long hidden = require_int(cfg, "hidden_size");
    const long long layers = require_int(cfg, "num_hidden_layers");
    const long long heads = require_int(cfg, "num_attention_heads");
    long long kv_heads = heads;
    alias<long long>(cfg, {"num_key_value_heads"}, typed_int, kv_heads);
    long long head_dim = heads > 0 ? hidden / heads : 0;
    alias<long long>(cfg, {"head_dim"}, typed_int, head_dim);
    double rope_theta = 0;
    if (!alias<double>(cfg, {"rope_theta", "rope_parameters.rope_theta"}, typed_float, rope_theta))
        throw ConfigError("config.json: required key 'rope_theta' is missing");
    const long long conv_l = require_int(cfg, "conv_L_cache");
    const long long max_pos = require_int(cfg, "max_position_embeddings");
    bool auto_adjust = false;
    alias<bool>(cfg, {"block_auto_adjust_ff_dim"}, typed_bool, auto_adjust);
    long long intermediate = 0;
    const bool has_intermediate = alias<long long>(cfg, {"intermediate_size", "block_ff_dim"}, typed_int, intermediate);
    const std::vector<std::string> kinds = layer_kinds(cfg, layers, shapes);
    if (!has_intermediate) {
        const auto w1 = shapes ? shapes->find("model.layers.0.feed_forward.w1.weight") : TensorShapes::const_iterator{};
        if (!shapes || w1 == shapes->end() || w1->second.empty())
            throw ConfigError("config.json: required key 'intermediate_size' is missing");
        // the width itself: no adjustment is applied to a size read off the weights
        intermediate = w1->second[0];
        auto_adjust = false;
    }
    Json eos = Json::array();
    if (raw["eos_token_id"].is_array()) {
        for (const Json& e : raw["eos_token_id"].items()) eos.push(Json(e.as_int()));
    } else {
        eos.push(Json(raw["eos_token_id"].is_null() ? 0LL : typed_int(cfg, "eos_token_id")));
    }
    Json multiplier = Json(1.0);
    if (raw.contains("block_ffn_dim_multiplier"))
        multiplier = raw["block_ffn_dim_multiplier"].is_null() ? Json() : Json(typed_float(cfg, "block_ffn_dim_multiplier"));
    bool conv_bias = false, tie = true;
    alias<bool>(cfg, {"conv_bias"}, typed_bool, conv_bias);
    alias<bool>(cfg, {"tie_word_embeddings", "tie_embedding"}, typed_bool, tie);
    double norm_eps = 1e-6;
    alias<double>(cfg, {"norm_eps", "rms_norm_eps"}, typed_float, norm_eps);
    long long multiple_of = 256, bos = 0, pad = 1;
    alias<long long>(cfg, {"block_multiple_of"}, typed_int, multiple_of);
    alias<long long>(cfg, {"bos_token_id"}, typed_int, bos);
    alias<long long>(cfg, {"pad_token_id"}, typed_int, pad);

    Json out = Json::object();
    out.set("architectures", Json::array_of(std::vector<std::string>{"Lfm2ForCausalLM"})).set("model_type", "lfm2")
        .set("vocab_size", vocab).set("hidden_size", hidden).set("num_hidden_layers", layers)
        .set("num_attention_heads", heads).set("num_key_value_heads", kv_heads).set("head_dim", head_dim)
        .set("intermediate_size", intermediate).set("layer_types", Json::array_of(kinds))
        .set("conv_L_cache", conv_l).set("conv_bias", conv_bias).set("rope_theta", rope_theta)
        .set("norm_eps", norm_eps).set("max_position_embeddings", max_pos)
        .set("block_auto_adjust_ff_dim", auto_adjust).set("block_multiple_of", multiple_of)
        .set("block_ffn_dim_multiplier", multiplier).set("tie_word_embeddings", tie)
        .set("bos_token_id", bos).set("eos_token_id", eos).set("pad_token_id", pad);

    // GQA divisibility, even head size and kv width as in
    // src/model/inference/rules_attention.cpp:194-204; positive cache length as in
    // src/model/inference/rules.cpp:36-40.
    for (const char* key : {"vocab_size", "hidden_size", "num_hidden_layers", "num_attention_heads",
                            "num_key_value_heads", "head_dim", "intermediate_size", "conv_L_cache",
                            "max_position_embeddings", "block_multiple_of"})
        if (out[key].as_int() <= 0)
            throw ConfigError(std::string("config.json: '") + key + "' must be positive, got " + repr(out[key]));
    if (static_cast<long long>(kinds.size()) != layers)
        throw ConfigError("config.json: 'layer_types' has " + std::to_string(kinds.size()) +
                          " entries but 'num_hidden_layers' is " + std::to_string(layers));
    for (size_t i = 0; i < kinds.size(); ++i)
        if (!known_kind(kinds[i]))
            throw ConfigError("config.json: 'layer_types'[" + std::to_string(i) + "] is '" + kinds[i] +
                              "'; known kinds are ['conv', 'full_attention']");
    if (heads % kv_heads)
        throw ConfigError("config.json: 'num_attention_heads' must be a multiple of 'num_key_value_heads'");
    if (head_dim % 2) throw ConfigError("config.json: 'head_dim' must be even");
    if (kv_heads * head_dim > hidden)
        throw ConfigError("config.json: 'num_key_value_heads' * 'head_dim' exceeds 'hidden_size'");
    if (!(rope_theta > 0)) throw ConfigError("config.json: 'rope_theta' must be positive");
    if (!(norm_eps > 0)) throw ConfigError("config.json: 'norm_eps' must be positive");
    if (!multiplier.is_null() && !(multiplier.as_double() > 0))
        throw ConfigError("config.json: 'block_ffn_dim_multiplier' must be positive");
    const double mult = multiplier.is_null() ? 0.0 : multiplier.as_double();
    out.set("ff_dim", lfm2_feed_forward_width(intermediate, auto_adjust, multiple_of, multiplier.is_null() ? nullptr : &mult));
    return out;
}

// Tensor names: embedding and head src/model/inference/global_facts.cpp:41-73 and
// layer_bindings.cpp:24-154; norms layer_bindings.cpp:276-303; short convolution
// src/model/inference/support.cpp:114-123; attention support.cpp:57-78 and
// rules_attention.cpp:72-92; feed-forward layer_bindings.cpp:439-473.
ModelSpec lfm2_build_spec(const Json& c) {
    const long long H = c["hidden_size"].as_int();
    const double eps = c["norm_eps"].as_double();
    auto norm = [&](const std::string& name) {
        PartSpec p;
        p.kind = "rmsnorm";
        p.params = Json::object().set("width", H).set("eps", eps);
        p.tensors = {{"weight", name}};
        return p;
    };
    const bool bias = c["conv_bias"].as_bool();
    ModelSpec spec;
    int i = 0;
    for (const Json& kind : c["layer_types"].items()) {
        const std::string p = "model.layers." + std::to_string(i) + ".";
        LayerSpec layer;
        if (kind.as_string() == "conv") {
            layer.mixer.kind = "short_conv";
            layer.mixer.params = Json::object().set("width", H).set("taps", c["conv_L_cache"]).set("bias", bias);
            layer.mixer.tensors = {{"in_proj", p + "conv.in_proj.weight"}, {"conv", p + "conv.conv.weight"},
                                   {"out_proj", p + "conv.out_proj.weight"}};
            if (bias) {
                layer.mixer.tensors.emplace_back("in_proj_bias", p + "conv.in_proj.bias");
                layer.mixer.tensors.emplace_back("conv_bias", p + "conv.conv.bias");
                layer.mixer.tensors.emplace_back("out_proj_bias", p + "conv.out_proj.bias");
            }
        } else {
            PartSpec rope;
            rope.kind = "rope";
            rope.params = Json::object().set("theta", c["rope_theta"]).set("rotary_dim", c["head_dim"]).set("head_dim", c["head_dim"]);
            layer.mixer.kind = "gqa_attention";
            layer.mixer.params = Json::object().set("width", H).set("heads", c["num_attention_heads"])
                                     .set("kv_heads", c["num_key_value_heads"]).set("head_dim", c["head_dim"])
                                     .set("qk_norm", true).set("eps", eps).set("window", Json())
                                     .set("position", rope.to_json());
            layer.mixer.tensors = {{"q_proj", p + "self_attn.q_proj.weight"}, {"k_proj", p + "self_attn.k_proj.weight"},
                                   {"v_proj", p + "self_attn.v_proj.weight"}, {"out_proj", p + "self_attn.out_proj.weight"},
                                   {"q_norm", p + "self_attn.q_layernorm.weight"}, {"k_norm", p + "self_attn.k_layernorm.weight"}};
        }
        layer.mixer_norm = norm(p + "operator_norm.weight");
        layer.ffn.kind = "swiglu";
        layer.ffn.params = Json::object().set("width", H).set("ff", c["ff_dim"]);
        layer.ffn.tensors = {{"gate", p + "feed_forward.w1.weight"}, {"up", p + "feed_forward.w3.weight"},
                             {"down", p + "feed_forward.w2.weight"}};
        layer.ffn_norm = norm(p + "ffn_norm.weight");
        spec.layers.push_back(std::move(layer));
        spec.order.push_back(RunStep{i, {}});
        ++i;
    }
    spec.architecture = "Lfm2ForCausalLM";
    spec.vocab_size = static_cast<int>(c["vocab_size"].as_int());
    spec.hidden_size = static_cast<int>(H);
    spec.max_context = static_cast<int>(c["max_position_embeddings"].as_int());
    spec.embedding.kind = "embedding";
    spec.embedding.params = Json::object().set("vocab", c["vocab_size"]).set("width", H);
    spec.embedding.tensors = {{"table", "model.embed_tokens.weight"}};
    spec.head.params = Json::object().set("vocab", c["vocab_size"]).set("width", H);
    if (c["tie_word_embeddings"].as_bool()) {
        spec.head.kind = "tied_head";
    } else {
        spec.head.kind = "linear_head";
        spec.head.tensors = {{"weight", "lm_head.weight"}};
    }
    spec.final_norm = norm("model.embedding_norm.weight");
    for (const Json& e : c["eos_token_id"].items()) spec.eos_token_ids.push_back(static_cast<int>(e.as_int()));
    spec.bos_token_id = static_cast<int>(c["bos_token_id"].as_int());
    spec.validate();
    return spec;
}

void register_builtin() {
    Architecture lfm2;
    lfm2.name = "Lfm2ForCausalLM";
    lfm2.aliases = {"lfm2"};
    lfm2.read_config = lfm2_read_config;
    lfm2.build_spec = lfm2_build_spec;
    std::lock_guard<std::mutex> guard(table_lock());
    table()["Lfm2ForCausalLM"] = lfm2;
    table()["lfm2"] = lfm2;
}

}  // namespace

long long lfm2_feed_forward_width(long long intermediate_size, bool auto_adjust, long long multiple_of,
                                  const double* multiplier) {
    if (!auto_adjust) return intermediate_size;
    long long width = static_cast<long long>(2.0 * static_cast<double>(intermediate_size) / 3.0);
    if (multiplier) width = static_cast<long long>(*multiplier * static_cast<double>(width));
    return multiple_of * ((width + multiple_of - 1) / multiple_of);
}

}  // namespace celeg
