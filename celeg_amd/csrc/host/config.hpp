// One registry from an architecture's name to its configuration and model.
//
// The reference selects among registered architectures by probing the checkpoint's
// metadata (src/model/architecture.cpp:31-78) and registers exactly one, automatic,
// architecture (src/composition/builtin_runtime.cpp:13-58).  Here the name in config.json
// ("architectures"[0], else "model_type") selects an entry; an unknown name is an error
// that lists the registered ones.
#pragma once
#include <functional>
#include <map>
#include <string>
#include <vector>

#include "spec.hpp"

namespace celeg {

// name -> shape of the checkpoint's tensors
using TensorShapes = std::map<std::string, std::vector<long long>>;

struct Architecture {
    std::string name;
    std::vector<std::string> aliases;
    // config.json (generation_config.json merged) and, if the checkpoint is at hand, its
    // tensors' shapes -> the architecture's typed configuration, as a flat JSON object of the
    // keys it reads, defaults filled in.  Throws ConfigError naming the key at fault.
    std::function<Json(const Json& config, const TensorShapes* shapes)> read_config;
    // typed configuration -> the parts list
    std::function<ModelSpec(const Json& typed)> build_spec;
};

void register_architecture(Architecture arch, bool replace = false);
std::vector<std::string> registered_architectures();
std::string architecture_name(const Json& config);
const Architecture& find_architecture(const Json& config);

// config.json of a model folder; a generation_config.json beside it overrides bos_token_id
// and eos_token_id (src/checkpoint/catalog.cpp:94-121) and is ignored if it cannot be read.
Json read_config_file(const std::string& model_dir);

struct Described {
    Json config;       // the typed configuration
    ModelSpec spec;
};
Described describe_config(const Json& config, const TensorShapes* shapes);

// The LFM2 feed-forward width: with block_auto_adjust_ff_dim two thirds of intermediate_size,
// times the multiplier (if any), rounded up to a multiple of block_multiple_of.
long long lfm2_feed_forward_width(long long intermediate_size, bool auto_adjust, long long multiple_of,
                                  const double* multiplier);

}  // namespace celeg
