// Architectures: one registry from the name in config.json to what builds the model. An
// architecture says which tensors it expects (for the loader and the random-weights mode) and
// assembles a DecoderModel from parts by its typed configuration; no size or constant that
// config.json gives stands in code.
#pragma once

#include <functional>
#include <map>
#include <memory>
#include <string>
#include <vector>

#include "json.h"
#include "parts.h"
#include "weights.h"

namespace minillm {

class ConfigError : public std::runtime_error {
public:
    explicit ConfigError(const std::string& what) : std::runtime_error(what) {}
};

// A model with its weights on the device.
struct LoadedModel {
    std::string architecture;
    Json config;
    int dtype = BF16;
    DecoderModel model;
    DeviceTensors store;
    std::vector<CacheNeed> caches;       // per cache index of the execution order (from the model's mixers)
    int max_positions = 0;               // 0: unbounded
    int eos_token_id = -1;               // -1: none
};

struct Architecture {
    std::string name;
    // the tensors a model of this configuration expects
    std::function<std::vector<ParamSpec>(const Json& config)> param_specs;
    // builds the model from its tensors (already on the device, by name)
    std::function<void(const Json& config, const std::map<std::string, Tensor2>& tensors, int dtype, LoadedModel& out)> assemble;
    std::vector<std::string> optional_prefixes;
    std::function<bool(const std::string&)> ignored_tensor;
};

// Adding an architecture is one call of this (from anywhere: this library's own gpt2.cc, or a plugin's
// static initialiser). `assemble` builds `out.model` from registered parts and sets `out.max_positions`
// and `out.eos_token_id`; the caches' needs are read off the model afterwards.
void register_architecture(const Architecture& a, const std::string& model_type = "");
void register_gpt2();              // gpt2.cc
// Loads a shared library whose initialisers register parts and architectures (dlopen; stays loaded).
// Also called for every path in the environment variable MINI_LLM_PLUGINS (colon-separated), once.
void load_plugin(const std::string& path);
// by config.json: architectures[0], else model_type; unknown -> ConfigError listing the registered names
const Architecture& architecture_of(const Json& config);
std::vector<std::string> registered_architectures();

Json read_config(const std::string& model_dir);
// dtype: BF16 or F32
std::unique_ptr<LoadedModel> load_model(const std::string& model_dir, int dtype);
// Reads a folder's config.json and tensor headers and checks them against the architecture (the
// configuration's refusals, then names and shapes, all mismatches in one WeightsError). No device is touched.
struct ModelFolderSummary {
    std::string architecture;
    int n_tensors = 0;
    int64_t n_parameters = 0;
};
ModelFolderSummary check_model_dir(const std::string& model_dir);
// The configuration's refusals, then the tensors a model of it expects, as JSON text:
// {"architecture": ..., "tensors": [{"name", "shape", "role": "matrix"|"vector", "transpose", "mean", "std"}]}
std::string describe_config(const Json& config);
std::unique_ptr<LoadedModel> random_model(const Json& config, uint64_t seed, int dtype,
                                          const std::string& weights_dtype = "bfloat16");
// a preset by name: config/presets/<name>.json beside the package
Json read_preset(const std::string& presets_dir, const std::string& name);

}  // namespace minillm
