#include "arch.h"

#include <dlfcn.h>

#include <cstdlib>
#include <fstream>
#include <mutex>
#include <set>
#include <sstream>

namespace minillm {

namespace {
std::map<std::string, Architecture>& archs() { static std::map<std::string, Architecture> m; return m; }
std::map<std::string, std::string>& by_model_type() { static std::map<std::string, std::string> m; return m; }

// built-in architectures (one file each) and the plugins named by the environment, once
void register_builtin_architectures() {
    static std::once_flag once;
    std::call_once(once, [] {
        register_gpt2();
        if (const char* env = std::getenv("MINI_LLM_PLUGINS")) {
            std::stringstream ss(env);
            for (std::string path; std::getline(ss, path, ':');)
                if (!path.empty()) load_plugin(path);
        }
    });
}

std::string read_file(const std::string& path) {
    std::ifstream f(path);
    if (!f) throw ConfigError(path + ": cannot be read");
    std::stringstream ss;
    ss << f.rdbuf();
    return ss.str();
}
}  // namespace

void register_architecture(const Architecture& a, const std::string& model_type) {
    if (a.name.empty() || !a.param_specs || !a.assemble) throw ConfigError("an architecture needs a name, param_specs and assemble");
    archs()[a.name] = a;
    if (!model_type.empty()) by_model_type()[model_type] = a.name;
}

void load_plugin(const std::string& path) {
    static std::mutex mutex;
    static std::set<std::string> loaded;
    std::lock_guard<std::mutex> lock(mutex);
    if (loaded.count(path)) return;
    // its static initialisers call register_* of this library
    void* h = dlopen(path.c_str(), RTLD_NOW | RTLD_GLOBAL);
    if (h == nullptr) {
        const char* why = dlerror();
        throw ConfigError("plugin " + path + " cannot be loaded: " + (why ? why : "unknown error"));
    }
    loaded.insert(path);
}

std::vector<std::string> registered_architectures() {
    register_builtin_architectures();
    std::vector<std::string> n;
    for (const auto& kv : archs()) n.push_back(kv.first);
    return n;
}

const Architecture& architecture_of(const Json& config) {
    register_builtin_architectures();
    std::string name;
    if (const Json* a = config.find("architectures"))
        if (a->is_array() && !a->array().empty() && a->array()[0].is_string()) name = a->array()[0].string();
    if (name.empty() || !archs().count(name)) {
        if (const Json* t = config.find("model_type"))
            if (t->is_string() && by_model_type().count(t->string())) name = by_model_type()[t->string()];
    }
    auto it = archs().find(name);
    if (it == archs().end()) {
        std::string known;
        for (const auto& kv : archs()) known += (known.empty() ? "" : ", ") + kv.first;
        throw ConfigError("config.json names no known architecture ('" + name + "'); registered: " + known);
    }
    return it->second;
}

Json read_config(const std::string& model_dir) {
    const std::string path = model_dir + "/config.json";
    try {
        Json j = Json::parse(read_file(path));
        if (!j.is_object()) throw ConfigError(path + ": not a JSON object");
        return j;
    } catch (const JsonError& e) {
        throw ConfigError(path + ": " + e.what());
    }
}

Json read_preset(const std::string& presets_dir, const std::string& name) {
    const std::string path = presets_dir + "/" + name + ".json";
    std::ifstream f(path);
    if (!f) throw ConfigError("unknown preset '" + name + "' (no " + path + ")");
    std::stringstream ss;
    ss << f.rdbuf();
    return Json::parse(ss.str());
}

static std::unique_ptr<LoadedModel> build(const Json& config, const TensorSource& source, int dtype, const std::string& where) {
    const Architecture& a = architecture_of(config);
    std::unique_ptr<LoadedModel> m(new LoadedModel());
    m->architecture = a.name;
    m->config = config;
    m->dtype = dtype;
    const auto specs = a.param_specs(config);
    const auto tensors = load_tensors(specs, source, dtype, m->store, a.optional_prefixes, a.ignored_tensor, where);
    a.assemble(config, tensors, dtype, *m);
    m->model.dtype = dtype;
    m->caches = m->model.cache_needs();
    if (m->max_positions == 0 && m->model.position) m->max_positions = m->model.position->max_positions();
    return m;
}

std::unique_ptr<LoadedModel> load_model(const std::string& model_dir, int dtype) {
    const Json config = read_config(model_dir);
    architecture_of(config);                     // a clear error before any file is mapped
    CheckpointSource source(model_dir);
    return build(config, source, dtype, model_dir);
}

ModelFolderSummary check_model_dir(const std::string& model_dir) {
    const Json config = read_config(model_dir);
    const Architecture& a = architecture_of(config);
    const auto specs = a.param_specs(config);
    CheckpointSource source(model_dir);
    check_checkpoint(specs, source, a.optional_prefixes, a.ignored_tensor, model_dir);
    ModelFolderSummary s;
    s.architecture = a.name;
    s.n_tensors = static_cast<int>(specs.size());
    for (const auto& sp : specs) {
        int64_t n = 1;
        for (int64_t d : sp.shape) n *= d;
        s.n_parameters += n;
    }
    return s;
}

std::string describe_config(const Json& config) {
    const Architecture& a = architecture_of(config);
    std::vector<Json> tensors;
    for (const ParamSpec& sp : a.param_specs(config)) {
        Json t = Json::object();
        t.set("name", Json::of(sp.name));
        std::vector<Json> shape;
        for (int64_t d : sp.shape) shape.push_back(Json::of(d));
        t.set("shape", Json::array_of(shape));
        t.set("role", Json::of(sp.role == ParamSpec::Matrix ? "matrix" : "vector"));
        t.set("transpose", Json::of(sp.transpose));
        t.set("mean", Json::of(sp.mean));
        t.set("std", Json::of(sp.std));
        tensors.push_back(t);
    }
    Json out = Json::object();
    out.set("architecture", Json::of(a.name));
    out.set("tensors", Json::array_of(tensors));
    return out.dump();
}

std::unique_ptr<LoadedModel> random_model(const Json& config, uint64_t seed, int dtype, const std::string& weights_dtype) {
    RandomSource source(seed, weights_dtype);
    return build(config, source, dtype, "random weights");
}

}  // namespace minillm
