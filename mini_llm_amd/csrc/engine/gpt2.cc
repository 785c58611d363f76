// GPT-2: which parts it is made of and what its tensors are called.
#include <cmath>
#include <regex>

#include "arch.h"

namespace minillm {

// ---------------------------------------------------------------------------------------------
// GPT-2 (GPT2LMHeadModel): which parts it is made of and what its tensors are called. Names are those
// of the GPT-2 checkpoint that the reference exports from
// (/root/reference/scripts/export_weights.py:34-66): wte, wpe,
// h.{i}.ln_1/attn.c_attn/attn.c_proj/ln_2/mlp.c_fc/mlp.c_proj, ln_f; Conv1D weights are stored [in, out].
// The reference fixes the sizes at compile time (/root/reference/include/constants.h:5-10,25-28).
// ---------------------------------------------------------------------------------------------
namespace {
struct GPT2Config {
    int64_t vocab_size = 0, n_positions = 0, n_embd = 0, n_layer = 0, n_head = 0, n_inner = 0;
    double eps = 1e-5;
    std::string activation = "gelu_tanh";
    int eos = -1;

    static int64_t req_int(const Json& c, const char* key) {
        const Json* v = c.find(key);
        if (v == nullptr || v->is_null()) throw ConfigError(std::string("config.json: required key '") + key + "' is missing");
        if (!v->is_integer()) throw ConfigError(std::string("config.json: key '") + key + "' must be an integer");
        return v->integer();
    }
    static bool flag(const Json& c, const char* key, bool fallback) {
        const Json* v = c.find(key);
        return (v == nullptr || !v->is_bool()) ? fallback : v->boolean();
    }
    explicit GPT2Config(const Json& c) {
        for (const char* k : {"scale_attn_by_inverse_layer_idx", "reorder_and_upcast_attn", "add_cross_attention"})
            if (flag(c, k, false)) throw ConfigError(std::string("config.json: ") + k + "=true is not supported");
        if (!flag(c, "scale_attn_weights", true)) throw ConfigError("config.json: scale_attn_weights=false is not supported");
        if (!flag(c, "tie_word_embeddings", true)) throw ConfigError("config.json: tie_word_embeddings=false (an untied head) is not supported");
        vocab_size = req_int(c, "vocab_size");
        n_positions = req_int(c, "n_positions");
        n_embd = req_int(c, "n_embd");
        n_layer = req_int(c, "n_layer");
        n_head = req_int(c, "n_head");
        const Json* e = c.find("layer_norm_epsilon");
        if (e == nullptr || !e->is_number()) throw ConfigError("config.json: required key 'layer_norm_epsilon' is missing");
        eps = e->number();
        for (auto kv : {std::make_pair("vocab_size", vocab_size), std::make_pair("n_positions", n_positions),
                        std::make_pair("n_embd", n_embd), std::make_pair("n_layer", n_layer), std::make_pair("n_head", n_head)})
            if (kv.second <= 0) throw ConfigError(std::string("config.json: '") + kv.first + "' must be positive, got " + std::to_string(kv.second));
        if (n_embd % n_head != 0)
            throw ConfigError("config.json: n_embd=" + std::to_string(n_embd) + " is not divisible by n_head=" + std::to_string(n_head));
        if (!(eps > 0)) throw ConfigError("config.json: layer_norm_epsilon must be positive");
        const Json* ni = c.find("n_inner");
        if (ni != nullptr && !ni->is_null()) {
            if (!ni->is_integer()) throw ConfigError("config.json: n_inner must be an integer or null");
            n_inner = ni->integer();
            if (n_inner <= 0) throw ConfigError("config.json: n_inner must be positive, got " + std::to_string(n_inner));
        } else {
            n_inner = 4 * n_embd;            // GPT-2's rule: a missing n_inner means four times the width
        }
        std::string act = "gelu_new";
        if (const Json* a = c.find("activation_function")) if (a->is_string()) act = a->string();
        if (act == "gelu_new" || act == "gelu_pytorch_tanh" || act == "gelu_fast") activation = "gelu_tanh";
        else if (act == "gelu") activation = "gelu_erf";
        else throw ConfigError("config.json: activation_function '" + act + "' is not supported (known: gelu, gelu_fast, gelu_new, gelu_pytorch_tanh)");
        if (const Json* t = c.find("eos_token_id")) if (t->is_integer()) eos = static_cast<int>(t->integer());
    }
};

std::vector<ParamSpec> gpt2_specs(const Json& config) {
    const GPT2Config c(config);
    const int64_t D = c.n_embd, F = c.n_inner;
    // residual projections are initialised with std 0.02 / sqrt(2 n_layer) in random-weights mode
    const double out_std = 0.02 / std::sqrt(2.0 * static_cast<double>(c.n_layer));
    std::vector<ParamSpec> s;
    auto matrix = [&](const std::string& n, int64_t r, int64_t k, bool t, double std) { s.push_back({n, {r, k}, ParamSpec::Matrix, t, 0.0, std}); };
    auto vector = [&](const std::string& n, int64_t k, double mean, double std) { s.push_back({n, {k}, ParamSpec::Vector, false, mean, std}); };
    matrix("wte.weight", c.vocab_size, D, false, 0.02);
    matrix("wpe.weight", c.n_positions, D, false, 0.02);
    for (int64_t i = 0; i < c.n_layer; ++i) {
        const std::string p = "h." + std::to_string(i) + ".";
        vector(p + "ln_1.weight", D, 1.0, 0.1);
        vector(p + "ln_1.bias", D, 0.0, 0.02);
        matrix(p + "attn.c_attn.weight", D, 3 * D, true, 0.02);
        vector(p + "attn.c_attn.bias", 3 * D, 0.0, 0.02);
        matrix(p + "attn.c_proj.weight", D, D, true, out_std);
        vector(p + "attn.c_proj.bias", D, 0.0, 0.02);
        vector(p + "ln_2.weight", D, 1.0, 0.1);
        vector(p + "ln_2.bias", D, 0.0, 0.02);
        matrix(p + "mlp.c_fc.weight", D, F, true, 0.02);
        vector(p + "mlp.c_fc.bias", F, 0.0, 0.02);
        matrix(p + "mlp.c_proj.weight", F, D, true, out_std);
        vector(p + "mlp.c_proj.bias", D, 0.0, 0.02);
    }
    vector("ln_f.weight", D, 1.0, 0.1);
    vector("ln_f.bias", D, 0.0, 0.02);
    return s;
}

void gpt2_assemble(const Json& config, const std::map<std::string, Tensor2>& t, int dtype, LoadedModel& out) {
    const GPT2Config c(config);
    const int head_dim = static_cast<int>(c.n_embd / c.n_head);
    DecoderModel& m = out.model;
    {
        Params e, pos, h;
        e.tensor["table"] = t.at("wte.weight");
        m.embedding = build_embedding("token_table", e);
        pos.tensor["table"] = t.at("wpe.weight");
        m.position = build_position("learned_absolute", pos);
        // the head is tied: it reads the embedding's table
        h.tensor["weight"] = t.at("wte.weight");
        h.num["dtype"] = dtype;
        m.head = build_head("linear", h);
    }
    auto norm = [&](const std::string& name) {
        Params p;
        p.num["size"] = static_cast<double>(c.n_embd);
        p.num["eps"] = c.eps;
        p.num["dtype"] = dtype;
        p.tensor["gamma"] = t.at(name + ".weight");
        p.tensor["beta"] = t.at(name + ".bias");
        return build_norm("layernorm", p);
    };
    for (int64_t i = 0; i < c.n_layer; ++i) {
        const std::string pre = "h." + std::to_string(i) + ".";
        Params a;
        a.num["n_heads"] = static_cast<double>(c.n_head);
        a.num["n_kv_heads"] = static_cast<double>(c.n_head);
        a.num["head_dim"] = head_dim;
        a.num["scale"] = 1.0 / std::sqrt(static_cast<double>(head_dim));
        a.num["window"] = 0;
        a.num["dtype"] = dtype;
        a.tensor["qkv.weight"] = t.at(pre + "attn.c_attn.weight");
        a.tensor["qkv.bias"] = t.at(pre + "attn.c_attn.bias");
        a.tensor["out.weight"] = t.at(pre + "attn.c_proj.weight");
        a.tensor["out.bias"] = t.at(pre + "attn.c_proj.bias");
        a.position = m.position;
        Params f;
        f.str["activation"] = c.activation;
        f.num["dtype"] = dtype;
        f.tensor["up.weight"] = t.at(pre + "mlp.c_fc.weight");
        f.tensor["up.bias"] = t.at(pre + "mlp.c_fc.bias");
        f.tensor["down.weight"] = t.at(pre + "mlp.c_proj.weight");
        f.tensor["down.bias"] = t.at(pre + "mlp.c_proj.bias");
        std::vector<std::unique_ptr<Norm>> norms;
        norms.push_back(norm(pre + "ln_1"));
        norms.push_back(norm(pre + "ln_2"));
        m.layers.push_back(build_block("pre_norm", build_mixer("causal_attention", a), build_feed_forward("dense_mlp", f), std::move(norms)));
        // every layer runs once, in order, on a cache of its own
        m.order.push_back({static_cast<int>(i), static_cast<int>(i), true});
    }
    m.final_norm = norm("ln_f");
    out.max_positions = static_cast<int>(c.n_positions);
    out.eos_token_id = c.eos;
}
}  // namespace

void register_gpt2() {
    Architecture a;
    a.name = "GPT2LMHeadModel";
    a.param_specs = gpt2_specs;
    a.assemble = gpt2_assemble;
    a.optional_prefixes = {"transformer."};
    // buffers of the attention mask that some checkpoints carry, and the tied head's alias
    a.ignored_tensor = [](const std::string& n) {
        static const std::regex mask("^h\\.[0-9]+\\.attn\\.(bias|masked_bias)$");
        return n == "lm_head.weight" || std::regex_match(n, mask);
    };
    register_architecture(a, "gpt2");
}

}  // namespace minillm
