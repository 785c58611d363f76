// Command line of the native engine.
//
//   mini-llm generate --model DIR [options] [--prompt-ids "15496 11 616" ...]
//       Prompts are lines of space-separated token ids (the reference server's request format,
//       /root/reference/src/runtime/server.cpp:13-23,292-297), from --prompt-ids, --prompts-file or
//       standard input. For every request one line comes back: its new token ids, then "[DONE]" (the
//       reference streams "<id>\n" per token and "<id> [DONE]\n" at the end, server.cpp:344-350;
//       --stream prints that form, prefixed with the request's index). A line that is not a list of ids
//       answers "invalid request". Instead of --model DIR: --preset NAME --weights-seed S generates with
//       random weights of that size.
//   mini-llm make-model (--preset NAME | --config FILE) --seed S --out DIR [--weights-dtype bfloat16|float32]
//       Writes a model folder with random weights.
//   mini-llm replay --model DIR --dtype bfloat16|float32 --out DIR --max-tokens N [--page-size P]
//       Trace replay: one JSON object a line on standard input
//       ({"step": 0, "entries": [{"id": "a", "tokens": [5, 17, 3], "want": [0, 2]}], "end": []}), logits of
//       the wanted places to OUT/<step>.f32, "done <step>" after every step. It samples nothing.
//
// Option names follow the reference's constants (/root/reference/include/constants.h:14-20):
// --max-new-tokens (DEFAULT_MAX_NEW_TOKENS 8), --kv-block-size (DEFAULT_KV_BLOCK_SIZE 16),
// --total-kv-blocks (DEFAULT_TOTAL_KV_BLOCKS 4096), --max-batch-num (MAX_BATCH_NUM 16).
// The reference's program takes no arguments and serves a socket (/root/reference/src/main.cpp:3-10).
#include <sys/stat.h>
#include <unistd.h>

#include <cstdio>
#include <cstdlib>
#include <fstream>
#include <iostream>
#include <map>
#include <set>
#include <sstream>

#include "engine.h"

using namespace minillm;

namespace {

struct Args {
    std::map<std::string, std::vector<std::string>> values;
    std::set<std::string> flags;
    bool has(const std::string& k) const { return values.count(k) || flags.count(k); }
    std::string get(const std::string& k, const std::string& fallback = "") const {
        auto it = values.find(k);
        return it == values.end() ? fallback : it->second.back();
    }
    long integer(const std::string& k, long fallback) const {
        if (!values.count(k)) return fallback;
        char* end = nullptr;
        const std::string v = get(k);
        const long n = std::strtol(v.c_str(), &end, 10);
        if (end == nullptr || *end != '\0') throw EngineError("--" + k + " wants an integer, got '" + v + "'");
        return n;
    }
    double real(const std::string& k, double fallback) const {
        if (!values.count(k)) return fallback;
        char* end = nullptr;
        const std::string v = get(k);
        const double n = std::strtod(v.c_str(), &end);
        if (end == nullptr || *end != '\0') throw EngineError("--" + k + " wants a number, got '" + v + "'");
        return n;
    }
};

Args parse_args(int argc, char** argv, int first, const std::set<std::string>& with_value, const std::set<std::string>& flags) {
    Args a;
    for (int i = first; i < argc; ++i) {
        std::string k = argv[i];
        if (k.rfind("--", 0) != 0) throw EngineError("unexpected argument '" + k + "'");
        k = k.substr(2);
        std::string inline_value;
        const size_t eq = k.find('=');
        bool has_inline = false;
        if (eq != std::string::npos) { inline_value = k.substr(eq + 1); k = k.substr(0, eq); has_inline = true; }
        if (flags.count(k)) { a.flags.insert(k); continue; }
        if (!with_value.count(k)) throw EngineError("unknown option '--" + k + "'");
        if (has_inline) a.values[k].push_back(inline_value);
        else if (i + 1 < argc) a.values[k].push_back(argv[++i]);
        else throw EngineError("option '--" + k + "' wants a value");
    }
    return a;
}

// A line of space-separated non-negative integers; false otherwise.
bool parse_request(const std::string& line, std::vector<int>& ids) {
    ids.clear();
    std::istringstream ss(line);
    std::string part;
    while (ss >> part) {
        if (part.empty() || part.size() > 9) return false;
        for (char c : part)
            if (c < '0' || c > '9') return false;
        ids.push_back(std::atoi(part.c_str()));
    }
    return !ids.empty();
}

// --plugin PATH (may be given several times): shared libraries that register parts and architectures
void load_plugins(const Args& a) {
    auto it = a.values.find("plugin");
    if (it == a.values.end()) return;
    for (const std::string& path : it->second) load_plugin(path);
}

int dtype_of(const std::string& name) {
    if (name == "bfloat16" || name == "bf16") return BF16;
    if (name == "float32" || name == "fp32") return F32;
    throw EngineError("dtype must be bfloat16 or float32, got '" + name + "'");
}

std::string presets_dir(const char* argv0) {
    if (const char* env = std::getenv("MINI_LLM_PRESETS")) return env;
    // the program lies in mini_llm_amd/_lib; the presets beside it in mini_llm_amd/config/presets
    std::string self = argv0;
    char buf[4096];
    const ssize_t n = readlink("/proc/self/exe", buf, sizeof buf - 1);
    if (n > 0) { buf[n] = 0; self = buf; }
    const size_t slash = self.rfind('/');
    const std::string dir = slash == std::string::npos ? "." : self.substr(0, slash);
    return dir + "/../config/presets";
}

int cmd_generate(int argc, char** argv) {
    const Args a = parse_args(argc, argv, 2,
                              {"model", "preset", "weights-seed", "dtype", "device", "prompt-ids", "prompts-file", "max-new-tokens",
                               "temperature", "seed", "kv-block-size", "total-kv-blocks", "kv-memory-fraction", "max-batch-num",
                               "max-tokens-per-step", "prefill-chunk", "plugin"},
                              {"ignore-eos", "stream", "stats", "no-overlap", "defer-decodes"});
    load_plugins(a);
    if (a.has("model") == a.has("preset")) { std::fprintf(stderr, "give either --model DIR or --preset NAME\n"); return 1; }
    const std::string device = a.get("device", "cuda:0");
    if (device.rfind("cuda", 0) != 0 && device != "gpu") {
        std::fprintf(stderr, "mini-llm: device '%s': the engine runs on the GPU only; it has no CPU path\n", device.c_str());
        return 1;
    }
    std::vector<std::string> lines;
    if (a.values.count("prompt-ids")) lines = a.values.at("prompt-ids");
    if (a.has("prompts-file")) {
        std::ifstream f(a.get("prompts-file"));
        if (!f) { std::fprintf(stderr, "cannot read %s\n", a.get("prompts-file").c_str()); return 1; }
        for (std::string l; std::getline(f, l);)
            if (l.find_first_not_of(" \t\r") != std::string::npos) lines.push_back(l);
    }
    if (lines.empty())
        for (std::string l; std::getline(std::cin, l);)
            if (l.find_first_not_of(" \t\r") != std::string::npos) lines.push_back(l);
    EngineOptions o;
    o.kv_block_size = static_cast<int>(a.integer("kv-block-size", 16));
    o.total_kv_blocks = static_cast<int>(a.integer("total-kv-blocks", 4096));
    o.kv_memory_fraction = a.real("kv-memory-fraction", 0.0);
    if (o.kv_memory_fraction < 0.0 || o.kv_memory_fraction > 1.0) throw EngineError("--kv-memory-fraction wants a number in (0, 1]");
    o.max_batch_num = static_cast<int>(a.integer("max-batch-num", 16));
    o.max_tokens_per_step = static_cast<int>(a.integer("max-tokens-per-step", 2048));
    o.prefill_chunk = static_cast<int>(a.integer("prefill-chunk", 512));
    o.overlap = !a.has("no-overlap");
    o.preempt_for_decode = !a.has("defer-decodes");
    const int dtype = dtype_of(a.get("dtype", "bfloat16"));
    std::unique_ptr<Engine> engine;
    if (a.has("preset"))
        engine = Engine::from_random(read_preset(presets_dir(argv[0]), a.get("preset")), static_cast<uint64_t>(a.integer("weights-seed", 0)), dtype, o);
    else
        engine = Engine::from_pretrained(a.get("model"), dtype, o);
    const bool stream = a.has("stream");
    std::vector<std::string> answer(lines.size());         // a message instead of tokens
    std::vector<std::vector<int>> tokens(lines.size());
    std::map<int64_t, size_t> index_of;
    std::vector<int> ids;
    for (size_t i = 0; i < lines.size(); ++i) {
        if (!parse_request(lines[i], ids)) { answer[i] = "invalid request"; continue; }
        SamplingParams sp;
        sp.temperature = static_cast<float>(a.real("temperature", 0.0));
        sp.seed = static_cast<uint64_t>(a.integer("seed", 0)) + i;
        sp.max_new_tokens = static_cast<int>(a.integer("max-new-tokens", 8));
        sp.ignore_eos = a.has("ignore-eos");
        try {
            index_of[engine->add_request(ids, sp)] = i;
        } catch (const EngineError& e) {
            answer[i] = std::string("invalid request (") + e.what() + ")";
        }
    }
    while (engine->has_unfinished()) {
        for (const RequestOutput& out : engine->step()) {
            const size_t i = index_of.at(out.request_id);
            if (out.token < 0) { answer[i] = "failed: " + out.error; continue; }
            tokens[i].push_back(out.token);
            if (stream) { std::printf("%zu %d%s\n", i, out.token, out.finished ? " [DONE]" : ""); std::fflush(stdout); }
        }
    }
    if (!stream) {
        for (size_t i = 0; i < lines.size(); ++i) {
            if (!answer[i].empty()) { std::printf("%s\n", answer[i].c_str()); continue; }
            for (int t : tokens[i]) std::printf("%d ", t);
            std::printf("[DONE]\n");
        }
    }
    if (a.has("stats")) {
        std::string s = "{";
        for (const auto& kv : engine->stats()) s += (s.size() > 1 ? ", \"" : "\"") + kv.first + "\": " + std::to_string(kv.second);
        std::fprintf(stderr, "%s}\n", s.c_str());
    }
    return 0;
}

// check --model DIR: configuration and tensors against the architecture, without a GPU
int cmd_check(int argc, char** argv) {
    const Args a = parse_args(argc, argv, 2, {"model", "plugin"}, {});
    load_plugins(a);
    if (!a.has("model")) {
        std::fprintf(stderr, "usage: mini-llm check --model DIR\n");
        return 1;
    }
    const ModelFolderSummary s = check_model_dir(a.get("model"));
    std::printf("ok: %s, %d tensors, %lld parameters\n", s.architecture.c_str(), s.n_tensors, static_cast<long long>(s.n_parameters));
    return 0;
}

int cmd_make_model(int argc, char** argv) {
    const Args a = parse_args(argc, argv, 2, {"preset", "config", "seed", "out", "weights-dtype", "plugin"}, {});
    load_plugins(a);
    if (a.has("preset") == a.has("config") || !a.has("seed") || !a.has("out")) {
        std::fprintf(stderr, "usage: mini-llm make-model (--preset NAME | --config FILE) --seed S --out DIR\n");
        return 1;
    }
    Json config;
    if (a.has("preset")) {
        config = read_preset(presets_dir(argv[0]), a.get("preset"));
    } else {
        std::ifstream f(a.get("config"));
        if (!f) { std::fprintf(stderr, "cannot read %s\n", a.get("config").c_str()); return 1; }
        std::stringstream ss;
        ss << f.rdbuf();
        config = Json::parse(ss.str());
    }
    const Architecture& arch = architecture_of(config);
    if (!config.has("architectures")) config.set("architectures", Json::array_of({Json::of(arch.name)}));
    write_random_model(a.get("out"), config, arch.param_specs(config), static_cast<uint64_t>(a.integer("seed", 0)),
                       a.get("weights-dtype", "bfloat16"));
    std::printf("%s\n", a.get("out").c_str());
    return 0;
}

int cmd_replay(int argc, char** argv) {
    const Args a = parse_args(argc, argv, 2, {"model", "dtype", "out", "max-tokens", "page-size", "max-requests", "device", "plugin"}, {});
    load_plugins(a);
    for (const char* k : {"model", "dtype", "out", "max-tokens"})
        if (!a.has(k)) { std::fprintf(stderr, "replay: --%s is required\n", k); return 1; }
    const int page = static_cast<int>(a.integer("page-size", 16));
    if (page < 1 || 64 % page != 0) { std::fprintf(stderr, "--page-size must divide 64\n"); return 1; }
    std::fprintf(stderr, "[replay] loading %s as %s ...\n", a.get("model").c_str(), a.get("dtype").c_str());
    std::unique_ptr<LoadedModel> model = load_model(a.get("model"), dtype_of(a.get("dtype")));
    const int n_pages = static_cast<int>((a.integer("max-tokens", 0) + page - 1) / page);
    ModelRunner runner(*model, page, n_pages, static_cast<int>(a.integer("max-requests", 16)));
    const std::string out_dir = a.get("out");
    for (size_t at = 1; at <= out_dir.size(); ++at)      // the folder and the folders above it
        if (at == out_dir.size() || out_dir[at] == '/') ::mkdir(out_dir.substr(0, at).c_str(), 0755);
    std::map<std::string, int64_t> ids;          // the trace's request ids (any JSON scalar) -> integers
    int64_t next_id = 0;
    // a scalar as it is written in file names and messages: a string without its quotes
    auto plain = [](const Json& v) { return v.is_string() ? v.string() : v.dump(); };
    for (std::string line; std::getline(std::cin, line);) {
        if (line.find_first_not_of(" \t\r") == std::string::npos) continue;
        const Json rec = Json::parse(line);
        const std::string step = plain(rec.at("step"));
        if (step.empty() || step.find('/') != std::string::npos) throw EngineError("a step's name must be a number or a plain word");
        std::vector<StepEntry> entries;
        if (const Json* es = rec.find("entries")) {
            for (const Json& e : es->array()) {
                const std::string key = e.at("id").dump();
                if (!ids.count(key)) ids[key] = next_id++;
                StepEntry se;
                se.request_id = ids[key];
                for (const Json& t : e.at("tokens").array()) se.tokens.push_back(static_cast<int>(t.integer()));
                if (const Json* w = e.find("want"))
                    for (const Json& x : w->array()) se.want.push_back(static_cast<int>(x.integer()));
                entries.push_back(std::move(se));
            }
        }
        if (!entries.empty()) {
            int rows = 0;
            const float* logits = nullptr;
            try {
                logits = runner.step(entries, true, &rows);
            } catch (const std::exception& e) {
                // the runner numbers requests; say which of the trace's ids those numbers are
                std::string msg = std::string("step ") + step + ": " + e.what() + " (";
                for (const auto& kv : ids)
                    for (const StepEntry& se : entries)
                        if (se.request_id == kv.second) msg += "request " + std::to_string(kv.second) + " is " + kv.first + "; ";
                throw EngineError(msg + "requests are numbered as they first appear)");
            }
            if (rows > 0) {
                std::ofstream f(out_dir + "/" + step + ".f32", std::ios::binary);
                f.write(reinterpret_cast<const char*>(logits),
                        static_cast<std::streamsize>(static_cast<size_t>(rows) * model->model.vocab_size() * sizeof(float)));
                if (!f) throw EngineError("cannot write " + out_dir + "/" + step + ".f32");
            }
        }
        if (const Json* end = rec.find("end")) {
            for (const Json& r : end->array()) {
                const std::string key = r.dump();
                auto it = ids.find(key);
                if (it == ids.end()) continue;
                if (runner.manager().has_request(it->second)) runner.end_request(it->second);
                ids.erase(it);
            }
        }
        std::printf("done %s\n", step.c_str());
        std::fflush(stdout);
    }
    return 0;
}

}  // namespace

int main(int argc, char** argv) {
    const std::string cmd = argc > 1 ? argv[1] : "";
    try {
        if (cmd == "generate") return cmd_generate(argc, argv);
        if (cmd == "make-model") return cmd_make_model(argc, argv);
        if (cmd == "replay") return cmd_replay(argc, argv);
        if (cmd == "check") return cmd_check(argc, argv);
    } catch (const std::exception& e) {
        std::fprintf(stderr, "mini-llm: %s\n", e.what());
        return 1;
    }
    std::fprintf(stderr,
                 "usage: mini-llm generate|make-model|replay|check [options]\n"
                 "  generate   --model DIR | --preset NAME [--weights-seed S]  [--dtype bfloat16|float32] [--prompt-ids \"1 2 3\"]...\n"
                 "             [--prompts-file F] [--max-new-tokens 8] [--temperature 0] [--seed 0] [--ignore-eos] [--stream] [--stats]\n"
                 "             [--kv-block-size 16] [--total-kv-blocks 4096 | --kv-memory-fraction F] [--max-batch-num 16] [--max-tokens-per-step 2048]\n"
                 "             [--prefill-chunk 512] [--defer-decodes] [--no-overlap]\n"
                 "  every command: [--plugin LIB.so]...  shared libraries that register further parts and architectures\n"
                 "             (also: the paths in the environment variable MINI_LLM_PLUGINS, separated by colons)\n"
                 "  make-model (--preset NAME | --config FILE) --seed S --out DIR [--weights-dtype bfloat16|float32]\n"
                 "  replay     --model DIR --dtype bfloat16|float32 --out DIR --max-tokens N [--page-size 16]\n"
                 "  check      --model DIR     (configuration and tensors against the architecture; needs no GPU)\n");
    return cmd.empty() || cmd == "--help" || cmd == "-h" ? (cmd.empty() ? 1 : 0) : 1;
}
