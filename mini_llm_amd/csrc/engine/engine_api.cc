// C ABI of the engine: the checked device operations, single parts, configurations and model folders,
// the runner (step function) and the engine loop. Loaded from Python with ctypes (mini_llm_amd/native.py,
// kernels/ops.py); a C++ program links the classes directly.
//
// Every function returns 0 on success and a non-zero code on failure; `mllm_last_error()` then
// returns the message (per thread). Handles are opaque pointers; a handle passed to a function that
// "takes" it is owned by the receiver from then on.
#include <algorithm>
#include <cstring>
#include <memory>
#include <string>
#include <vector>

#include "arch.h"
#include "engine.h"
#include "ops.h"
#include "parts.h"

using namespace minillm;

namespace {
thread_local std::string g_error;

template <typename F>
int guarded(F&& f) {
    try {
        f();
        return 0;
    } catch (const std::exception& e) {
        g_error = e.what();
        return 1;
    }
}
}  // namespace

extern "C" {

const char* mllm_last_error(void) { return g_error.c_str(); }

// Copies `text` into out[cap] (truncated, always terminated) and returns its full length.
static int put_text(const std::string& text, char* out, int cap) {
    if (out != nullptr && cap > 0) {
        const size_t n = std::min(text.size(), static_cast<size_t>(cap - 1));
        std::memcpy(out, text.data(), n);
        out[n] = 0;
    }
    return static_cast<int>(text.size());
}

// -- scratch and tuning ------------------------------------------------------------------------------
void* mllm_scratch_address(const char* name, hipStream_t stream) {
    void* p = nullptr;
    guarded([&] { p = scratch_address(name, stream); });
    return p;
}
unsigned long long mllm_scratch_bytes(void) {
    size_t n = 0;
    guarded([&] { n = scratch_bytes(); });
    return n;
}
int mllm_release_scratch(hipStream_t stream) { return guarded([&] { release_scratch(stream); }); }
// name: "decode_shape" (nsplit, waves; 0, 0 = automatic), "unmerged_shape", "merge_max_rows" (a), "ln_fuse_max_rows" (a), "long_context_splits" (a: 0 off, 1 on)
int mllm_set_tuning(const char* name, int a, int b) {
    return guarded([&] {
        Tuning& t = tuning();
        const std::string n(name);
        if (n == "decode_shape") { t.decode_nsplit = a; t.decode_waves = b; }
        else if (n == "unmerged_shape") { t.unmerged_nsplit = a; t.unmerged_waves = b; }
        else if (n == "merge_max_rows") t.merge_max_rows = a;
        else if (n == "ln_fuse_max_rows") t.ln_fuse_max_rows = a;
        else if (n == "long_context_splits") t.long_context_splits = a;
        else if (n == "reset_seen") t.seen = Tuning::Seen();
        else fail("unknown tuning value '%s'", name);
    });
}
// What the ops chose since the last "reset_seen": "max_decode_splits" (most workgroups a (token, head) pair's keys
// were split over), "merge_kernel_launches", "prefill_tile_launches" (the bfloat16 matrix-core kernel), "tiled_f32_launches" (the 32-bit one),
// "generic_attention_launches". -1: unknown name.
long long mllm_get_seen(const char* name) {
    const Tuning::Seen& s = tuning().seen;
    const std::string n(name);
    if (n == "max_decode_splits") return s.max_decode_splits;
    if (n == "merge_kernel_launches") return s.merge_kernel_launches;
    if (n == "prefill_tile_launches") return s.prefill_tile_launches;
    if (n == "tiled_f32_launches") return s.tiled_f32_launches;
    if (n == "generic_attention_launches") return s.generic_attention_launches;
    return -1;
}

// -- the ops (see ops.h) -----------------------------------------------------------------------------
int mllm_op_embed(const int* ids, const int* positions, const Tensor2* wte, const Tensor2* wpe, const Tensor2* out,
                  const int* src, const int* prev, int n_prev, hipStream_t s) {
    return guarded([&] {
        FedTokens fed;
        fed.src = src; fed.prev = prev; fed.n_prev = n_prev;
        embed(ids, positions, *wte, wpe, *out, s, src ? &fed : nullptr);
    });
}
int mllm_op_select_tokens(int* ids, const int* src, const int* prev, int n, int n_prev, hipStream_t s) {
    return guarded([&] { select_tokens(ids, src, prev, n, n_prev, s); });
}
int mllm_op_reset_state(void* state, size_t slot_bytes, int n_slots, const int* slots, const int* starts, int n_seqs,
                        hipStream_t s) {
    return guarded([&] { reset_state(state, slot_bytes, n_slots, slots, starts, n_seqs, s); });
}
int mllm_op_layernorm(const Tensor2* x, const float* gamma, const float* beta, float eps, const Tensor2* out,
                      const int* rows, hipStream_t s) {
    return guarded([&] { layernorm(*x, gamma, beta, eps, *out, rows, s); });
}
int mllm_op_kv_append(const Tensor2* src, int k_col, int v_col, const Tensor2* k_pages, const Tensor2* v_pages,
                      const int* slots, hipStream_t s) {
    return guarded([&] { kv_append(*src, k_col, v_col, *k_pages, *v_pages, slots, s); });
}
int mllm_op_linear(const Tensor2* a, const Tensor2* w, const float* bias, const Tensor2* out, int epilogue,
                   const KvScatter* kv, hipStream_t s) {
    return guarded([&] { linear(*a, *w, bias, *out, epilogue, kv, s); });
}
int mllm_op_linear_from_splits(const AttentionSplits* a, const Tensor2* w, const float* bias, const Tensor2* out,
                               int epilogue, void* tmp, hipStream_t s) {
    return guarded([&] { linear_from_splits(*a, *w, bias, *out, epilogue, tmp, s); });
}
int mllm_op_merge_splits(const AttentionSplits* a, const Tensor2* out, hipStream_t s) {
    return guarded([&] { merge_splits(*a, *out, s); });
}
int mllm_op_ln_linear(const Tensor2* x, const float* gamma, const float* beta, float eps, const Tensor2* w,
                      const float* bias, const Tensor2* out, int epilogue, const int* rows, void* tmp,
                      const KvScatter* kv, hipStream_t s) {
    return guarded([&] { ln_linear(*x, gamma, beta, eps, *w, bias, *out, epilogue, rows, tmp, kv, s); });
}
// *unmerged = 1 and *splits filled when the result was left as splits (only with may_split)
int mllm_op_paged_attention(const AttentionArgs* a, AttentionSplits* splits, int* unmerged, hipStream_t s) {
    return guarded([&] { *unmerged = paged_attention(*a, splits, s) ? 1 : 0; });
}
int mllm_op_argmax(const Tensor2* logits, int* out, hipStream_t s) { return guarded([&] { argmax(*logits, out, s); }); }
int mllm_op_sample(const Tensor2* logits, const float* temperature, const float* u, int* out, hipStream_t s) {
    return guarded([&] { sample(*logits, temperature, u, out, s); });
}

// -- parameters of a part ----------------------------------------------------------------------------
void* mllm_params_create(void) { return new Params(); }
void mllm_params_destroy(void* p) { delete static_cast<Params*>(p); }
void mllm_params_set_number(void* p, const char* key, double v) { static_cast<Params*>(p)->num[key] = v; }
void mllm_params_set_string(void* p, const char* key, const char* v) { static_cast<Params*>(p)->str[key] = v; }
void mllm_params_set_tensor(void* p, const char* key, const Tensor2* t) { static_cast<Params*>(p)->tensor[key] = *t; }

// -- single parts, for tests of a part alone -----------------------------------------------------------
// (A mixer needs a step's index arrays and a cache: it is tested through a model, not here.)
int mllm_has_part(const char* category, const char* kind) { return has_part(category, kind) ? 1 : 0; }
void* mllm_norm_create(const char* kind, const void* params) {
    Norm* n = nullptr;
    guarded([&] { n = build_norm(kind, *static_cast<const Params*>(params)).release(); });
    return n;
}
void mllm_norm_destroy(void* n) { delete static_cast<Norm*>(n); }
// out[i,:] = norm(x[rows ? rows[i] : i, :]); `arena` is device memory for temporaries
int mllm_norm_forward(const void* norm, const Tensor2* x, const int* rows, const Tensor2* out, void* arena, size_t arena_bytes,
                      hipStream_t s) {
    return guarded([&] {
        Arena a(arena, arena_bytes);
        const Tensor2 h = static_cast<const Norm*>(norm)->forward(*x, rows, static_cast<int>(out->rows), a, s);
        if (h.dtype != out->dtype || h.cols != out->cols) fail("the norm's output is %s [%lld], the buffer %s [%lld]", dtype_name(h.dtype), (long long)h.cols, dtype_name(out->dtype), (long long)out->cols);
        if (hipMemcpy2DAsync(out->data, out->stride * out->esz(), h.data, h.stride * h.esz(), h.cols * h.esz(), h.rows, hipMemcpyDeviceToDevice, s) != hipSuccess)
            fail("copy of the norm's output failed");
    });
}
void* mllm_feed_forward_create(const char* kind, const void* params) {
    FeedForward* f = nullptr;
    guarded([&] { f = build_feed_forward(kind, *static_cast<const Params*>(params)).release(); });
    return f;
}
void mllm_feed_forward_destroy(void* f) { delete static_cast<FeedForward*>(f); }
// x += feed_forward(h), h already normalised [T, hidden] in the compute dtype
int mllm_feed_forward_forward(const void* ff, const Tensor2* h, const Tensor2* x, void* arena, size_t arena_bytes, hipStream_t s) {
    return guarded([&] {
        Arena a(arena, arena_bytes);
        StepView step;
        step.n_tokens = static_cast<int>(h->rows);
        NormedInput in(*h);
        static_cast<const FeedForward*>(ff)->forward(in, step, *x, a, s);
    });
}
void* mllm_embedding_create(const char* kind, const void* params) {
    Embedding* e = nullptr;
    guarded([&] { e = build_embedding(kind, *static_cast<const Params*>(params)).release(); });
    return e;
}
void mllm_embedding_destroy(void* e) { delete static_cast<Embedding*>(e); }
// x[t,:] = embedding(ids[t]) (+ row positions[t] of a position encoding of kind position_kind, built from position_params)
int mllm_embedding_forward(const void* emb, const char* position_kind, const void* position_params, const int* ids,
                           const int* positions, const Tensor2* x, hipStream_t s) {
    return guarded([&] {
        std::shared_ptr<const PositionEncoding> pos;
        if (position_kind != nullptr && position_kind[0] != 0) pos = build_position(position_kind, *static_cast<const Params*>(position_params));
        StepView step;
        step.n_tokens = static_cast<int>(x->rows);
        step.token_ids = ids;
        step.positions = positions;
        static_cast<const Embedding*>(emb)->forward(step, pos.get(), *x, s);
    });
}
void* mllm_head_create(const char* kind, const void* params) {
    Head* h = nullptr;
    guarded([&] { h = build_head(kind, *static_cast<const Params*>(params)).release(); });
    return h;
}
void mllm_head_destroy(void* h) { delete static_cast<Head*>(h); }
// logits[i,:] = head(norm(x[rows ? rows[i] : i, :]))
int mllm_head_forward(const void* head, const void* norm, const Tensor2* x, const int* rows, const Tensor2* logits, void* arena,
                      size_t arena_bytes, hipStream_t s) {
    return guarded([&] {
        Arena a(arena, arena_bytes);
        static_cast<const Head*>(head)->forward(*x, *static_cast<const Norm*>(norm), rows, *logits, a, s);
    });
}

// -- configurations, architectures, model folders (no device is touched) -------------------------------
int mllm_load_plugin(const char* path) { return guarded([&] { load_plugin(path); }); }
// JSON array of names; returns the text's full length
int mllm_registered_architectures(char* out, int cap) {
    std::string text;
    guarded([&] {
        std::vector<Json> names;
        for (const std::string& n : registered_architectures()) names.push_back(Json::of(n));
        text = Json::array_of(names).dump();
    });
    return put_text(text, out, cap);
}
// The architecture and the tensors a model of this config.json expects, as JSON (arch.h: describe_config);
// returns the text's full length, or -1 when the configuration is refused (mllm_last_error says why).
int mllm_describe_config(const char* config_json, char* out, int cap) {
    std::string text;
    if (guarded([&] { text = describe_config(Json::parse(config_json)); }) != 0) return -1;
    return put_text(text, out, cap);
}
// Checks a folder's config.json and tensor headers against its architecture; out: "architecture tensors parameters"
int mllm_check_model_dir(const char* model_dir, char* out, int cap) {
    return guarded([&] {
        const ModelFolderSummary s = check_model_dir(model_dir);
        put_text(s.architecture + " " + std::to_string(s.n_tensors) + " " + std::to_string(s.n_parameters), out, cap);
    });
}
// Writes config.json and model.safetensors with random weights (weights_dtype: "bfloat16" or "float32")
int mllm_write_random_model(const char* config_json, unsigned long long seed, const char* out_dir, const char* weights_dtype) {
    return guarded([&] {
        Json config = Json::parse(config_json);
        const Architecture& arch = architecture_of(config);
        if (!config.has("architectures")) config.set("architectures", Json::array_of({Json::of(arch.name)}));
        write_random_model(out_dir, config, arch.param_specs(config), seed, weights_dtype);
    });
}
// n values of the random generator for tensor `name` under `seed`, from element `first` on
int mllm_normal_values(unsigned long long seed, const char* name, long long first, long long n, double mean, double std, float* out) {
    return guarded([&] { normal_values(seed, name, first, n, mean, std, out); });
}

// -- a runner: a model, its caches and the step function (engine.h: ModelRunner) ------------------------
namespace {
struct RunnerBox {
    std::unique_ptr<LoadedModel> model;
    std::unique_ptr<ModelRunner> runner;
};
}  // namespace
// Either model_dir, or config_json with a seed (random weights, rounded as a written folder holds them).
void* mllm_runner_create(const char* model_dir, const char* config_json, unsigned long long seed, int dtype, int page_size,
                         int n_pages, int max_num_seqs) {
    RunnerBox* box = nullptr;
    guarded([&] {
        std::unique_ptr<RunnerBox> b(new RunnerBox());
        if (model_dir != nullptr && model_dir[0] != 0) b->model = load_model(model_dir, dtype);
        else b->model = random_model(Json::parse(config_json), seed, dtype);
        b->runner.reset(new ModelRunner(*b->model, page_size, n_pages, max_num_seqs));
        box = b.release();
    });
    return box;
}
void mllm_runner_destroy(void* box) { delete static_cast<RunnerBox*>(box); }
void* mllm_runner_of_box(void* box) { return static_cast<RunnerBox*>(box)->runner.get(); }
// One step of B entries: entry i is request ids[i] with its next n_tokens[i] tokens (flattened in `tokens`) and
// n_want[i] wanted places among them (flattened in `want`). The fp32 logits [wanted, vocab] go to `logits`
// (room for cap_rows rows). The runner registers new requests, takes pages and commits lengths itself.
// Returns the number of rows, or -1.
int mllm_runner_step(void* runner, const long long* ids, const int* n_tokens, const int* tokens, const int* n_want,
                     const int* want, int B, float* logits, long long cap_rows) {
    int rows = -1;
    guarded([&] {
        if (B < 0) fail("a step of %d entries", B);
        std::vector<StepEntry> entries(B);
        size_t t = 0, w = 0;
        long long total = 0;
        for (int i = 0; i < B; ++i) {
            if (n_tokens[i] < 0 || n_want[i] < 0) fail("entry %d brings %d tokens and wants %d places", i, n_tokens[i], n_want[i]);
            entries[i].request_id = ids[i];
            entries[i].tokens.assign(tokens + t, tokens + t + n_tokens[i]);
            entries[i].want.assign(want + w, want + w + n_want[i]);
            t += n_tokens[i];
            w += n_want[i];
            total += n_want[i];
        }
        if (total > cap_rows) fail("%lld rows of logits are wanted, the buffer holds %lld", total, cap_rows);
        int n = 0;
        ModelRunner* r = static_cast<ModelRunner*>(runner);
        const float* host = r->step(entries, true, &n);
        if (host != nullptr) std::memcpy(logits, host, static_cast<size_t>(n) * r->model().model.vocab_size() * sizeof(float));
        rows = n;
    });
    return rows;
}
int mllm_runner_end_request(void* runner, long long id) {
    return guarded([&] {
        ModelRunner* r = static_cast<ModelRunner*>(runner);
        if (!r->manager().has_request(id)) fail("request %lld is not live", id);
        r->end_request(id);
    });
}
int mllm_runner_poison(void* runner) { return guarded([&] { static_cast<ModelRunner*>(runner)->cache().poison(); }); }
// The cache manager's consistency report (empty: no page or slot is lost, held twice or both held and free)
int mllm_runner_check(void* runner, char* out, int cap) {
    std::string text;
    guarded([&] { text = static_cast<ModelRunner*>(runner)->manager().check(); });
    return put_text(text, out, cap);
}
// Sizes and costs as JSON: architecture, vocab_size, hidden_size, max_positions, eos_token_id, dtype, n_layers,
// n_calls, n_caches, n_groups, page_size, n_pages, free_pages, n_requests, cache_bytes_per_token, and the step's
// cost (parts.h: StepCost): weight_bytes, flops_per_token, attention_flops_per_key, flops_per_logits_row
int mllm_runner_info(void* runner, char* out, int cap) {
    std::string text;
    guarded([&] {
        ModelRunner* r = static_cast<ModelRunner*>(runner);
        const LoadedModel& m = r->model();
        const StepCost c = m.model.cost();
        Json j = Json::object();
        j.set("architecture", Json::of(m.architecture));
        j.set("vocab_size", Json::of(m.model.vocab_size()));
        j.set("hidden_size", Json::of(m.model.hidden_size()));
        j.set("max_positions", Json::of(m.max_positions));
        j.set("eos_token_id", Json::of(m.eos_token_id));
        j.set("dtype", Json::of(dtype_name(m.dtype)));
        j.set("n_layers", Json::of(static_cast<int>(m.model.layers.size())));
        j.set("n_calls", Json::of(static_cast<int>(m.model.order.size())));
        j.set("n_caches", Json::of(static_cast<int>(m.caches.size())));
        j.set("n_groups", Json::of(r->cache().n_groups()));
        j.set("page_size", Json::of(r->cache().page_size()));
        j.set("n_pages", Json::of(r->n_pages()));
        j.set("free_pages", Json::of(r->manager().n_groups() ? r->manager().free_pages(0) : 0));
        j.set("n_requests", Json::of(r->manager().n_requests()));
        j.set("cache_bytes_per_token", Json::of(static_cast<int64_t>(r->cache().bytes_per_token())));
        j.set("weight_bytes", Json::of(c.weight_bytes));
        j.set("flops_per_token", Json::of(c.flops_per_token));
        j.set("attention_flops_per_key", Json::of(c.attention_flops_per_key));
        j.set("flops_per_logits_row", Json::of(c.flops_per_logits_row));
        text = j.dump();
    });
    return put_text(text, out, cap);
}
void mllm_runner_synchronize(void* runner) { guarded([&] { static_cast<ModelRunner*>(runner)->synchronize(); }); }

// -- the engine (engine.h) ---------------------------------------------------------------------------
// options: kv_block_size, total_kv_blocks, max_batch_num, max_tokens_per_step, prefill_chunk, overlap (0/1),
// kv_memory_fraction in millionths (0: total_kv_blocks counts), preempt_for_decode (0/1)
static EngineOptions options_of(const int* o) {
    EngineOptions e;
    e.kv_block_size = o[0]; e.total_kv_blocks = o[1]; e.max_batch_num = o[2]; e.max_tokens_per_step = o[3];
    e.prefill_chunk = o[4]; e.overlap = o[5] != 0; e.kv_memory_fraction = o[6] * 1e-6; e.preempt_for_decode = o[7] != 0;
    return e;
}
void* mllm_engine_from_pretrained(const char* model_dir, int dtype, const int* options8) {
    Engine* e = nullptr;
    guarded([&] { e = Engine::from_pretrained(model_dir, dtype, options_of(options8)).release(); });
    return e;
}
// config_json: the text of a config.json. The weights are the values a written folder holds (matrices rounded
// to bfloat16 whatever `dtype` computes in), so this and make-model + from_pretrained give the same model.
void* mllm_engine_from_random(const char* config_json, unsigned long long seed, int dtype, const int* options8) {
    Engine* e = nullptr;
    guarded([&] { e = Engine::from_random(Json::parse(config_json), seed, dtype, options_of(options8)).release(); });
    return e;
}
void mllm_engine_destroy(void* e) { delete static_cast<Engine*>(e); }
// The engine's runner, for the mllm_runner_* functions (borrowed: it lives as long as the engine). Requests
// stepped through it directly must not share ids with requests added to the engine.
void* mllm_engine_runner(void* e) { return &static_cast<Engine*>(e)->runner(); }
// Returns the request's id, or -1 (see mllm_last_error).
long long mllm_engine_add_request(void* e, const int* tokens, int n, float temperature, unsigned long long seed,
                                  int max_new_tokens, int ignore_eos, long long request_id) {
    long long id = -1;
    guarded([&] {
        if (n < 0 || (n > 0 && tokens == nullptr)) fail("a prompt of %d tokens", n);
        SamplingParams sp;
        sp.temperature = temperature; sp.seed = seed; sp.max_new_tokens = max_new_tokens; sp.ignore_eos = ignore_eos != 0;
        id = static_cast<Engine*>(e)->add_request(std::vector<int>(tokens, tokens + n), sp, request_id);
    });
    return id;
}
int mllm_engine_has_unfinished(void* e) {
    int r = 0;
    guarded([&] { r = static_cast<Engine*>(e)->has_unfinished() ? 1 : 0; });
    return r;
}
// One iteration. Up to `cap` outputs are written (ids, tokens, finished flags; a token of -1 is a failed request);
// outputs beyond `cap` wait for the next call, and mllm_engine_has_unfinished stays 1 meanwhile. Returns their
// number, or -1 on an error. The reason of the i-th output's failure: mllm_engine_output_error(i), on the thread
// that made the call.
namespace { thread_local std::vector<std::string> g_output_errors; }
int mllm_engine_step(void* e, long long* ids, int* tokens, int* finished, int cap) {
    int n = -1;
    guarded([&] {
        const std::vector<RequestOutput> outs = static_cast<Engine*>(e)->step_some(static_cast<size_t>(std::max(cap, 1)));
        g_output_errors.assign(outs.size(), "");
        n = 0;
        for (const RequestOutput& o : outs) {
            ids[n] = o.request_id; tokens[n] = o.token; finished[n] = o.finished ? 1 : 0;
            g_output_errors[n] = o.error;
            ++n;
        }
    });
    return n;
}
const char* mllm_engine_output_error(int i) {
    return (i >= 0 && i < static_cast<int>(g_output_errors.size())) ? g_output_errors[i].c_str() : "";
}
int mllm_engine_abort(void* e, long long id) { return guarded([&] { static_cast<Engine*>(e)->abort(id); }); }
// names: steps, scheduled_tokens, prefill_tokens, decode_tokens, deferred_decodes, deferred_prefills, preemptions,
// failures, finished, peak_pages_used, free_pages, total_pages, aborted (in this order)
int mllm_engine_stats(void* e, long long* out13) {
    return guarded([&] {
        const auto st = static_cast<Engine*>(e)->stats();
        const char* names[13] = {"steps", "scheduled_tokens", "prefill_tokens", "decode_tokens", "deferred_decodes", "deferred_prefills",
                                 "preemptions", "failures", "finished", "peak_pages_used", "free_pages", "total_pages", "aborted"};
        for (int i = 0; i < 13; ++i) out13[i] = st.at(names[i]);
    });
}
void mllm_engine_synchronize(void* e) { guarded([&] { static_cast<Engine*>(e)->runner().synchronize(); }); }

}  // extern "C"
