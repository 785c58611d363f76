// C ABI of the native engine: the checked device operations, the parts and the model's step
// function. Loaded from Python with ctypes (kernels/ops.py, models/native.py); a C++ program links
// the classes directly.
//
// Every function returns 0 on success and a non-zero code on failure; `mllm_last_error()` then
// returns the message (per thread). Handles are opaque pointers; a handle passed to a function that
// "takes" it is owned by the receiver from then on.
#include <cstring>
#include <memory>
#include <string>
#include <vector>

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

// -- scratch and tuning ------------------------------------------------------------------------------
int mllm_reserve_scratch(int rows, int vocab, int n_heads, int head_dim) {
    return guarded([&] { reserve_scratch(rows, vocab, n_heads, head_dim); });
}
unsigned long long mllm_scratch_generation(void) { return scratch_generation(); }
void* mllm_scratch_address(const char* name) {
    void* p = nullptr;
    guarded([&] { p = scratch_address(name); });
    return p;
}
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
        else fail("unknown tuning value '%s'", name);
    });
}

// -- the ops (see ops.h) -----------------------------------------------------------------------------
int mllm_op_embed(const int* ids, const int* positions, const Tensor2* wte, const Tensor2* wpe, const Tensor2* out,
                  hipStream_t s) {
    return guarded([&] { embed(ids, positions, *wte, wpe, *out, s); });
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

// -- parts -------------------------------------------------------------------------------------------
int mllm_has_part(const char* category, const char* kind) { return has_part(category, kind) ? 1 : 0; }

void* mllm_norm_create(const char* kind, const void* params) {
    Norm* n = nullptr;
    guarded([&] { n = build_norm(kind, *static_cast<const Params*>(params)).release(); });
    return n;
}
void* mllm_mixer_create(const char* kind, const void* params) {
    Mixer* m = nullptr;
    guarded([&] { m = build_mixer(kind, *static_cast<const Params*>(params)).release(); });
    return m;
}
void* mllm_feed_forward_create(const char* kind, const void* params) {
    FeedForward* f = nullptr;
    guarded([&] { f = build_feed_forward(kind, *static_cast<const Params*>(params)).release(); });
    return f;
}
// Takes the mixer, the feed-forward and the norms.
void* mllm_block_create(const char* kind, void* mixer, void* feed_forward, void** norms, int n_norms) {
    Block* b = nullptr;
    std::unique_ptr<Mixer> m(static_cast<Mixer*>(mixer));
    std::unique_ptr<FeedForward> f(static_cast<FeedForward*>(feed_forward));
    std::vector<std::unique_ptr<Norm>> ns;
    for (int i = 0; i < n_norms; ++i) ns.emplace_back(static_cast<Norm*>(norms[i]));
    guarded([&] { b = build_block(kind, std::move(m), std::move(f), std::move(ns)).release(); });
    return b;
}
void mllm_norm_destroy(void* n) { delete static_cast<Norm*>(n); }
void mllm_block_destroy(void* b) { delete static_cast<Block*>(b); }

// -- the model ---------------------------------------------------------------------------------------
void* mllm_model_create(const Tensor2* wte, const Tensor2* wpe, int dtype) {
    auto* m = new DecoderModel();
    m->wte = *wte;
    if (wpe != nullptr) m->wpe = *wpe;
    m->dtype = dtype;
    return m;
}
void mllm_model_destroy(void* m) { delete static_cast<DecoderModel*>(m); }
// Takes the block. Returns the layer's index.
int mllm_model_add_layer(void* m, void* block) {
    auto* model = static_cast<DecoderModel*>(m);
    model->layers.emplace_back(static_cast<Block*>(block));
    return static_cast<int>(model->layers.size()) - 1;
}
void mllm_model_set_order(void* m, const int* layer, const int* cache, const int* write, int n) {
    auto* model = static_cast<DecoderModel*>(m);
    model->order.clear();
    for (int i = 0; i < n; ++i) model->order.push_back({layer[i], cache[i], write[i] != 0});
}
// Takes the norm.
void mllm_model_set_final_norm(void* m, void* norm) { static_cast<DecoderModel*>(m)->final_norm.reset(static_cast<Norm*>(norm)); }
size_t mllm_model_workspace_bytes(const void* m, int tokens, int n_logits) {
    return static_cast<const DecoderModel*>(m)->workspace_bytes(tokens, n_logits);
}
// One step: the tokens of `step` through every call of the execution order, fp32 logits of the wanted
// rows into `logits`. `arena` is device memory of at least mllm_model_workspace_bytes bytes.
int mllm_model_forward(const void* m, const StepView* step, const CacheView* caches, int n_caches, void* arena,
                       size_t arena_bytes, const Tensor2* logits, hipStream_t s) {
    return guarded([&] {
        Arena a(arena, arena_bytes);
        std::vector<CacheView> cv(caches, caches + n_caches);
        static_cast<const DecoderModel*>(m)->forward(*step, cv, a, logits ? *logits : Tensor2(), s);
    });
}

// -- the engine (engine.h) ---------------------------------------------------------------------------
// options: kv_block_size, total_kv_blocks, max_batch_num, max_tokens_per_step, prefill_chunk, overlap (0/1),
// kv_memory_fraction in millionths (0: total_kv_blocks counts)
static EngineOptions options_of(const int* o) {
    EngineOptions e;
    e.kv_block_size = o[0]; e.total_kv_blocks = o[1]; e.max_batch_num = o[2]; e.max_tokens_per_step = o[3];
    e.prefill_chunk = o[4]; e.overlap = o[5] != 0; e.kv_memory_fraction = o[6] * 1e-6;
    return e;
}
void* mllm_engine_from_pretrained(const char* model_dir, int dtype, const int* options7) {
    Engine* e = nullptr;
    guarded([&] { e = Engine::from_pretrained(model_dir, dtype, options_of(options7)).release(); });
    return e;
}
// config_json: the text of a config.json
void* mllm_engine_from_random(const char* config_json, unsigned long long seed, int dtype, const int* options7) {
    Engine* e = nullptr;
    guarded([&] { e = Engine::from_random(Json::parse(config_json), seed, dtype, options_of(options7)).release(); });
    return e;
}
void mllm_engine_destroy(void* e) { delete static_cast<Engine*>(e); }
// Returns the request's id, or -1 (see mllm_last_error).
long long mllm_engine_add_request(void* e, const int* tokens, int n, float temperature, unsigned long long seed,
                                  int max_new_tokens, int ignore_eos, long long request_id) {
    long long id = -1;
    guarded([&] {
        SamplingParams sp;
        sp.temperature = temperature; sp.seed = seed; sp.max_new_tokens = max_new_tokens; sp.ignore_eos = ignore_eos != 0;
        id = static_cast<Engine*>(e)->add_request(std::vector<int>(tokens, tokens + n), sp, request_id);
    });
    return id;
}
int mllm_engine_has_unfinished(void* e) { return static_cast<Engine*>(e)->has_unfinished() ? 1 : 0; }
// One iteration. Up to `cap` outputs are written (ids, tokens, finished flags; a token of -1 is a failed
// request, whose reason mllm_last_error holds); returns their number, or -1 on an error.
int mllm_engine_step(void* e, long long* ids, int* tokens, int* finished, int cap) {
    int n = -1;
    guarded([&] {
        const std::vector<RequestOutput> outs = static_cast<Engine*>(e)->step();
        if (static_cast<int>(outs.size()) > cap) fail("more outputs (%zu) than room (%d)", outs.size(), cap);
        n = 0;
        for (const RequestOutput& o : outs) {
            ids[n] = o.request_id; tokens[n] = o.token; finished[n] = o.finished ? 1 : 0;
            if (o.token < 0) g_error = o.error;
            ++n;
        }
    });
    return n;
}
int mllm_engine_abort(void* e, long long id) { return guarded([&] { static_cast<Engine*>(e)->abort(id); }); }
// names: steps, scheduled_tokens, prefill_tokens, decode_tokens, deferred_decodes, deferred_prefills, preemptions,
// failures, finished, peak_pages_used, free_pages, total_pages (in this order)
void mllm_engine_stats(void* e, long long* out12) {
    const auto st = static_cast<Engine*>(e)->stats();
    const char* names[12] = {"steps", "scheduled_tokens", "prefill_tokens", "decode_tokens", "deferred_decodes", "deferred_prefills",
                             "preemptions", "failures", "finished", "peak_pages_used", "free_pages", "total_pages"};
    for (int i = 0; i < 12; ++i) out12[i] = st.at(names[i]);
}
int mllm_engine_vocab_size(void* e) { return static_cast<Engine*>(e)->model().model.vocab_size(); }
// weights bytes read once per step, flops per token... are the Python model's business; here: the cache's bytes per token
unsigned long long mllm_engine_cache_bytes_per_token(void* e) { return static_cast<Engine*>(e)->runner().cache().bytes_per_token(); }
void mllm_engine_synchronize(void* e) { guarded([&] { static_cast<Engine*>(e)->runner().synchronize(); }); }

}  // extern "C"
