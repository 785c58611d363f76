#include "parts.h"

#include <algorithm>
#include <cstdio>
#include <cstdlib>

namespace minillm {

// ---------------------------------------------------------------------------------------------
// stage times
// ---------------------------------------------------------------------------------------------
StageTimes::StageTimes() : enabled_(std::getenv("MINI_LLM_STAGE_TIMES") != nullptr) {}

StageTimes& StageTimes::get() {
    static StageTimes t;
    return t;
}

hipEvent_t StageTimes::event(hipStream_t s) {
    hipEvent_t e = nullptr;
    if (!spare_.empty()) { e = spare_.back(); spare_.pop_back(); }
    else if (hipEventCreate(&e) != hipSuccess) fail("stage times: an event could not be created");
    if (hipEventRecord(e, s) != hipSuccess) fail("stage times: an event could not be recorded");
    return e;
}

void StageTimes::begin_step(const char* kind, int batch, int tokens, hipStream_t s) {
    if (!enabled_) return;
    // (a step that is being captured into a graph is not timed: its events would become part of the graph)
    hipStreamCaptureStatus capturing = hipStreamCaptureStatusNone;
    if (hipStreamIsCapturing(s, &capturing) != hipSuccess || capturing != hipStreamCaptureStatusNone) { start_ = nullptr; return; }
    kind_ = kind; batch_ = batch; tokens_ = tokens; layer_ = -1;
    start_ = event(s);
}

void StageTimes::mark(const char* stage, hipStream_t s) {
    if (!enabled_ || start_ == nullptr) return;
    marks_.push_back(Mark{layer_, stage, event(s)});
}

void StageTimes::end_step(hipStream_t s) {
    if (!enabled_ || start_ == nullptr) return;
    if (!marks_.empty() && hipEventSynchronize(marks_.back().at) != hipSuccess) fail("stage times: the step failed");
    if (!header_) { std::fprintf(stderr, "kind,batch_size,total_tokens,layer,stage,ms\n"); header_ = true; }
    hipEvent_t before = start_;
    for (const Mark& m : marks_) {
        float ms = 0.f;
        (void)hipEventElapsedTime(&ms, before, m.at);
        std::fprintf(stderr, "%s,%d,%d,%d,%s,%.4f\n", kind_, batch_, tokens_, m.layer, m.stage, ms);
        spare_.push_back(before);
        before = m.at;
    }
    spare_.push_back(before);
    marks_.clear();
    start_ = nullptr;
    (void)s;
}


// ---------------------------------------------------------------------------------------------
void* Arena::take(size_t bytes) {
    const size_t at = (used_ + 255) & ~static_cast<size_t>(255);
    if (at + bytes > capacity_)
        fail("the step's workspace is too small: %zu bytes wanted at %zu of %zu", bytes, at, capacity_);
    used_ = at + bytes;
    peak_ = std::max(peak_, used_);
    return base_ + at;
}

double Params::number(const std::string& key) const {
    auto it = num.find(key);
    if (it == num.end()) fail("parameter '%s' is missing", key.c_str());
    return it->second;
}
double Params::number(const std::string& key, double fallback) const {
    auto it = num.find(key);
    return it == num.end() ? fallback : it->second;
}
const std::string& Params::string(const std::string& key) const {
    auto it = str.find(key);
    if (it == str.end()) fail("parameter '%s' is missing", key.c_str());
    return it->second;
}
const Tensor2& Params::weights(const std::string& key) const {
    auto it = tensor.find(key);
    if (it == tensor.end() || it->second.data == nullptr) fail("tensor '%s' is missing", key.c_str());
    return it->second;
}
const Tensor2* Params::weights_or_null(const std::string& key) const {
    auto it = tensor.find(key);
    return (it == tensor.end() || it->second.data == nullptr) ? nullptr : &it->second;
}

Linear::Linear(const Tensor2& w, const Tensor2* b) : weight(w) {
    if (b != nullptr) {
        if (b->dtype != F32 || b->rows * b->cols != w.rows || !b->contiguous())
            fail("a linear map's bias must be contiguous float32 [%lld]", (long long)w.rows);
        bias = static_cast<const float*>(b->data);
    }
}

// ---------------------------------------------------------------------------------------------
void Norm::linear(const Tensor2& x, const Linear& lin, const Tensor2& out, int epilogue, const int* rows,
                  const KvScatter* kv, Arena& arena, hipStream_t s) const {
    const Tensor2 h = forward(x, rows, static_cast<int>(out.rows), arena, s);
    lin(h, out, epilogue, kv, s);
}

const Tensor2& NormedInput::tensor(Arena& arena, hipStream_t s) {
    if (!have_) {
        h_ = norm_.forward(x_, nullptr, static_cast<int>(x_.rows), arena, s);
        have_ = true;
    }
    return h_;
}

void NormedInput::linear(const Linear& lin, const Tensor2& out, int epilogue, const KvScatter* kv, Arena& arena,
                         hipStream_t s) {
    if (have_) lin(h_, out, epilogue, kv, s);
    else norm_.linear(x_, lin, out, epilogue, nullptr, kv, arena, s);
}

// y = (x - mean) * rsqrt(var + eps) * gamma + beta over the last dimension, biased variance,
// statistics in fp32 (/root/reference/src/kernels/layernorm.cu:32-49). Input: the fp32 stream.
class LayerNorm final : public Norm {
public:
    explicit LayerNorm(const Params& p) {
        size_ = p.integer("size");
        eps_ = static_cast<float>(p.number("eps"));
        dtype = p.integer("dtype");
        const Tensor2& g = p.weights("gamma");
        if (g.dtype != F32 || g.rows * g.cols != size_) fail("layernorm: gamma must be float32 [%d]", size_);
        gamma_ = static_cast<const float*>(g.data);
        if (const Tensor2* b = p.weights_or_null("beta")) {
            if (b->dtype != F32 || b->rows * b->cols != size_) fail("layernorm: beta must be float32 [%d]", size_);
            beta_ = static_cast<const float*>(b->data);
        }
    }
    Tensor2 forward(const Tensor2& x, const int* rows, int n, Arena& arena, hipStream_t s) const override {
        Tensor2 h = arena.tensor(dtype, n, size_);
        layernorm(x, gamma_, beta_, eps_, h, rows, s);
        return h;
    }
    void linear(const Tensor2& x, const Linear& lin, const Tensor2& out, int epilogue, const int* rows,
                const KvScatter* kv, Arena& arena, hipStream_t s) const override {
        // the norm fused into the product where the kernels allow it; otherwise the rows pass through the arena
        const size_t mark = arena.mark();
        void* tmp = arena.take(static_cast<size_t>(out.rows) * size_ * dtype_size(lin.weight.dtype));
        ln_linear(x, gamma_, beta_, eps_, lin.weight, lin.bias, out, epilogue, rows, tmp, kv, s);
        arena.release(mark);
    }
    size_t workspace_bytes(int rows) const override { return static_cast<size_t>(rows) * size_ * dtype_size(dtype) + 256; }

private:
    int size_ = 0;
    float eps_ = 1e-5f;
    const float* gamma_ = nullptr;
    const float* beta_ = nullptr;
};

// qkv = h W_qkv + b; keys/values of the step's tokens go to the pages; every query attends causally
// (optionally within a window) to its sequence's keys in the pages; x += concat_heads(attn) W_out + b.
// Reference: /root/reference/src/model/gpt2_model.cu:289-334. Column layout of qkv: queries, then
// keys, then values; head h at h * head_dim (/root/reference/src/kernels/prefill/append_kv.cu:31-33).
class CausalSelfAttention final : public Mixer {
public:
    explicit CausalSelfAttention(const Params& p) {
        n_heads_ = p.integer("n_heads");
        n_kv_heads_ = p.integer("n_kv_heads");
        head_dim_ = p.integer("head_dim");
        scale_ = static_cast<float>(p.number("scale"));
        window_ = static_cast<int>(p.number("window", 0));
        dtype_ = p.integer("dtype");
        if (n_kv_heads_ < 1 || n_heads_ % n_kv_heads_ != 0) fail("n_heads=%d is not a multiple of n_kv_heads=%d", n_heads_, n_kv_heads_);
        if (head_dim_ % 16 != 0 || head_dim_ > 256) fail("head_dim=%d is not supported (multiples of 16 up to 256)", head_dim_);
        q_dim_ = n_heads_ * head_dim_;
        kv_dim_ = n_kv_heads_ * head_dim_;
        qkv_ = Linear(p.weights("qkv.weight"), p.weights_or_null("qkv.bias"));
        out_ = Linear(p.weights("out.weight"), p.weights_or_null("out.bias"));
        if (qkv_.out_features() != q_dim_ + 2 * kv_dim_ || out_.in_features() != q_dim_)
            fail("attention: the projections' shapes do not fit %d heads of %d (kv heads %d)", n_heads_, head_dim_, n_kv_heads_);
    }
    void forward(NormedInput& h, const StepView& step, const CacheView& cache, const Tensor2& x, bool write, Arena& arena,
                 hipStream_t s) const override {
        if (cache.kind != 1) fail("attention needs a cache of pages");
        const int T = step.n_tokens, g = cache.group;
        Tensor2 qkv = arena.tensor(dtype_, T, q_dim_ + 2 * kv_dim_);
        // Prompt portions: the QKV product is asked to put the new keys and values into the pages (how
        // is the linear map's business). Single tokens: the attention kernel writes them.
        const bool scatter = write && step.max_q_len > 1;
        KvScatter kv;
        if (scatter) {
            kv.slots = step.slots[g];
            kv.k_pages = cache.k_pages;
            kv.v_pages = cache.v_pages;
            kv.q_cols = q_dim_;
        }
        h.linear(qkv_, qkv, STORE, scatter ? &kv : nullptr, arena, s);
        StageTimes::get().mark("qkv", s);
        AttentionArgs a;
        a.q = qkv;
        a.q_col = 0;
        a.n_heads = n_heads_;
        a.n_kv_heads = n_kv_heads_;
        a.head_dim = head_dim_;
        a.k_pages = cache.k_pages;
        a.v_pages = cache.v_pages;
        a.page_size = cache.page_size;
        a.block_tables = step.block_tables[g];
        a.n_seqs = step.n_seqs;
        a.max_blocks = step.max_blocks[g];
        a.token_seq = step.token_seq;
        a.positions = step.positions;
        a.scale = scale_;
        a.window = window_;
        a.out = arena.tensor(dtype_, T, q_dim_);
        a.cu_q = step.cu_q;
        a.ctx_len = step.ctx_len;
        a.max_q_len = step.max_q_len;
        a.max_ctx_len = step.max_ctx_len;
        a.append = (write && !scatter) ? 1 : 0;
        a.k_col = q_dim_;
        a.v_col = q_dim_ + kv_dim_;
        a.slots = step.slots[g];
        a.n_single = step.n_single;
        a.may_split = 1;
        AttentionSplits splits;
        // (the result may come back unmerged, as the states of several workgroups per token and head:
        // the output projection takes either)
        const bool unmerged = paged_attention(a, &splits, s);
        StageTimes::get().mark("attention", s);
        if (unmerged) linear_from_splits(splits, out_.weight, out_.bias, x, ADD_RESIDUAL, a.out.data, s);
        else out_(a.out, x, ADD_RESIDUAL, nullptr, s);
        StageTimes::get().mark("out_proj", s);
    }
    size_t workspace_bytes(int tokens) const override {
        return static_cast<size_t>(tokens) * (2 * q_dim_ + 2 * kv_dim_) * dtype_size(dtype_) + 1024;
    }

private:
    int n_heads_ = 0, n_kv_heads_ = 0, head_dim_ = 0, window_ = 0, q_dim_ = 0, kv_dim_ = 0, dtype_ = BF16;
    float scale_ = 1.f;
    Linear qkv_, out_;
};

// x += act(h W_up + b_up) W_down + b_down, the activation fused into the first product and the
// residual add into the second (/root/reference/src/model/gpt2_model.cu:345-363).
class DenseMLP final : public FeedForward {
public:
    explicit DenseMLP(const Params& p) {
        dtype_ = p.integer("dtype");
        const std::string& act = p.string("activation");
        if (act == "gelu_tanh") act_ = GELU_TANH;
        else if (act == "gelu_erf") act_ = GELU_ERF;
        else fail("unknown activation '%s' (known: gelu_erf, gelu_tanh)", act.c_str());
        up_ = Linear(p.weights("up.weight"), p.weights_or_null("up.bias"));
        down_ = Linear(p.weights("down.weight"), p.weights_or_null("down.bias"));
        if (down_.in_features() != up_.out_features()) fail("feed-forward: the two products' shapes do not fit");
    }
    void forward(NormedInput& h, const StepView& step, const Tensor2& x, Arena& arena, hipStream_t s) const override {
        Tensor2 inner = arena.tensor(dtype_, step.n_tokens, up_.out_features());
        h.linear(up_, inner, act_, nullptr, arena, s);
        StageTimes::get().mark("fc1", s);
        down_(inner, x, ADD_RESIDUAL, nullptr, s);
        StageTimes::get().mark("fc2", s);
    }
    size_t workspace_bytes(int tokens) const override {
        return static_cast<size_t>(tokens) * up_.out_features() * dtype_size(dtype_) + 512;
    }

private:
    int dtype_ = BF16, act_ = GELU_TANH;
    Linear up_, down_;
};

// x += mixer(norm1(x)); x += feed_forward(norm2(x)): the norm stands before each sub-layer, on the
// residual stream (/root/reference/src/model/gpt2_model.cu:279-363).
class PreNormBlock final : public Block {
public:
    PreNormBlock(std::unique_ptr<Mixer> m, std::unique_ptr<FeedForward> f, std::vector<std::unique_ptr<Norm>> norms)
        : mixer_(std::move(m)), ff_(std::move(f)) {
        if (norms.size() != 2) fail("a pre-norm block has two norms");
        norm1_ = std::move(norms[0]);
        norm2_ = std::move(norms[1]);
    }
    void forward(const Tensor2& x, const StepView& step, const CacheView& cache, bool write, Arena& arena,
                 hipStream_t s) const override {
        size_t mark = arena.mark();
        {
            NormedInput h(*norm1_, x);
            mixer_->forward(h, step, cache, x, write, arena, s);
        }
        arena.release(mark);
        {
            NormedInput h(*norm2_, x);
            ff_->forward(h, step, x, arena, s);
        }
        arena.release(mark);
    }
    size_t workspace_bytes(int tokens) const override {
        return std::max(mixer_->workspace_bytes(tokens) + 2 * norm1_->workspace_bytes(tokens),
                        ff_->workspace_bytes(tokens) + 2 * norm2_->workspace_bytes(tokens));
    }

private:
    std::unique_ptr<Mixer> mixer_;
    std::unique_ptr<FeedForward> ff_;
    std::unique_ptr<Norm> norm1_, norm2_;
};

// ---------------------------------------------------------------------------------------------
namespace {
std::map<std::string, NormFactory>& norms() { static std::map<std::string, NormFactory> m; return m; }
std::map<std::string, MixerFactory>& mixers() { static std::map<std::string, MixerFactory> m; return m; }
std::map<std::string, FeedForwardFactory>& feed_forwards() { static std::map<std::string, FeedForwardFactory> m; return m; }
std::map<std::string, BlockFactory>& blocks() { static std::map<std::string, BlockFactory> m; return m; }

void register_builtin_parts() {
    static bool done = false;
    if (done) return;
    done = true;
    norms()["layernorm"] = [](const Params& p) { return std::unique_ptr<Norm>(new LayerNorm(p)); };
    mixers()["causal_attention"] = [](const Params& p) { return std::unique_ptr<Mixer>(new CausalSelfAttention(p)); };
    feed_forwards()["dense_mlp"] = [](const Params& p) { return std::unique_ptr<FeedForward>(new DenseMLP(p)); };
    blocks()["pre_norm"] = [](std::unique_ptr<Mixer> m, std::unique_ptr<FeedForward> f, std::vector<std::unique_ptr<Norm>> n) {
        return std::unique_ptr<Block>(new PreNormBlock(std::move(m), std::move(f), std::move(n)));
    };
}

template <typename Map>
std::string known(const Map& m) {
    std::string s;
    for (const auto& kv : m) s += (s.empty() ? "" : ", ") + kv.first;
    return s;
}
}  // namespace

void register_norm(const std::string& kind, NormFactory f) { register_builtin_parts(); norms()[kind] = std::move(f); }
void register_mixer(const std::string& kind, MixerFactory f) { register_builtin_parts(); mixers()[kind] = std::move(f); }
void register_feed_forward(const std::string& kind, FeedForwardFactory f) { register_builtin_parts(); feed_forwards()[kind] = std::move(f); }
void register_block(const std::string& kind, BlockFactory f) { register_builtin_parts(); blocks()[kind] = std::move(f); }

bool has_part(const std::string& category, const std::string& kind) {
    register_builtin_parts();
    if (category == "norm") return norms().count(kind) != 0;
    if (category == "mixer") return mixers().count(kind) != 0;
    if (category == "feed_forward") return feed_forwards().count(kind) != 0;
    if (category == "block") return blocks().count(kind) != 0;
    return false;
}

std::unique_ptr<Norm> build_norm(const std::string& kind, const Params& p) {
    register_builtin_parts();
    auto it = norms().find(kind);
    if (it == norms().end()) fail("unknown norm '%s'; registered: %s", kind.c_str(), known(norms()).c_str());
    return it->second(p);
}
std::unique_ptr<Mixer> build_mixer(const std::string& kind, const Params& p) {
    register_builtin_parts();
    auto it = mixers().find(kind);
    if (it == mixers().end()) fail("unknown mixer '%s'; registered: %s", kind.c_str(), known(mixers()).c_str());
    return it->second(p);
}
std::unique_ptr<FeedForward> build_feed_forward(const std::string& kind, const Params& p) {
    register_builtin_parts();
    auto it = feed_forwards().find(kind);
    if (it == feed_forwards().end()) fail("unknown feed-forward '%s'; registered: %s", kind.c_str(), known(feed_forwards()).c_str());
    return it->second(p);
}
std::unique_ptr<Block> build_block(const std::string& kind, std::unique_ptr<Mixer> m, std::unique_ptr<FeedForward> f,
                                   std::vector<std::unique_ptr<Norm>> n) {
    register_builtin_parts();
    auto it = blocks().find(kind);
    if (it == blocks().end()) fail("unknown block arrangement '%s'; registered: %s", kind.c_str(), known(blocks()).c_str());
    return it->second(std::move(m), std::move(f), std::move(n));
}

// ---------------------------------------------------------------------------------------------
size_t DecoderModel::workspace_bytes(int tokens, int n_logits) const {
    size_t per_layer = 0;
    for (const auto& l : layers) per_layer = std::max(per_layer, l->workspace_bytes(tokens));
    const size_t stream = static_cast<size_t>(tokens) * hidden_size() * 4 + 256;
    const size_t head = final_norm ? 2 * final_norm->workspace_bytes(std::max(n_logits, 1)) : 0;
    return stream + std::max(per_layer, head) + 4096;
}

void DecoderModel::forward(const StepView& step, const std::vector<CacheView>& caches, Arena& arena,
                           const Tensor2& logits, hipStream_t s) const {
    if (step.n_tokens < 1) fail("a step needs at least one token");
    // x[t,:] = wte[id[t],:] (+ the position table's row, fused into the same kernel)
    StageTimes& times = StageTimes::get();
    times.begin_step(step.max_q_len == 1 ? "decode" : (step.n_single > 0 ? "mixed" : "prefill"), step.n_seqs, step.n_tokens, s);
    Tensor2 x = arena.tensor(F32, step.n_tokens, hidden_size());
    embed(step.token_ids, step.positions, wte, wpe.data ? &wpe : nullptr, x, s);
    times.mark("embed", s);
    for (const LayerCall& c : order) {
        if (c.layer < 0 || c.layer >= static_cast<int>(layers.size()) || c.cache < 0 || c.cache >= static_cast<int>(caches.size()))
            fail("the execution order names layer %d / cache %d, the model has %zu layers and %zu caches", c.layer, c.cache,
                 layers.size(), caches.size());
        times.set_layer(c.layer);
        layers[c.layer]->forward(x, step, caches[c.cache], c.write, arena, s);
    }
    times.set_layer(-1);
    if (step.n_logits == 0) { times.end_step(s); return; }
    // logits = norm(x[rows]) wte^T, fp32, no bias: the embedding matrix [V, D] is read in place as the
    // [N, K] operand (the reference builds a transposed copy: /root/reference/src/model/gpt2_model.cu:87-113)
    if (logits.rows != step.n_logits || logits.cols != vocab_size() || logits.dtype != F32)
        fail("logits must be float32 [%d, %d]", step.n_logits, vocab_size());
    Linear head(wte, nullptr);
    final_norm->linear(x, head, logits, STORE_F32, step.logit_rows, nullptr, arena, s);
    times.mark("head", s);
    times.end_step(s);
}

}  // namespace minillm
