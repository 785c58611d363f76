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
    // (said when the model is built, not at its first step: the bfloat16 products read 16 bytes at a time)
    if (w.dtype == BF16 && (w.cols % 8 != 0 || w.stride % 8 != 0))
        fail("a linear map of %lld inputs has no bfloat16 kernel: the number of inputs must be a multiple of 8 (float32 takes any)",
             (long long)w.cols);
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
        h_ = norm_->forward(x_, nullptr, static_cast<int>(x_.rows), arena, s);
        have_ = true;
    }
    return h_;
}

void NormedInput::linear(const Linear& lin, const Tensor2& out, int epilogue, const KvScatter* kv, Arena& arena,
                         hipStream_t s) {
    if (have_) lin(h_, out, epilogue, kv, s);
    else norm_->linear(x_, lin, out, epilogue, nullptr, kv, arena, s);
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
    void add_cost(StepCost& c) const override { c.weight_bytes += 4.0 * size_ * (beta_ ? 2 : 1); }

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
        if (p.position && p.position->applies_in_mixer()) position_ = p.position;
    }
    void forward(NormedInput& h, const StepView& step, const CacheView& cache, const Tensor2& x, bool write, Arena& arena,
                 hipStream_t s) const override {
        if (cache.kind != 1) fail("attention needs a cache of pages");
        const int T = step.n_tokens, g = cache.group;
        Tensor2 qkv = arena.tensor(dtype_, T, q_dim_ + 2 * kv_dim_);
        // Prompt portions: the QKV product is asked to put the new keys and values into the pages (how
        // is the linear map's business). Single tokens: the attention kernel writes them.
        // A position encoding that turns queries and keys does so on the qkv rows first: the keys are final
        // only then, so they go to the pages afterwards (by the attention op), not from the product.
        const bool scatter = write && step.max_q_len > 1 && !position_;
        KvScatter kv;
        if (scatter) {
            kv.slots = step.slots[g];
            kv.k_pages = cache.k_pages;
            kv.v_pages = cache.v_pages;
            kv.q_cols = q_dim_;
        }
        h.linear(qkv_, qkv, STORE, scatter ? &kv : nullptr, arena, s);
        if (position_) position_->in_mixer(qkv, n_heads_, n_kv_heads_, head_dim_, step, s);
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
    CacheNeed cache_need() const override {
        CacheNeed n;
        n.kind = 1; n.n_kv_heads = n_kv_heads_; n.head_dim = head_dim_; n.window = window_;
        return n;
    }
    void reserve(int max_seqs, hipStream_t s) const override {
        reserve_attention_scratch((max_seqs + 7) / 8 * 8, n_heads_, head_dim_, s);
        reserve_linear_scratch(s);
    }
    void add_cost(StepCost& c) const override {
        qkv_.add_cost(c);
        out_.add_cost(c);
        c.attention_flops_per_key += 4.0 * q_dim_;        // q.k and p.v, a multiply and an add each
        if (position_) position_->add_cost(c);
    }

private:
    int n_heads_ = 0, n_kv_heads_ = 0, head_dim_ = 0, window_ = 0, q_dim_ = 0, kv_dim_ = 0, dtype_ = BF16;
    float scale_ = 1.f;
    Linear qkv_, out_;
    std::shared_ptr<const PositionEncoding> position_;     // only one that works inside the mixer
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
    void reserve(int, hipStream_t s) const override { reserve_linear_scratch(s); }
    void add_cost(StepCost& c) const override { up_.add_cost(c); down_.add_cost(c); }

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
        if (!mixer_) fail("a pre-norm block needs a mixer");
        if (norms.size() != (ff_ ? 2u : 1u)) fail("a pre-norm block has one norm per sub-layer (%d here), got %zu", ff_ ? 2 : 1, norms.size());
        norm1_ = std::move(norms[0]);
        if (ff_) norm2_ = std::move(norms[1]);
    }
    void forward(const Tensor2& x, const StepView& step, const CacheView& cache, bool write, Arena& arena,
                 hipStream_t s) const override {
        size_t mark = arena.mark();
        {
            NormedInput h(*norm1_, x);
            mixer_->forward(h, step, cache, x, write, arena, s);
        }
        arena.release(mark);
        if (!ff_) return;                              // a layer without a feed-forward
        {
            NormedInput h(*norm2_, x);
            ff_->forward(h, step, x, arena, s);
        }
        arena.release(mark);
    }
    size_t workspace_bytes(int tokens) const override {
        const size_t a = mixer_->workspace_bytes(tokens) + 2 * norm1_->workspace_bytes(tokens);
        return ff_ ? std::max(a, ff_->workspace_bytes(tokens) + 2 * norm2_->workspace_bytes(tokens)) : a;
    }
    CacheNeed cache_need() const override { return mixer_->cache_need(); }
    void reserve(int max_seqs, hipStream_t s) const override {
        mixer_->reserve(max_seqs, s);
        if (ff_) ff_->reserve(max_seqs, s);
    }
    void add_cost(StepCost& c) const override {
        norm1_->add_cost(c);
        mixer_->add_cost(c);
        if (ff_) { norm2_->add_cost(c); ff_->add_cost(c); }
    }

private:
    std::unique_ptr<Mixer> mixer_;
    std::unique_ptr<FeedForward> ff_;
    std::unique_ptr<Norm> norm1_, norm2_;
};

// Learned absolute positions: row pos[t] of a table is added to the token's embedding, in the embedding
// kernel (/root/reference/src/kernels/embedding.cu:23-43).
class LearnedAbsolutePositions final : public PositionEncoding {
public:
    explicit LearnedAbsolutePositions(const Params& p) : table_(p.weights("table")) {}
    const Tensor2* table() const override { return &table_; }
    int max_positions() const override { return static_cast<int>(table_.rows); }

private:
    Tensor2 table_;         // [P, D]
};

// x[t,:] = table[id[t],:] (+ the position table's row), into the fp32 stream.
class TokenTable final : public Embedding {
public:
    explicit TokenTable(const Params& p) : table_(p.weights("table")) {}
    int vocab_size() const override { return static_cast<int>(table_.rows); }
    int hidden_size() const override { return static_cast<int>(table_.cols); }
    void forward(const StepView& step, const PositionEncoding* position, const Tensor2& x, hipStream_t s) const override {
        embed(step.token_ids, step.positions, table_, position ? position->table() : nullptr, x, s, &step.fed);
    }
    bool resolves_fed_tokens() const override { return true; }

private:
    Tensor2 table_;         // [V, D]
};

// logits = norm(x[rows]) W^T (+ b), fp32. `weight` is [V, D]: a tied head is handed the embedding's table
// and reads it in place as the [N, K] operand (the reference builds a transposed copy:
// /root/reference/src/model/gpt2_model.cu:87-113); an untied head owns its matrix.
class LinearHead final : public Head {
public:
    explicit LinearHead(const Params& p) : lin_(p.weights("weight"), p.weights_or_null("bias")), dtype_(p.integer("dtype")) {}
    int vocab_size() const override { return lin_.out_features(); }
    void forward(const Tensor2& x, const Norm& final_norm, const int* rows, const Tensor2& logits, Arena& arena,
                 hipStream_t s) const override {
        // (the norm gathers the wanted rows and, where the kernels allow, is fused into the product)
        final_norm.linear(x, lin_, logits, STORE_F32, rows, nullptr, arena, s);
    }
    size_t workspace_bytes(int rows) const override {
        return static_cast<size_t>(rows) * lin_.in_features() * dtype_size(dtype_) + 512;
    }
    void add_cost(StepCost& c) const override {
        c.weight_bytes += static_cast<double>(lin_.weight.rows) * lin_.weight.cols * lin_.weight.esz() + (lin_.bias ? 4.0 * lin_.weight.rows : 0.0);
        c.flops_per_logits_row += 2.0 * lin_.weight.rows * lin_.weight.cols;
    }

private:
    Linear lin_;
    int dtype_ = BF16;
};

// ---------------------------------------------------------------------------------------------
// registries: kind name -> factory, one per category of part
// ---------------------------------------------------------------------------------------------
namespace {
template <typename F>
struct Registry {
    const char* what;
    std::map<std::string, F> kinds;
    const F& get(const std::string& kind) const {
        auto it = kinds.find(kind);
        if (it == kinds.end()) {
            std::string known;
            for (const auto& kv : kinds) known += (known.empty() ? "" : ", ") + kv.first;
            fail("unknown %s '%s'; registered: %s", what, kind.c_str(), known.c_str());
        }
        return it->second;
    }
};
Registry<PositionFactory>& positions() { static Registry<PositionFactory> r{"position encoding", {}}; return r; }
Registry<EmbeddingFactory>& embeddings() { static Registry<EmbeddingFactory> r{"embedding", {}}; return r; }
Registry<HeadFactory>& heads() { static Registry<HeadFactory> r{"head", {}}; return r; }
Registry<NormFactory>& norms() { static Registry<NormFactory> r{"norm", {}}; return r; }
Registry<MixerFactory>& mixers() { static Registry<MixerFactory> r{"mixer", {}}; return r; }
Registry<FeedForwardFactory>& feed_forwards() { static Registry<FeedForwardFactory> r{"feed-forward", {}}; return r; }
Registry<BlockFactory>& blocks() { static Registry<BlockFactory> r{"block arrangement", {}}; return r; }

void register_builtin_parts() {
    static bool done = false;
    if (done) return;
    done = true;
    positions().kinds["learned_absolute"] = [](const Params& p) { return std::shared_ptr<const PositionEncoding>(new LearnedAbsolutePositions(p)); };
    embeddings().kinds["token_table"] = [](const Params& p) { return std::unique_ptr<Embedding>(new TokenTable(p)); };
    heads().kinds["linear"] = [](const Params& p) { return std::unique_ptr<Head>(new LinearHead(p)); };
    norms().kinds["layernorm"] = [](const Params& p) { return std::unique_ptr<Norm>(new LayerNorm(p)); };
    mixers().kinds["causal_attention"] = [](const Params& p) { return std::unique_ptr<Mixer>(new CausalSelfAttention(p)); };
    feed_forwards().kinds["dense_mlp"] = [](const Params& p) { return std::unique_ptr<FeedForward>(new DenseMLP(p)); };
    blocks().kinds["pre_norm"] = [](std::unique_ptr<Mixer> m, std::unique_ptr<FeedForward> f, std::vector<std::unique_ptr<Norm>> n) {
        return std::unique_ptr<Block>(new PreNormBlock(std::move(m), std::move(f), std::move(n)));
    };
}
}  // namespace

void register_position(const std::string& kind, PositionFactory f) { register_builtin_parts(); positions().kinds[kind] = std::move(f); }
void register_embedding(const std::string& kind, EmbeddingFactory f) { register_builtin_parts(); embeddings().kinds[kind] = std::move(f); }
void register_head(const std::string& kind, HeadFactory f) { register_builtin_parts(); heads().kinds[kind] = std::move(f); }
void register_norm(const std::string& kind, NormFactory f) { register_builtin_parts(); norms().kinds[kind] = std::move(f); }
void register_mixer(const std::string& kind, MixerFactory f) { register_builtin_parts(); mixers().kinds[kind] = std::move(f); }
void register_feed_forward(const std::string& kind, FeedForwardFactory f) { register_builtin_parts(); feed_forwards().kinds[kind] = std::move(f); }
void register_block(const std::string& kind, BlockFactory f) { register_builtin_parts(); blocks().kinds[kind] = std::move(f); }

bool has_part(const std::string& category, const std::string& kind) {
    register_builtin_parts();
    if (category == "position") return positions().kinds.count(kind) != 0;
    if (category == "embedding") return embeddings().kinds.count(kind) != 0;
    if (category == "head") return heads().kinds.count(kind) != 0;
    if (category == "norm") return norms().kinds.count(kind) != 0;
    if (category == "mixer") return mixers().kinds.count(kind) != 0;
    if (category == "feed_forward") return feed_forwards().kinds.count(kind) != 0;
    if (category == "block") return blocks().kinds.count(kind) != 0;
    return false;
}

std::shared_ptr<const PositionEncoding> build_position(const std::string& kind, const Params& p) {
    register_builtin_parts();
    return positions().get(kind)(p);
}
std::unique_ptr<Embedding> build_embedding(const std::string& kind, const Params& p) {
    register_builtin_parts();
    return embeddings().get(kind)(p);
}
std::unique_ptr<Head> build_head(const std::string& kind, const Params& p) {
    register_builtin_parts();
    return heads().get(kind)(p);
}
std::unique_ptr<Norm> build_norm(const std::string& kind, const Params& p) {
    register_builtin_parts();
    return norms().get(kind)(p);
}
std::unique_ptr<Mixer> build_mixer(const std::string& kind, const Params& p) {
    register_builtin_parts();
    return mixers().get(kind)(p);
}
std::unique_ptr<FeedForward> build_feed_forward(const std::string& kind, const Params& p) {
    register_builtin_parts();
    return feed_forwards().get(kind)(p);
}
std::unique_ptr<Block> build_block(const std::string& kind, std::unique_ptr<Mixer> m, std::unique_ptr<FeedForward> f,
                                   std::vector<std::unique_ptr<Norm>> n) {
    register_builtin_parts();
    return blocks().get(kind)(std::move(m), std::move(f), std::move(n));
}

// ---------------------------------------------------------------------------------------------
// the model
// ---------------------------------------------------------------------------------------------
static void check_order(const DecoderModel& m) {
    if (!m.embedding || !m.head || !m.final_norm) fail("a model needs an embedding, a final norm and a head");
    for (const LayerCall& c : m.order)
        if (c.layer < 0 || c.layer >= static_cast<int>(m.layers.size()) || c.cache < 0)
            fail("the execution order names layer %d / cache %d, the model has %zu layers", c.layer, c.cache, m.layers.size());
}

std::vector<CacheNeed> DecoderModel::cache_needs() const {
    check_order(*this);
    int n = 0;
    for (const LayerCall& c : order) n = std::max(n, c.cache + 1);
    std::vector<CacheNeed> needs(n);
    std::vector<bool> written(n, false);
    for (const LayerCall& c : order) {
        if (!c.write) continue;
        if (written[c.cache]) fail("cache %d is written by two calls of the execution order", c.cache);
        needs[c.cache] = layers[c.layer]->cache_need();
        written[c.cache] = true;
    }
    for (const LayerCall& c : order) {
        if (c.write) continue;
        if (!written[c.cache]) fail("cache %d is read by layer %d but no call writes it", c.cache, c.layer);
        // a call that only reads must see the cache as the kind of pages or state it would write itself
        const CacheNeed mine = layers[c.layer]->cache_need(), theirs = needs[c.cache];
        if (mine.kind != theirs.kind || mine.n_kv_heads != theirs.n_kv_heads || mine.head_dim != theirs.head_dim ||
            mine.state_bytes != theirs.state_bytes)
            fail("layer %d reads cache %d, which another kind of mixer writes", c.layer, c.cache);
    }
    return needs;
}

void DecoderModel::reserve(int max_seqs, hipStream_t s) const {
    for (const auto& l : layers) l->reserve(max_seqs, s);
    reserve_linear_scratch(s);
}

StepCost DecoderModel::cost() const {
    check_order(*this);
    StepCost c;
    // weights: every layer that the order names, once; flops: once per call
    std::vector<bool> seen(layers.size(), false);
    for (const LayerCall& call : order) {
        StepCost one;
        layers[call.layer]->add_cost(one);
        if (!seen[call.layer]) c.weight_bytes += one.weight_bytes;
        seen[call.layer] = true;
        c.flops_per_token += one.flops_per_token;
        c.attention_flops_per_key += one.attention_flops_per_key;
    }
    final_norm->add_cost(c);
    head->add_cost(c);
    return c;
}

// ---------------------------------------------------------------------------------------------
size_t DecoderModel::workspace_bytes(int tokens, int n_logits) const {
    size_t per_layer = 0;
    for (const auto& l : layers) per_layer = std::max(per_layer, l->workspace_bytes(tokens));
    const size_t stream = static_cast<size_t>(tokens) * hidden_size() * 4 + 256;
    const int rows = std::max(n_logits, 1);
    const size_t at_head = head->workspace_bytes(rows) + 2 * final_norm->workspace_bytes(rows);
    return stream + std::max(per_layer, at_head) + 4096;
}

void DecoderModel::forward(const StepView& step, const std::vector<CacheView>& caches, Arena& arena,
                           const Tensor2& logits, hipStream_t s) const {
    if (step.n_tokens < 1) fail("a step needs at least one token");
    check_order(*this);
    StageTimes& times = StageTimes::get();
    times.begin_step(step.max_q_len == 1 ? "decode" : (step.n_single > 0 ? "mixed" : "prefill"), step.n_seqs, step.n_tokens, s);
    Tensor2 x = arena.tensor(F32, step.n_tokens, hidden_size());
    embedding->forward(step, position.get(), x, s);
    times.mark("embed", s);
    for (const LayerCall& c : order) {
        if (c.cache >= static_cast<int>(caches.size()))
            fail("the execution order names cache %d, the step brings %zu caches", c.cache, caches.size());
        times.set_layer(c.layer);
        layers[c.layer]->forward(x, step, caches[c.cache], c.write, arena, s);
    }
    times.set_layer(-1);
    if (step.n_logits == 0) { times.end_step(s); return; }
    if (logits.rows != step.n_logits || logits.cols != vocab_size() || logits.dtype != F32)
        fail("logits must be float32 [%d, %d]", step.n_logits, vocab_size());
    head->forward(x, *final_norm, step.logit_rows, logits, arena, s);
    times.mark("head", s);
    times.end_step(s);
}

}  // namespace minillm
