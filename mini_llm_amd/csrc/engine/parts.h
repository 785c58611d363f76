// The parts a model is put together from, natively: mixer, feed-forward, norm, block arrangement,
// and the model that runs them in the order its configuration gives.
//
// A part knows its own sizes and constants (parameters) and the tensors it owns; it does not know
// which model it is in. Parts are built by kind name through registries, from a bag of parameters
// (numbers, strings, device tensors), so that another kind of part is one class and one
// registration, and a configuration chooses layer by layer.
//
// Interfaces (`x` is the fp32 residual stream [T, hidden]; `h` a normalised activation in the
// compute dtype; `step` the batch's index arrays; `arena` memory for the step's temporaries):
//   Embedding::forward(step, position, x)     x[t,:] = the token's row (+ the position table's)
//   PositionEncoding::table() / in_mixer(qkv, heads, step)   a table for the embedding, or a turn of
//                                             queries and keys inside the mixer before keys are written
//   Norm::forward(x, rows, n) -> h            Norm::linear(x, lin, out, epilogue, rows)
//   Mixer::forward(h, step, cache, x, write)  adds the mixer's output into x
//   FeedForward::forward(h, step, x)          adds its output into x
//   Block::forward(x, step, cache, write)     runs one layer on the stream
//   Head::forward(x, final_norm, rows, logits)  fp32 logits of the wanted rows
// Every part also says what it asks of the cache (Mixer::cache_need), what scratch its kernels need
// (reserve), how much of the step's arena it takes (workspace_bytes) and what a step costs through it
// (add_cost: bytes of weights, flops).
//
// The reference's model has these pieces fixed in one class
// (/root/reference/src/model/gpt2_model.cu:275-363 block_prefill, :404-428 the head).
#pragma once

#include <functional>
#include <map>
#include <memory>
#include <string>
#include <vector>

#include "ops.h"

namespace minillm {

// Optional per-stage times of the native forward pass. With the environment variable MINI_LLM_STAGE_TIMES
// set, every step records an event behind each stage (embedding; per layer the QKV product with its norm,
// attention, output projection, first and second product of the feed-forward; final norm and head), waits
// for the step once at its end, and prints one line per stage to standard error in the reference's format
// `kind,batch_size,total_tokens,layer,stage,ms` (kind: prefill, decode or mixed)
// (/root/reference/include/profiling/stage_timer.cuh:13-101, which synchronises the device around every
// stage instead). Off: one branch per stage. A part of another kind marks its own stages with `mark`.
class StageTimes {
public:
    static StageTimes& get();
    bool enabled() const { return enabled_; }
    void begin_step(const char* kind, int batch, int tokens, hipStream_t s);
    void set_layer(int layer) { layer_ = layer; }
    void mark(const char* stage, hipStream_t s);        // the stage that ends here
    void end_step(hipStream_t s);                        // waits for the step and prints

private:
    StageTimes();
    hipEvent_t event(hipStream_t s);
    struct Mark { int layer; const char* stage; hipEvent_t at; };
    bool enabled_ = false, header_ = false;
    int layer_ = -1, batch_ = 0, tokens_ = 0;
    const char* kind_ = "";
    hipEvent_t start_ = nullptr;
    std::vector<Mark> marks_;
    std::vector<hipEvent_t> spare_;
};


// Memory for a step's temporaries: a bump allocator over one device buffer that the caller owns.
class Arena {
public:
    Arena(void* base, size_t bytes) : base_(static_cast<char*>(base)), capacity_(bytes) {}
    void* take(size_t bytes);
    Tensor2 tensor(int dtype, int64_t rows, int64_t cols) {
        return Tensor2(take(static_cast<size_t>(rows) * cols * dtype_size(dtype)), dtype, rows, cols);
    }
    size_t mark() const { return used_; }
    void release(size_t mark) { used_ = mark; }
    size_t peak() const { return peak_; }

private:
    char* base_;
    size_t capacity_, used_ = 0, peak_ = 0;
};

// The step's batch: sizes known to the host and device arrays (int32).
struct StepView {
    int n_tokens = 0, n_seqs = 0, n_logits = 0, max_q_len = 0, max_ctx_len = 0, n_single = 0;
    const int* token_ids = nullptr;    // [T]
    FedTokens fed;                     // tokens to take on the device from the step before (only if the model's embedding
                                       // says that it resolves them; otherwise token_ids holds every id already)
    const int* positions = nullptr;    // [T]
    const int* token_seq = nullptr;    // [T]
    const int* cu_q = nullptr;         // [B+1]
    const int* ctx_len = nullptr;      // [B]
    const int* starts = nullptr;       // [B]
    const int* state_slots = nullptr;  // [B]
    const int* logit_rows = nullptr;   // [n_logits]
    int n_groups = 0;
    const int* const* block_tables = nullptr;   // per group [B, max_blocks[g]]
    const int* max_blocks = nullptr;            // per group
    const int* const* slots = nullptr;          // per group [T]
};

// What a call of the execution order sees of its cache.
struct CacheView {
    int kind = 0;                  // 0 none, 1 pages of keys and values, 2 fixed-size state slots
    Tensor2 k_pages, v_pages;      // [n_pages * page_size, kv_dim]
    int group = 0, page_size = 0, window = 0;
    void* state = nullptr;         // [n_slots, slot_bytes]
    size_t slot_bytes = 0;
    int n_slots = 0;
};

// What a cache of the execution order asks of the cache manager: said by the mixer that writes it.
struct CacheNeed {
    int kind = 0;                        // 1 keys and values in pages, 2 fixed-size state, 0 none
    int n_kv_heads = 0, head_dim = 0, window = 0;
    size_t state_bytes = 0;
};

// What one step costs, summed over the parts (the benchmark's roofline figures are made from these).
struct StepCost {
    double weight_bytes = 0;             // weights a step reads once, whatever its batch
    double flops_per_token = 0;          // matrix products of the layers, per token
    double attention_flops_per_key = 0;  // per (token, attended key), summed over the attention calls
    double flops_per_logits_row = 0;     // the head's product for one wanted row
};

class PositionEncoding;

// A bag of parameters a part is built from.
struct Params {
    std::map<std::string, double> num;
    std::map<std::string, std::string> str;
    std::map<std::string, Tensor2> tensor;
    std::shared_ptr<const PositionEncoding> position;      // the model's position encoding, for mixers that take one

    double number(const std::string& key) const;
    double number(const std::string& key, double fallback) const;
    int integer(const std::string& key) const { return static_cast<int>(number(key)); }
    const std::string& string(const std::string& key) const;
    const Tensor2& weights(const std::string& key) const;          // must be there
    const Tensor2* weights_or_null(const std::string& key) const;
};

class Linear {
public:
    Linear() = default;
    // weight [out, in] in the compute dtype (k contiguous: the layout the matrix kernels read), bias fp32 [out] or none
    Linear(const Tensor2& weight, const Tensor2* bias);
    void operator()(const Tensor2& a, const Tensor2& out, int epilogue, const KvScatter* kv, hipStream_t s) const {
        linear(a, weight, bias, out, epilogue, kv, s);
    }
    Tensor2 weight;
    const float* bias = nullptr;
    int in_features() const { return static_cast<int>(weight.cols); }
    int out_features() const { return static_cast<int>(weight.rows); }
    void add_cost(StepCost& c) const {
        c.weight_bytes += static_cast<double>(weight.rows) * weight.cols * weight.esz() + (bias ? 4.0 * weight.rows : 0.0);
        c.flops_per_token += 2.0 * weight.rows * weight.cols;
    }
};

// How positions enter the model. Either a table whose row is added to the token's embedding (learned
// absolute positions: the embedding kernel adds it), or a turn of queries and keys inside the mixer,
// in place on the qkv rows, before the keys go to the pages (rotary schemes), or nothing.
class PositionEncoding {
public:
    virtual ~PositionEncoding() = default;
    virtual const Tensor2* table() const { return nullptr; }
    virtual bool applies_in_mixer() const { return false; }
    // qkv rows: n_heads query heads, then n_kv_heads key heads, then the values (left alone)
    virtual void in_mixer(const Tensor2& qkv, int n_heads, int n_kv_heads, int head_dim, const StepView& step,
                          hipStream_t s) const {
        (void)qkv; (void)n_heads; (void)n_kv_heads; (void)head_dim; (void)step; (void)s;
    }
    virtual int max_positions() const { return 0; }       // 0: unbounded
    virtual void add_cost(StepCost&) const {}
};

// Token ids to rows of the fp32 stream.
class Embedding {
public:
    virtual ~Embedding() = default;
    virtual int vocab_size() const = 0;
    virtual int hidden_size() const = 0;
    virtual void forward(const StepView& step, const PositionEncoding* position, const Tensor2& x, hipStream_t s) const = 0;
    // true: forward() takes `step.fed` into account itself (one kernel fewer in a decode step); false: the runner
    // writes the fed ids into token_ids with a kernel of its own before the step
    virtual bool resolves_fed_tokens() const { return false; }
    virtual void add_cost(StepCost&) const {}
};

class Norm {
public:
    virtual ~Norm() = default;
    // h[i,:] = norm(x[rows ? rows[i] : i, :]), n rows, from the arena
    virtual Tensor2 forward(const Tensor2& x, const int* rows, int n, Arena& arena, hipStream_t s) const = 0;
    // out = epilogue(lin(norm(x[rows]))); a norm with a fused kernel overrides this
    // (kv: a key/value scatter of the linear map, passed through to it)
    virtual void linear(const Tensor2& x, const Linear& lin, const Tensor2& out, int epilogue, const int* rows,
                        const KvScatter* kv, Arena& arena, hipStream_t s) const;
    virtual size_t workspace_bytes(int rows) const = 0;
    virtual void add_cost(StepCost&) const {}
    int dtype = BF16;
};

// The input of a sub-layer as (stream, norm), not yet normalised: a part's first linear map may
// absorb the norm.
class NormedInput {
public:
    NormedInput(const Norm& norm, const Tensor2& x) : norm_(&norm), x_(x) {}
    explicit NormedInput(const Tensor2& h) : norm_(nullptr), x_(h), h_(h), have_(true) {}     // normalised already
    const Tensor2& tensor(Arena& arena, hipStream_t s);
    void linear(const Linear& lin, const Tensor2& out, int epilogue, const KvScatter* kv, Arena& arena, hipStream_t s);
    int64_t rows() const { return x_.rows; }

private:
    const Norm* norm_;
    Tensor2 x_, h_;
    bool have_ = false;
};

class Mixer {
public:
    virtual ~Mixer() = default;
    virtual void forward(NormedInput& h, const StepView& step, const CacheView& cache, const Tensor2& x, bool write,
                         Arena& arena, hipStream_t s) const = 0;
    virtual size_t workspace_bytes(int tokens) const = 0;
    virtual CacheNeed cache_need() const = 0;
    // Scratch that the mixer's kernels need on stream `s` for steps of up to max_seqs sequences: taken
    // now, so that no step allocates.
    virtual void reserve(int max_seqs, hipStream_t s) const { (void)max_seqs; (void)s; }
    virtual void add_cost(StepCost&) const {}
};

class FeedForward {
public:
    virtual ~FeedForward() = default;
    virtual void forward(NormedInput& h, const StepView& step, const Tensor2& x, Arena& arena, hipStream_t s) const = 0;
    virtual size_t workspace_bytes(int tokens) const = 0;
    virtual void reserve(int max_seqs, hipStream_t s) const { (void)max_seqs; (void)s; }
    virtual void add_cost(StepCost&) const {}
};

class Block {
public:
    virtual ~Block() = default;
    virtual void forward(const Tensor2& x, const StepView& step, const CacheView& cache, bool write, Arena& arena,
                         hipStream_t s) const = 0;
    virtual size_t workspace_bytes(int tokens) const = 0;
    virtual CacheNeed cache_need() const = 0;             // its mixer's
    virtual void reserve(int max_seqs, hipStream_t s) const = 0;
    virtual void add_cost(StepCost&) const = 0;
};

// The stream's wanted rows to fp32 logits.
class Head {
public:
    virtual ~Head() = default;
    virtual int vocab_size() const = 0;
    // logits[i,:] = head(final_norm(x[rows[i],:]))
    virtual void forward(const Tensor2& x, const Norm& final_norm, const int* rows, const Tensor2& logits, Arena& arena,
                         hipStream_t s) const = 0;
    virtual size_t workspace_bytes(int rows) const = 0;
    virtual void add_cost(StepCost&) const {}
};

// -- registries: kind name -> factory ---------------------------------------------------------------
using PositionFactory = std::function<std::shared_ptr<const PositionEncoding>(const Params&)>;
using EmbeddingFactory = std::function<std::unique_ptr<Embedding>(const Params&)>;
using HeadFactory = std::function<std::unique_ptr<Head>(const Params&)>;
using NormFactory = std::function<std::unique_ptr<Norm>(const Params&)>;
using MixerFactory = std::function<std::unique_ptr<Mixer>(const Params&)>;
using FeedForwardFactory = std::function<std::unique_ptr<FeedForward>(const Params&)>;
using BlockFactory = std::function<std::unique_ptr<Block>(std::unique_ptr<Mixer>, std::unique_ptr<FeedForward>,
                                                         std::vector<std::unique_ptr<Norm>>)>;
void register_position(const std::string& kind, PositionFactory f);
void register_embedding(const std::string& kind, EmbeddingFactory f);
void register_head(const std::string& kind, HeadFactory f);
void register_norm(const std::string& kind, NormFactory f);
void register_mixer(const std::string& kind, MixerFactory f);
void register_feed_forward(const std::string& kind, FeedForwardFactory f);
void register_block(const std::string& kind, BlockFactory f);
// category: position | embedding | head | norm | mixer | feed_forward | block
bool has_part(const std::string& category, const std::string& kind);
std::shared_ptr<const PositionEncoding> build_position(const std::string& kind, const Params& p);
std::unique_ptr<Embedding> build_embedding(const std::string& kind, const Params& p);
std::unique_ptr<Head> build_head(const std::string& kind, const Params& p);
std::unique_ptr<Norm> build_norm(const std::string& kind, const Params& p);
std::unique_ptr<Mixer> build_mixer(const std::string& kind, const Params& p);
std::unique_ptr<FeedForward> build_feed_forward(const std::string& kind, const Params& p);
// (the feed-forward may be null: a layer without one; the norms are those of the sub-layers that exist)
std::unique_ptr<Block> build_block(const std::string& kind, std::unique_ptr<Mixer> m, std::unique_ptr<FeedForward> f,
                                   std::vector<std::unique_ptr<Norm>> norms);

// One entry of the execution order: which layer runs, on which cache, and whether it writes it.
struct LayerCall {
    int layer = 0, cache = 0;
    bool write = true;
};

// A decoder-only model: the embedding (with the position encoding's table, if it has one), the calls
// of the execution order, and the final norm and the head on the wanted rows only.
class DecoderModel {
public:
    std::unique_ptr<Embedding> embedding;
    std::shared_ptr<const PositionEncoding> position;     // may be null: no position encoding
    std::vector<std::unique_ptr<Block>> layers;
    std::vector<LayerCall> order;
    std::unique_ptr<Norm> final_norm;
    std::unique_ptr<Head> head;
    int dtype = BF16;

    int vocab_size() const { return head->vocab_size(); }
    int hidden_size() const { return embedding->hidden_size(); }
    // What each cache index of the execution order asks for: the need of the layer that writes it.
    std::vector<CacheNeed> cache_needs() const;
    // Every part takes the scratch its kernels need on `s` for steps of up to max_seqs sequences.
    void reserve(int max_seqs, hipStream_t s) const;
    StepCost cost() const;
    // Bytes of arena that a step of `tokens` tokens and `n_logits` wanted rows needs at most.
    size_t workspace_bytes(int tokens, int n_logits) const;
    // Runs the step; fp32 logits [n_logits, V] into `logits` (untouched if no logits are wanted).
    void forward(const StepView& step, const std::vector<CacheView>& caches, Arena& arena, const Tensor2& logits,
                 hipStream_t s) const;
};

}  // namespace minillm
