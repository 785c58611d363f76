#include "engine.h"

#include <algorithm>
#include <cmath>
#include <cstring>
#include <set>

namespace minillm {

#define HIP_OK(expr)                                                                              \
    do {                                                                                          \
        hipError_t e_ = (expr);                                                                   \
        if (e_ != hipSuccess) throw EngineError(std::string(#expr) + ": " + hipGetErrorString(e_)); \
    } while (0)

float uniform01(uint64_t seed, uint64_t index) {
    const uint64_t h = splitmix64(splitmix64(seed) ^ index);
    return static_cast<float>(h >> 40) / static_cast<float>(1 << 24);
}

// ---------------------------------------------------------------------------------------------
// cache storage
// ---------------------------------------------------------------------------------------------
CacheStorage::CacheStorage(const std::vector<CacheNeed>& needs, int page_size, int n_pages, int n_state_slots, int dtype)
    : page_size_(page_size), dtype_(dtype) {
    if (page_size < 1 || n_pages < 0 || n_state_slots < 1) throw EngineError("cache: bad page size, page count or slot count");
    try {
        allocate(needs, n_pages, n_state_slots);
    } catch (...) {
        for (void* p : allocations_) (void)hipFree(p);    // (no destructor runs for a constructor that throws)
        throw;
    }
}

void CacheStorage::allocate(const std::vector<CacheNeed>& needs, int n_pages, int n_state_slots) {
    const int page_size = page_size_, dtype = dtype_;
    struct Key { int hkv, hd, window; bool operator==(const Key& o) const { return hkv == o.hkv && hd == o.hd && window == o.window; } };
    std::vector<Key> keys;
    std::vector<std::vector<int>> members;
    std::vector<int> group_of(needs.size(), -1);
    for (size_t c = 0; c < needs.size(); ++c) {
        if (needs[c].kind != 1) continue;
        const Key k{needs[c].n_kv_heads, needs[c].head_dim, needs[c].window};
        size_t g = 0;
        while (g < keys.size() && !(keys[g] == k)) ++g;
        if (g == keys.size()) { keys.push_back(k); members.emplace_back(); }
        members[g].push_back(static_cast<int>(c));
        group_of[c] = static_cast<int>(g);
    }
    views_.resize(needs.size());
    const size_t esz = dtype_size(dtype);
    for (size_t g = 0; g < keys.size(); ++g) {
        GroupSpec gs;
        gs.page_size = page_size;
        gs.n_pages = n_pages;
        gs.window = keys[g].window;
        group_specs_.push_back(gs);
        const int64_t rows = static_cast<int64_t>(n_pages) * page_size, kv_dim = static_cast<int64_t>(keys[g].hkv) * keys[g].hd;
        const size_t one = static_cast<size_t>(rows) * kv_dim * esz;
        const size_t bytes = one * 2 * members[g].size();
        void* pool = nullptr;
        HIP_OK(hipMalloc(&pool, std::max<size_t>(bytes, 16)));
        allocations_.push_back(pool);
        allocation_bytes_.push_back(bytes);
        HIP_OK(hipMemset(pool, 0, std::max<size_t>(bytes, 16)));
        for (size_t j = 0; j < members[g].size(); ++j) {
            CacheView& v = views_[members[g][j]];
            v.kind = 1;
            v.k_pages = Tensor2(static_cast<char*>(pool) + (2 * j) * one, dtype, rows, kv_dim);
            v.v_pages = Tensor2(static_cast<char*>(pool) + (2 * j + 1) * one, dtype, rows, kv_dim);
            v.group = static_cast<int>(g);
            v.page_size = page_size;
            v.window = keys[g].window;
            bytes_per_token_ += 2 * static_cast<size_t>(kv_dim) * esz;
        }
    }
    for (size_t c = 0; c < needs.size(); ++c) {
        if (needs[c].kind != 2) continue;
        void* state = nullptr;
        const size_t bytes = needs[c].state_bytes * n_state_slots;
        HIP_OK(hipMalloc(&state, std::max<size_t>(bytes, 16)));
        allocations_.push_back(state);
        allocation_bytes_.push_back(bytes);
        HIP_OK(hipMemset(state, 0, std::max<size_t>(bytes, 16)));
        views_[c].kind = 2;
        views_[c].state = state;
        views_[c].slot_bytes = needs[c].state_bytes;
        views_[c].n_slots = n_state_slots;
    }
    manager_.reset(new CacheManager(group_specs_, n_state_slots));
}

CacheStorage::~CacheStorage() {
    for (void* p : allocations_) (void)hipFree(p);
}

void CacheStorage::reset_fresh_states(const StepView& step, hipStream_t s) const {
    for (const CacheView& v : views_)
        if (v.kind == 2) reset_state(v.state, v.slot_bytes, v.n_slots, step.state_slots, step.starts, step.n_seqs, s);
}

void CacheStorage::poison() {
    for (size_t i = 0; i < allocations_.size(); ++i) HIP_OK(hipMemset(allocations_[i], 0xFF, allocation_bytes_[i]));   // all-ones: NaN in bf16 and fp32
}

// ---------------------------------------------------------------------------------------------
// runner
// ---------------------------------------------------------------------------------------------
// Pages that `fraction` of the free device memory holds, for caches with these needs.
static int pages_for_memory_fraction(const std::vector<CacheNeed>& needs, int dtype, int page_size, double fraction) {
    if (fraction > 1.0) throw EngineError("kv_memory_fraction must be at most 1");
    size_t per_token = 0;
    for (const CacheNeed& n : needs)
        if (n.kind == 1) per_token += 2 * static_cast<size_t>(n.n_kv_heads) * n.head_dim * dtype_size(dtype);
    if (per_token == 0) return 1;
    size_t free_bytes = 0, total_bytes = 0;
    HIP_OK(hipMemGetInfo(&free_bytes, &total_bytes));
    // what later, small allocations may still want (buffers that grow, the runtime's own): kept out of the pool
    const size_t margin = std::min<size_t>(free_bytes / 50, size_t(1) << 30);
    const double pages = fraction * static_cast<double>(free_bytes - margin) / (static_cast<double>(per_token) * page_size);
    const double most = 2147483647.0 / page_size;          // rows of a pool are indexed with 32 bits
    if (pages < 1.0) throw EngineError("kv_memory_fraction leaves no room for a single page");
    return static_cast<int>(std::min(pages, most));
}

ModelRunner::ModelRunner(LoadedModel& model, const RunnerOptions& o)
    : model_(model), page_size_(o.page_size), n_pages_(o.n_pages), max_num_seqs_(std::max(o.max_num_seqs, 1)) {
    try {
        init(o);
    } catch (...) {
        destroy();                   // (no destructor runs for a constructor that throws)
        throw;
    }
}

ModelRunner::ModelRunner(LoadedModel& model, int page_size, int n_pages, int max_num_seqs)
    : model_(model), page_size_(page_size), n_pages_(n_pages), max_num_seqs_(std::max(max_num_seqs, 1)) {
    RunnerOptions o;
    o.page_size = page_size; o.n_pages = n_pages; o.max_num_seqs = max_num_seqs;
    try {
        init(o);
    } catch (...) {
        destroy();
        throw;
    }
}

void ModelRunner::init(const RunnerOptions& o) {
    HIP_OK(hipStreamCreate(&stream_));
    for (auto& st : staging_) HIP_OK(hipEventCreateWithFlags(&st.copied, hipEventDisableTiming));
    for (auto& e : host_tok_event_) HIP_OK(hipEventCreateWithFlags(&e, hipEventDisableTiming));
    // every part takes the scratch its kernels need, and the sampler its own, for the largest batch
    const int rows = (max_num_seqs_ + 7) / 8 * 8;
    model_.model.reserve(rows, stream_);
    reserve_sampling_scratch(rows, model_.model.vocab_size(), stream_);
    host_tok_cap_ = std::max(max_num_seqs_, 64) * 2;
    for (int i = 0; i < 2; ++i)
        HIP_OK(hipHostMalloc(reinterpret_cast<void**>(&host_tok_[i]), host_tok_cap_ * sizeof(int), hipHostMallocDefault));
    if (o.max_tokens_per_step > 0) {
        // the largest step's workspace, logits and index arrays now: nothing of that size is allocated in
        // the middle of serving, and a pool sized from the free memory leaves room for them
        const int T = std::max(o.max_tokens_per_step, max_num_seqs_);
        arena_for(T, max_num_seqs_);
        void* p = logits_;
        grow(&p, &logits_bytes_, static_cast<size_t>(max_num_seqs_) * model_.model.vocab_size() * sizeof(float));
        logits_ = static_cast<float*>(p);
        p = dev_ints_;
        size_t have = 0;
        const size_t max_blocks = model_.max_positions > 0 ? (model_.max_positions + page_size_ - 1) / page_size_ : 256;
        grow(&p, &have, (static_cast<size_t>(T) * (5 + 2 * model_.caches.size()) + static_cast<size_t>(max_num_seqs_) * (8 + max_blocks * model_.caches.size())) * sizeof(int));
        dev_ints_ = static_cast<int*>(p);
        dev_ints_cap_ = have / sizeof(int);
    }
    if (o.memory_fraction > 0.0) n_pages_ = pages_for_memory_fraction(model_.caches, model_.dtype, page_size_, o.memory_fraction);
    cache_.reset(new CacheStorage(model_.caches, page_size_, n_pages_, max_num_seqs_, model_.dtype));
}

ModelRunner::~ModelRunner() { destroy(); }

void ModelRunner::destroy() noexcept {
    if (stream_) (void)hipStreamSynchronize(stream_);
    cache_.reset();
    for (auto& st : staging_) {
        if (st.host) (void)hipHostFree(st.host);
        if (st.copied) (void)hipEventDestroy(st.copied);
    }
    for (int i = 0; i < 2; ++i) {
        if (host_tok_[i]) (void)hipHostFree(host_tok_[i]);
        if (host_tok_event_[i]) (void)hipEventDestroy(host_tok_event_[i]);
    }
    if (host_logits_) (void)hipHostFree(host_logits_);
    for (void* p : {static_cast<void*>(dev_ints_), arena_, static_cast<void*>(logits_), static_cast<void*>(tok_out_)})
        if (p) (void)hipFree(p);
    if (stream_) {
        try { release_scratch(stream_); } catch (...) {}
        (void)hipStreamDestroy(stream_);
        stream_ = nullptr;
    }
}

void ModelRunner::synchronize() { HIP_OK(hipStreamSynchronize(stream_)); }

void ModelRunner::grow(void** ptr, size_t* have, size_t need) {
    if (*ptr != nullptr && *have >= need) return;
    HIP_OK(hipStreamSynchronize(stream_));      // nothing in flight still reads the old buffer
    if (*ptr != nullptr) HIP_OK(hipFree(*ptr));
    const size_t bytes = need + need / 4 + 4096;
    HIP_OK(hipMalloc(ptr, bytes));
    *have = bytes;
}

void* ModelRunner::arena_for(int tokens, int n_logits) {
    grow(&arena_, &arena_bytes_, model_.model.workspace_bytes(tokens, n_logits));
    return arena_;
}

// Offsets of the step's int32 arrays in one packed buffer: token ids, positions, token_seq, cu_q, ctx_len,
// starts, state slots, logit rows; per group block tables and page rows; then the rows of the previous
// launch that tokens come from, temperatures and uniform numbers (as raw floats).
StepView ModelRunner::build(const std::vector<StepEntry>& entries, const std::vector<float>* temps,
                            const std::vector<float>* uniforms, const float** d_temps, const float** d_uniforms) {
    const int B = static_cast<int>(entries.size());
    if (B == 0) throw EngineError("a step needs at least one entry");
    CacheManager& mgr = manager();
    const int vocab = model_.model.vocab_size();
    std::vector<int64_t> ids(B);
    std::vector<int> n_tok(B);
    std::set<int64_t> seen;
    int T = 0, n_logits = 0, max_q = 0, max_ctx = 0;
    bool any_feed = false;
    for (int i = 0; i < B; ++i) {
        const StepEntry& e = entries[i];
        ids[i] = e.request_id;
        if (!seen.insert(e.request_id).second) throw EngineError("request " + std::to_string(e.request_id) + " appears twice in one step");
        n_tok[i] = static_cast<int>(e.tokens.size());
        if (n_tok[i] < 1) throw EngineError("request " + std::to_string(e.request_id) + ": an entry needs at least one token");
        for (int w : e.want)
            if (w < 0 || w >= n_tok[i])
                throw EngineError("request " + std::to_string(e.request_id) + ": wanted index " + std::to_string(w) + " is outside its " +
                                  std::to_string(n_tok[i]) + " tokens");
        const int len = mgr.length(e.request_id);
        if (len < 0) throw EngineError("request " + std::to_string(e.request_id) + " is not registered");
        if (model_.max_positions > 0 && len + n_tok[i] > model_.max_positions)
            throw EngineError("request " + std::to_string(e.request_id) + ": " + std::to_string(len + n_tok[i]) +
                              " tokens exceed the model's " + std::to_string(model_.max_positions) + " positions");
        if (e.feed_row >= 0) {
            if (n_tok[i] != 1) throw EngineError("only a single token can come from the previous launch");
            any_feed = true;
        }
        T += n_tok[i];
        n_logits += static_cast<int>(e.want.size());
        max_q = std::max(max_q, n_tok[i]);
        max_ctx = std::max(max_ctx, len + n_tok[i]);
    }
    const int G = cache_->n_groups();
    max_blocks_.assign(G, std::max(1, (max_ctx + page_size_ - 1) / page_size_));
    // layout
    std::vector<size_t> offs;
    size_t at = 0;
    auto seg = [&](size_t n) { offs.push_back(at); at += n; };
    seg(T); seg(T); seg(T); seg(B + 1); seg(B); seg(B); seg(B); seg(std::max(n_logits, 1));
    for (int g = 0; g < G; ++g) { seg(static_cast<size_t>(B) * max_blocks_[g]); seg(T); }
    const size_t o_src = at; at += T;
    const size_t o_temp = at; at += std::max(n_logits, 1);
    const size_t o_u = at; at += std::max(n_logits, 1);
    const size_t n_ints = at;
    // a pinned buffer whose last copy is done
    turn_ ^= 1;
    Staging& st = staging_[turn_];
    if (st.in_use) HIP_OK(hipEventSynchronize(st.copied));
    if (st.capacity < n_ints) {
        if (st.host) HIP_OK(hipHostFree(st.host));
        st.capacity = std::max<size_t>(n_ints, 4096) * 2;
        HIP_OK(hipHostMalloc(reinterpret_cast<void**>(&st.host), st.capacity * sizeof(int), hipHostMallocDefault));
    }
    int* h = st.host;
    if (mgr.fill_step_common(ids.data(), n_tok.data(), B, h + offs[1], h + offs[2], h + offs[3], h + offs[5], h + offs[4], h + offs[6]) != 0)
        throw EngineError("a request of the step is not registered");
    for (int g = 0; g < G; ++g)
        if (mgr.fill_step_group(ids.data(), n_tok.data(), B, g, max_blocks_[g], h + offs[8 + 2 * g], h + offs[9 + 2 * g]) != 0)
            throw EngineError("a request of the step holds no pages for its tokens (reserve before the step)");
    int t = 0, r = 0;
    for (int i = 0; i < B; ++i) {
        const StepEntry& e = entries[i];
        for (int k = 0; k < n_tok[i]; ++k) {
            const int tok = e.tokens[k];
            if (e.feed_row < 0 && (tok < 0 || tok >= vocab)) throw EngineError("token ids must lie in [0, " + std::to_string(vocab) + ")");
            h[offs[0] + t + k] = e.feed_row < 0 ? tok : 0;
            h[o_src + t + k] = e.feed_row;
        }
        for (int w : e.want) h[offs[7] + r++] = t + w;
        t += n_tok[i];
    }
    float* hf = reinterpret_cast<float*>(h);
    for (int i = 0; i < std::max(n_logits, 1); ++i) {
        hf[o_temp + i] = (temps != nullptr && i < static_cast<int>(temps->size())) ? (*temps)[i] : 0.f;
        hf[o_u + i] = (uniforms != nullptr && i < static_cast<int>(uniforms->size())) ? (*uniforms)[i] : 0.f;
    }
    {
        void* p = dev_ints_;
        size_t have = dev_ints_cap_ * sizeof(int);
        grow(&p, &have, n_ints * sizeof(int));
        dev_ints_ = static_cast<int*>(p);
        dev_ints_cap_ = have / sizeof(int);
    }
    HIP_OK(hipMemcpyAsync(dev_ints_, h, n_ints * sizeof(int), hipMemcpyHostToDevice, stream_));
    HIP_OK(hipEventRecord(st.copied, stream_));
    st.in_use = true;
    int n_single = B;
    for (int i = 0; i < B; ++i)
        if (n_tok[i] != 1) { n_single = i; break; }
    StepView sv;
    sv.n_tokens = T; sv.n_seqs = B; sv.n_logits = n_logits; sv.max_q_len = max_q; sv.max_ctx_len = max_ctx; sv.n_single = n_single;
    const int* d = dev_ints_;
    sv.token_ids = d + offs[0]; sv.positions = d + offs[1]; sv.token_seq = d + offs[2]; sv.cu_q = d + offs[3];
    sv.ctx_len = d + offs[4]; sv.starts = d + offs[5]; sv.state_slots = d + offs[6]; sv.logit_rows = d + offs[7];
    tables_.assign(G, nullptr);
    slots_.assign(G, nullptr);
    for (int g = 0; g < G; ++g) { tables_[g] = d + offs[8 + 2 * g]; slots_[g] = d + offs[9 + 2 * g]; }
    sv.n_groups = G;
    sv.block_tables = tables_.data();
    sv.max_blocks = max_blocks_.data();
    sv.slots = slots_.data();
    if (d_temps) *d_temps = reinterpret_cast<const float*>(d + o_temp);
    if (d_uniforms) *d_uniforms = reinterpret_cast<const float*>(d + o_u);
    if (any_feed) {
        if (tok_out_ == nullptr) throw EngineError("no earlier launch has sampled a token");
        if (model_.model.embedding->resolves_fed_tokens()) {
            sv.fed.src = d + o_src;
            sv.fed.prev = tok_out_;
            sv.fed.n_prev = tok_out_cap_;
        } else {
            select_tokens(dev_ints_ + offs[0], d + o_src, tok_out_, T, tok_out_cap_, stream_);
        }
    }
    return sv;
}

float* ModelRunner::run(const StepView& step) {
    cache_->reset_fresh_states(step, stream_);
    float* logits = nullptr;
    if (step.n_logits > 0) {
        void* p = logits_;
        grow(&p, &logits_bytes_, static_cast<size_t>(step.n_logits) * model_.model.vocab_size() * sizeof(float));
        logits_ = logits = static_cast<float*>(p);
    }
    void* arena = arena_for(step.n_tokens, step.n_logits);
    Arena a(arena, arena_bytes_);
    Tensor2 out = logits ? Tensor2(logits, F32, step.n_logits, model_.model.vocab_size()) : Tensor2();
    model_.model.forward(step, cache_->views(), a, out, stream_);
    return logits;
}

const float* ModelRunner::step(const std::vector<StepEntry>& entries, bool manage_cache, int* n_rows) {
    CacheManager& mgr = manager();
    std::vector<int64_t> fresh;
    if (manage_cache) {
        try {
            for (const StepEntry& e : entries) {
                if (!mgr.has_request(e.request_id)) {
                    if (mgr.add_request(e.request_id) < 0) throw EngineError("no free state slot");
                    fresh.push_back(e.request_id);
                }
                const int rc = mgr.reserve(e.request_id, mgr.length(e.request_id) + static_cast<int>(e.tokens.size()));
                if (rc == -1) throw EngineError("request " + std::to_string(e.request_id) + ": not enough free pages");
                if (rc != 0) throw EngineError("request " + std::to_string(e.request_id) + ": cannot reserve");
            }
        } catch (...) {
            for (int64_t id : fresh) mgr.free_request(id);
            throw;
        }
    }
    StepView sv;
    float* logits = nullptr;
    try {
        sv = build(entries, nullptr, nullptr, nullptr, nullptr);
        logits = run(sv);
    } catch (...) {
        for (int64_t id : fresh) mgr.free_request(id);       // a step that fails registers nothing
        throw;
    }
    if (manage_cache)
        for (const StepEntry& e : entries) mgr.commit(e.request_id, mgr.length(e.request_id) + static_cast<int>(e.tokens.size()));
    if (n_rows) *n_rows = logits != nullptr ? sv.n_logits : 0;
    if (logits != nullptr) {
        const size_t bytes = static_cast<size_t>(sv.n_logits) * model_.model.vocab_size() * sizeof(float);
        if (host_logits_bytes_ < bytes) {
            if (host_logits_) HIP_OK(hipHostFree(host_logits_));
            host_logits_ = nullptr;
            host_logits_bytes_ = bytes + bytes / 4;
            HIP_OK(hipHostMalloc(reinterpret_cast<void**>(&host_logits_), host_logits_bytes_, hipHostMallocDefault));
        }
        HIP_OK(hipMemcpyAsync(host_logits_, logits, bytes, hipMemcpyDeviceToHost, stream_));
    }
    HIP_OK(hipStreamSynchronize(stream_));
    return logits != nullptr ? host_logits_ : nullptr;
}

int ModelRunner::launch(const std::vector<StepEntry>& entries, const std::vector<float>& temperatures,
                        const std::vector<float>& uniforms) {
    if (pending_.size() >= 2) throw EngineError("two launches have tokens unread: collect() before a third");
    const float *d_temps = nullptr, *d_u = nullptr;
    const StepView sv = build(entries, &temperatures, &uniforms, &d_temps, &d_u);
    float* logits = run(sv);
    if (logits == nullptr) return 0;
    const int n = sv.n_logits;
    if (tok_out_cap_ < n) {
        // (sized for the most requests a step may hold, so this happens once; tokens that a later launch
        // may still take from the old buffer are kept)
        const int cap = std::max({n, (max_num_seqs_ + 7) / 8 * 8, 8});
        int* fresh = nullptr;
        HIP_OK(hipStreamSynchronize(stream_));
        HIP_OK(hipMalloc(reinterpret_cast<void**>(&fresh), cap * sizeof(int)));
        HIP_OK(hipMemset(fresh, 0, cap * sizeof(int)));
        if (tok_out_ != nullptr) {
            HIP_OK(hipMemcpy(fresh, tok_out_, tok_out_cap_ * sizeof(int), hipMemcpyDeviceToDevice));
            HIP_OK(hipFree(tok_out_));
        }
        tok_out_ = fresh;
        tok_out_cap_ = cap;
    }
    // two host buffers in turn: one may still be unread when the next step writes its own
    host_turn_ ^= 1;
    if (host_tok_cap_ < n) {
        HIP_OK(hipStreamSynchronize(stream_));
        if (!pending_.empty()) throw EngineError("tokens of an earlier launch are unread while the host buffers grow");
        host_tok_cap_ = std::max(n, 64) * 2;
        for (int i = 0; i < 2; ++i) {
            if (host_tok_[i]) HIP_OK(hipHostFree(host_tok_[i]));
            host_tok_[i] = nullptr;
            HIP_OK(hipHostMalloc(reinterpret_cast<void**>(&host_tok_[i]), host_tok_cap_ * sizeof(int), hipHostMallocDefault));
        }
    }
    // the sampling kernel writes the tokens to the device (for the next launch) and to the pinned host buffer
    // itself; the event behind it tells the host when they are there
    const Tensor2 lg(logits, F32, n, model_.model.vocab_size());
    bool greedy = true;
    for (float t : temperatures) greedy = greedy && t <= 0.f;
    if (greedy) argmax(lg, tok_out_, stream_, host_tok_[host_turn_]);
    else sample(lg, d_temps, d_u, tok_out_, stream_, host_tok_[host_turn_]);
    HIP_OK(hipEventRecord(host_tok_event_[host_turn_], stream_));
    pending_.push_back({host_tok_[host_turn_], n, host_tok_event_[host_turn_]});
    return n;
}

std::vector<int> ModelRunner::collect() {
    if (pending_.empty()) throw EngineError("no launch has tokens pending");
    const PendingTokens p = pending_.front();
    pending_.pop_front();
    HIP_OK(hipEventSynchronize(p.done));
    return std::vector<int>(p.host, p.host + p.n);
}

// ---------------------------------------------------------------------------------------------
// engine
// ---------------------------------------------------------------------------------------------
Engine::Engine(std::unique_ptr<LoadedModel> model, const EngineOptions& o) : model_(std::move(model)), options_(o) {
    if (o.kv_block_size < 1 || o.max_batch_num < 1 || o.max_tokens_per_step < 1 || o.prefill_chunk < 1)
        throw EngineError("kv_block_size, max_batch_num, max_tokens_per_step and prefill_chunk must be positive");
    if (o.kv_memory_fraction < 0.0 || o.kv_memory_fraction > 1.0) throw EngineError("kv_memory_fraction must lie in [0, 1]");
    RunnerOptions ro;
    ro.page_size = o.kv_block_size;
    ro.n_pages = o.total_kv_blocks;
    ro.memory_fraction = o.kv_memory_fraction;
    ro.max_num_seqs = o.max_batch_num;
    ro.max_tokens_per_step = o.max_tokens_per_step;
    runner_.reset(new ModelRunner(*model_, ro));
    options_.total_kv_blocks = runner_->n_pages();
    SchedulerOptions so;
    so.max_num_seqs = o.max_batch_num;
    so.max_tokens_per_step = o.max_tokens_per_step;
    so.prefill_chunk = o.prefill_chunk;
    so.max_positions = model_->max_positions;
    so.preempt_for_decode = o.preempt_for_decode;
    scheduler_.reset(new Scheduler(&runner_->manager(), so));
}

std::unique_ptr<Engine> Engine::from_pretrained(const std::string& model_dir, int dtype, const EngineOptions& o) {
    return std::unique_ptr<Engine>(new Engine(load_model(model_dir, dtype), o));
}

std::unique_ptr<Engine> Engine::from_random(const Json& config, uint64_t seed, int dtype, const EngineOptions& o) {
    return std::unique_ptr<Engine>(new Engine(random_model(config, seed, dtype), o));
}

int64_t Engine::add_request(const std::vector<int>& prompt, const SamplingParams& params, int64_t request_id) {
    const int vocab = model_->model.vocab_size();
    for (int t : prompt)
        if (t < 0 || t >= vocab) throw EngineError("token ids must lie in [0, " + std::to_string(vocab) + ")");
    if (params.temperature < 0.f) throw EngineError("temperature must be >= 0");
    const int64_t id = request_id < 0 ? next_id_ : request_id;
    const int rc = scheduler_->add_request(id, static_cast<int>(prompt.size()), params.max_new_tokens);
    if (rc == -2) throw EngineError("request " + std::to_string(id) + " already exists");
    if (rc != 0)
        throw EngineError("request refused: prompt of " + std::to_string(prompt.size()) + " tokens (must be 1..max positions) and max_new_tokens=" +
                          std::to_string(params.max_new_tokens) + " (must be >= 1)");
    next_id_ = std::max(next_id_, id) + 1;
    auto r = std::make_shared<Request>();
    r->id = id;
    r->tokens = prompt;
    r->prompt_len = static_cast<int>(prompt.size());
    r->params = params;
    requests_[id] = r;
    return id;
}

void Engine::drop(const RequestPtr& r) {
    auto it = requests_.find(r->id);
    if (it != requests_.end() && it->second == r) {
        requests_.erase(it);
        scheduler_->forget(r->id);
    }
}

std::vector<int> Engine::abort(int64_t request_id) {
    auto it = requests_.find(request_id);
    if (it == requests_.end()) throw EngineError("request " + std::to_string(request_id) + " is not live");
    RequestPtr r = it->second;
    scheduler_->abort(request_id);
    r->finished = true;
    r->failed = "aborted";
    drop(r);
    return std::vector<int>(r->tokens.begin() + r->prompt_len, r->tokens.end());
}

bool Engine::has_unfinished() const { return scheduler_->has_work() || in_flight_ || !undelivered_.empty(); }

bool Engine::is_eos(const Request& r, int tok) const {
    return !r.params.ignore_eos && model_->eos_token_id >= 0 && tok == model_->eos_token_id;
}

// Reads the tokens of the step in flight, if any. A request that an earlier token already ended (seen
// late) or that was aborted drops its token.
std::vector<RequestOutput> Engine::collect() {
    std::vector<RequestOutput> outputs;
    if (!in_flight_) return outputs;
    in_flight_ = false;
    const std::vector<int> toks = runner_->collect();
    auto rows = std::move(in_flight_rows_);
    in_flight_rows_.clear();
    for (size_t i = 0; i < rows.size() && i < toks.size(); ++i) {
        const RequestPtr& r = rows[i].first;
        bool done = rows[i].second;
        auto it = requests_.find(r->id);
        if (r->finished || it == requests_.end() || it->second != r) continue;      // ended by an earlier token, or aborted
        const int tok = toks[i];
        r->tokens.push_back(tok);
        if (!done && is_eos(*r, tok)) {
            // the scheduler has planned on without knowing: take the request out now
            scheduler_->stop(r->id);
            r->ended_early = done = true;
        }
        r->finished = done;
        outputs.push_back({r->id, tok, done, ""});
        if (done) drop(r);
    }
    return outputs;
}

std::vector<RequestOutput> Engine::step() {
    std::vector<PlanEntry> plan = scheduler_->schedule();
    std::vector<RequestOutput> outputs;
    Event ev;
    while (scheduler_->pop_event(&ev)) {
        if (ev.kind != EventKind::Failed) continue;
        auto it = requests_.find(ev.id);
        if (it == requests_.end()) continue;           // aborted by the caller, who knows
        RequestPtr r = it->second;
        r->finished = true;
        r->failed = "the page pool cannot hold this request";
        outputs.push_back({r->id, -1, true, r->failed});
        drop(r);
    }
    auto append = [&](std::vector<RequestOutput> more) { for (auto& o : more) outputs.push_back(std::move(o)); };
    if (plan.empty()) {
        append(collect());
        return outputs;
    }
    // only a single decoded token can be fed on the device; a portion that reaches past what the host has
    // read (a request recomputed right after it was preempted) waits for the read
    bool unread_portion = false;
    for (const PlanEntry& e : plan) {
        const RequestPtr& r = requests_.at(e.id);
        if (e.n_tokens > 1 && e.start + e.n_tokens > static_cast<int>(r->tokens.size())) unread_portion = true;
    }
    if (!options_.overlap || unread_portion) {
        // the host knows every token it feeds: read what is in flight first
        append(collect());
        std::vector<PlanEntry> live;
        for (const PlanEntry& e : plan)
            if (requests_.count(e.id)) live.push_back(e);
        if (live.size() != plan.size()) {      // ended by a token just read; the scheduler dropped them too
            plan = live;
            if (plan.empty()) return outputs;
        }
    }
    // A token that the step in flight has sampled and the host has not read is fed on the device: its row
    // among that step's sampled tokens stands in for it.
    std::map<int64_t, int> row_in_flight;
    if (in_flight_)
        for (size_t i = 0; i < in_flight_rows_.size(); ++i) row_in_flight[in_flight_rows_[i].first->id] = static_cast<int>(i);
    std::vector<StepEntry> entries;
    std::vector<float> temps, us;
    std::vector<const PlanEntry*> sampled;
    for (const PlanEntry& e : plan) {
        const RequestPtr& r = requests_.at(e.id);
        StepEntry se;
        se.request_id = e.id;
        if (e.start + e.n_tokens <= static_cast<int>(r->tokens.size())) {
            se.tokens.assign(r->tokens.begin() + e.start, r->tokens.begin() + e.start + e.n_tokens);
        } else {                                    // a decoded token still in flight
            auto it = row_in_flight.find(e.id);
            if (e.n_tokens != 1 || it == row_in_flight.end()) throw EngineError("a planned token is neither known nor in flight");
            se.tokens.assign(1, 0);
            se.feed_row = it->second;
        }
        if (e.want_last) {
            se.want.push_back(e.n_tokens - 1);
            temps.push_back(r->params.temperature);
            us.push_back(r->params.temperature > 0.f ? uniform01(r->params.seed, r->n_launched) : 0.f);
            r->n_launched += 1;
            sampled.push_back(&e);
        }
        entries.push_back(std::move(se));
    }
    const int n = runner_->launch(entries, temps, us);
    // the scheduler moves on as if no token were the end of sequence; collect() corrects it
    std::vector<std::pair<RequestPtr, bool>> rows;
    scheduler_->commit();
    for (const PlanEntry* e : sampled) rows.emplace_back(requests_.at(e->id), scheduler_->on_token(e->id, false) == 1);
    append(collect());
    if (n > 0) {
        in_flight_ = true;
        in_flight_rows_ = std::move(rows);
    }
    if (!options_.overlap) append(collect());
    return outputs;
}

std::vector<RequestOutput> Engine::step_some(size_t cap) {
    if (undelivered_.empty())
        for (RequestOutput& o : step()) undelivered_.push_back(std::move(o));
    std::vector<RequestOutput> out;
    while (!undelivered_.empty() && out.size() < cap) {
        out.push_back(std::move(undelivered_.front()));
        undelivered_.pop_front();
    }
    return out;
}

std::vector<std::vector<int>> Engine::generate(const std::vector<std::vector<int>>& prompts,
                                               const std::vector<SamplingParams>& params) {
    std::vector<int64_t> ids;
    std::map<int64_t, std::vector<int>> got;
    std::map<int64_t, std::string> errors;
    for (size_t i = 0; i < prompts.size(); ++i) {
        ids.push_back(add_request(prompts[i], params.size() == 1 ? params[0] : params.at(i)));
        got[ids.back()];
    }
    while (has_unfinished()) {
        for (const RequestOutput& o : step()) {
            if (!got.count(o.request_id)) continue;
            if (o.token < 0) errors[o.request_id] = o.error.empty() ? "failed" : o.error;
            else got[o.request_id].push_back(o.token);
        }
    }
    std::vector<std::vector<int>> out;
    for (int64_t id : ids) {
        if (errors.count(id)) throw EngineError("request " + std::to_string(id) + " failed: " + errors[id]);
        out.push_back(got[id]);
    }
    return out;
}

std::map<std::string, int64_t> Engine::stats() const {
    const Counters& c = scheduler_->counters();
    CacheManager& m = runner_->manager();
    return {{"steps", c.steps}, {"scheduled_tokens", c.scheduled_tokens}, {"prefill_tokens", c.prefill_tokens},
            {"decode_tokens", c.decode_tokens}, {"deferred_decodes", c.deferred_decodes}, {"deferred_prefills", c.deferred_prefills},
            {"preemptions", c.preemptions}, {"failures", c.failures}, {"finished", c.finished}, {"aborted", c.aborted},
            {"peak_pages_used", c.peak_pages_used},
            {"free_pages", m.n_groups() ? m.free_pages(0) : 0}, {"total_pages", m.n_groups() ? m.total_pages(0) : 0}};
}

}  // namespace minillm
