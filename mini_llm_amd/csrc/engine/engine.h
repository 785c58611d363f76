// The native engine: requests in, tokens out. Scheduler above, step function below, on one GPU.
//
// One iteration: the scheduler plans a mixed batch (decoded tokens first, then prompt portions
// under the token budget), the runner runs it through the model and samples on the device, finished
// requests give their pages back. The reference's loop: /root/reference/src/runtime/scheduler.cpp:322-356;
// its model entry points, one for whole prompts and one for single tokens:
// /root/reference/include/model/gpt2_model.cuh:84-109; its program: /root/reference/src/main.cpp:3-10.
//
// Steps run one ahead of the host: a step is launched with the decoded tokens among its inputs taken
// on the device from the step before, and only then are that earlier step's tokens read. What the
// host learns late is only whether a token was the end of sequence; such a request has then run one
// step too many, whose token is dropped.
#pragma once

#include <hip/hip_runtime.h>

#include <cstdint>
#include <deque>
#include <map>
#include <memory>
#include <string>
#include <vector>

#include "arch.h"
#include "cache_manager.h"
#include "scheduler.h"

namespace minillm {

class EngineError : public std::runtime_error {
public:
    explicit EngineError(const std::string& what) : std::runtime_error(what) {}
};

struct EngineOptions {
    int kv_block_size = 16;            // tokens per page (reference: DEFAULT_KV_BLOCK_SIZE, constants.h:16)
    int total_kv_blocks = 4096;        // pages in the pool (reference: DEFAULT_TOTAL_KV_BLOCKS, constants.h:17)
    double kv_memory_fraction = 0.0;   // > 0: the pool takes this share of the device memory that is free once the
                                       // weights are loaded and the runner's buffers for the largest step are
                                       // taken, whatever total_kv_blocks says
    int max_batch_num = 16;            // sequences in one step (reference: MAX_BATCH_NUM, constants.h:20)
    int max_tokens_per_step = 2048;    // token budget of one step
    int prefill_chunk = 512;           // longest prompt portion
    bool overlap = true;               // launch a step before the previous one's tokens are read
    bool preempt_for_decode = true;    // a decode that gets no page preempts a younger request at once (scheduler.h);
                                       // false: it waits on its pages until somebody finishes, the reference's manner
                                       // (measured under page pressure, 256 requests of 512 + 512 tokens through a pool of
                                       // 60 % of a full batch: 12 % more tokens a second at GPT-2 small sizes, 18 % at XL)
};

struct SamplingParams {
    float temperature = 0.f;           // 0: greedy
    uint64_t seed = 0;
    int max_new_tokens = 8;            // the reference's default (/root/reference/include/constants.h:14)
    bool ignore_eos = false;
};

struct RequestOutput {
    int64_t request_id = 0;
    int token = -1;                    // -1: no token (the request failed)
    bool finished = false;
    std::string error;
};

// A number in [0, 1) with 24 random bits (exact in fp32) for output `index` of a request sampled with `seed`.
float uniform01(uint64_t seed, uint64_t index);

// Device memory for the caches of a model, grouped by need, and the bookkeeping of who holds what.
// Caches with equal needs share a group and therefore page ids: pool layout
// [caches in group][K|V][n_pages * page_size][kv_dim].
class CacheStorage {
public:
    CacheStorage(const std::vector<CacheNeed>& needs, int page_size, int n_pages, int n_state_slots, int dtype);
    ~CacheStorage();
    CacheStorage(const CacheStorage&) = delete;
    CacheStorage& operator=(const CacheStorage&) = delete;
    CacheManager& manager() { return *manager_; }
    const std::vector<CacheView>& views() const { return views_; }
    int n_groups() const { return static_cast<int>(group_specs_.size()); }
    int page_size() const { return page_size_; }
    size_t bytes_per_token() const { return bytes_per_token_; }
    void reset_fresh_states(const StepView& step, hipStream_t s) const;
    void poison();                     // fills every page with NaN (tests)

private:
    void allocate(const std::vector<CacheNeed>& needs, int n_pages, int n_state_slots);
    int page_size_, dtype_;
    std::vector<GroupSpec> group_specs_;
    std::vector<CacheView> views_;
    std::vector<void*> allocations_;
    std::vector<size_t> allocation_bytes_;
    std::unique_ptr<CacheManager> manager_;
    size_t bytes_per_token_ = 0;
};

// A request's share of a step.
struct StepEntry {
    int64_t request_id = 0;
    std::vector<int> tokens;           // its next tokens
    std::vector<int> want;             // indices into `tokens` whose logits are wanted
    int feed_row = -1;                 // >= 0: the single token is row feed_row of what the previous launch sampled
};

struct RunnerOptions {
    int page_size = 16;
    int n_pages = 0;                   // pages of every group's pool ...
    double memory_fraction = 0.0;      // ... or, if > 0, this share of the device memory that is free once the
                                       // runner's own buffers (workspace, logits, index arrays, scratch) exist
    int max_num_seqs = 16;             // most sequences in a step: scratch, state slots and token buffers are sized for it
    int max_tokens_per_step = 0;       // > 0: the step's workspace is taken now for this many tokens, not at the first large step
};

// Owns the cache storage and runs steps of a model, on a stream of its own.
class ModelRunner {
public:
    ModelRunner(LoadedModel& model, const RunnerOptions& options);
    ModelRunner(LoadedModel& model, int page_size, int n_pages, int max_num_seqs);
    ~ModelRunner();
    CacheStorage& cache() { return *cache_; }
    CacheManager& manager() { return cache_->manager(); }
    const LoadedModel& model() const { return model_; }

    // Runs one batch and returns the fp32 logits [wanted, vocab] on the host, in the order of the entries
    // and of each entry's `want` (nullptr and 0 rows if nothing is wanted). The rows lie in a pinned buffer of
    // the runner and stay valid until its next step. With manage_cache the runner registers new requests,
    // takes their pages and commits the new lengths itself (replay, tests).
    const float* step(const std::vector<StepEntry>& entries, bool manage_cache, int* n_rows);
    void end_request(int64_t id) { manager().free_request(id); }

    // Starts one step (pages reserved, lengths committed by the caller) and returns at once. One token is
    // sampled for every wanted place, left on the device for the next launch to take, and copied to the
    // host behind the step. Returns how many tokens will arrive (0: nothing was wanted, nothing pending).
    int launch(const std::vector<StepEntry>& entries, const std::vector<float>& temperatures,
               const std::vector<float>& uniforms);
    // Waits for the oldest launch that has tokens pending and returns them.
    std::vector<int> collect();
    bool pending() const { return !pending_.empty(); }
    void synchronize();
    hipStream_t stream() const { return stream_; }
    int n_pages() const { return n_pages_; }

private:
    void init(const RunnerOptions& o);
    void destroy() noexcept;
    struct Staging {
        int* host = nullptr;
        size_t capacity = 0;
        hipEvent_t copied = nullptr;
        bool in_use = false;
    };
    struct PendingTokens {
        int* host;
        int n;
        hipEvent_t done;
    };
    StepView build(const std::vector<StepEntry>& entries, const std::vector<float>* temps,
                   const std::vector<float>* uniforms, const float** d_temps, const float** d_uniforms);
    float* run(const StepView& step);          // model forward; device logits or nullptr
    void* arena_for(int tokens, int n_logits);
    void grow(void** ptr, size_t* have, size_t need);

    LoadedModel& model_;
    std::unique_ptr<CacheStorage> cache_;
    int page_size_, n_pages_, max_num_seqs_;
    hipStream_t stream_ = nullptr;
    Staging staging_[2];
    int turn_ = 0;
    int* dev_ints_ = nullptr;
    size_t dev_ints_cap_ = 0;
    void* arena_ = nullptr;
    size_t arena_bytes_ = 0;
    float* logits_ = nullptr;
    size_t logits_bytes_ = 0;
    float* host_logits_ = nullptr;     // pinned: what step() returns
    size_t host_logits_bytes_ = 0;
    int* tok_out_ = nullptr;           // sampled tokens of the last launched step
    int tok_out_cap_ = 0;
    int* host_tok_[2] = {nullptr, nullptr};
    hipEvent_t host_tok_event_[2] = {nullptr, nullptr};
    int host_tok_cap_ = 0, host_turn_ = 0;
    std::deque<PendingTokens> pending_;
    // per step: pointer arrays that the StepView points into
    std::vector<const int*> tables_, slots_;
    std::vector<int> max_blocks_;
};

class Engine {
public:
    Engine(std::unique_ptr<LoadedModel> model, const EngineOptions& options);
    static std::unique_ptr<Engine> from_pretrained(const std::string& model_dir, int dtype, const EngineOptions& o);
    static std::unique_ptr<Engine> from_random(const Json& config, uint64_t seed, int dtype, const EngineOptions& o);

    // Returns the request's id. Throws EngineError for token ids outside the vocabulary or a prompt that
    // the scheduler refuses (empty, longer than the model's positions).
    int64_t add_request(const std::vector<int>& prompt, const SamplingParams& params, int64_t request_id = -1);
    std::vector<int> abort(int64_t request_id);
    bool has_unfinished() const;
    std::vector<RequestOutput> step();
    // The same, at most `cap` outputs at a time: what does not fit waits for the next call (which then runs
    // no iteration of its own), and has_unfinished() stays true meanwhile. For callers with fixed buffers.
    std::vector<RequestOutput> step_some(size_t cap);
    // Generates for every prompt (continuous batching) and returns the new tokens of each.
    std::vector<std::vector<int>> generate(const std::vector<std::vector<int>>& prompts,
                                           const std::vector<SamplingParams>& params);
    ModelRunner& runner() { return *runner_; }
    Scheduler& scheduler() { return *scheduler_; }
    const LoadedModel& model() const { return *model_; }
    std::map<std::string, int64_t> stats() const;

private:
    struct Request {
        int64_t id;
        std::vector<int> tokens;
        int prompt_len;
        SamplingParams params;
        bool finished = false, ended_early = false;
        std::string failed;
        uint64_t n_launched = 0;
    };
    using RequestPtr = std::shared_ptr<Request>;
    bool is_eos(const Request& r, int tok) const;
    std::vector<RequestOutput> collect();
    void drop(const RequestPtr& r);

    std::unique_ptr<LoadedModel> model_;
    EngineOptions options_;
    std::unique_ptr<ModelRunner> runner_;
    std::unique_ptr<Scheduler> scheduler_;
    std::map<int64_t, RequestPtr> requests_;       // live requests only
    int64_t next_id_ = 0;
    bool in_flight_ = false;
    std::vector<std::pair<RequestPtr, bool>> in_flight_rows_;      // (request, finished by that token)
    std::deque<RequestOutput> undelivered_;                        // outputs that a step_some call had no room for
};

}  // namespace minillm
