// Scheduler: admits requests, cuts prompts into portions under a token budget,
// decodes, finishes and frees.
//
// Queues and states follow the reference's
// (/root/reference/include/runtime/scheduler.h:26-36,
//  /root/reference/include/runtime/request.h:16-29,
//  /root/reference/src/runtime/scheduler.cpp:38-100,124-266,322-356), with these
// differences: one mixed batch per iteration (decoded tokens first, then prompt
// portions) instead of separate decode and prefill calls; prompts are cut into
// portions; pages are taken per portion; and when nobody can take a step the
// most recently admitted request is preempted and recomputed later (the reference
// swaps to host memory instead).
#pragma once

#include <cstdint>
#include <deque>
#include <unordered_map>
#include <vector>

#include "cache_manager.h"

namespace minillm {

enum class RequestState : int {
    WaitingPrefill = 0,
    DeferredPrefill = 1,   // could not be admitted: too few free pages or slots
    Prefill = 2,           // admitted, prompt partly consumed
    DecodeReady = 3,
    DeferredDecode = 4,    // no page for its next token in this iteration
    Finished = 5,
    Failed = 6,            // can never run (larger than the whole pool)
    Aborted = 7,           // taken out by the caller
    Unknown = -1,
};

enum class EventKind : int { Preempted = 1, Failed = 2, Deferred = 3 };

struct SchedulerOptions {
    int max_num_seqs = 16;          // sequences in one step
    int max_tokens_per_step = 2048; // token budget of one step
    int prefill_chunk = 512;        // longest prompt portion
    int max_positions = 0;          // 0: unbounded; else no token at a position >= this
    // What happens to a decode that gets no page. false (the reference's manner): it is deferred and keeps its
    // pages until somebody finishes; only when nobody can step is a request preempted. true: the most recently
    // admitted running request that is younger than it and not in this step's plan is preempted at once (its
    // pages freed, recomputed later), so that pages do not idle under requests that wait; if there is none
    // (it is the youngest itself), it is deferred.
    bool preempt_for_decode = false;
};

struct PlanEntry {
    int64_t id;
    int start;      // tokens already in the cache
    int n_tokens;   // tokens this step feeds: positions [start, start + n_tokens)
    int want_last;  // 1 if the last of them is the request's newest token (sample after it)
};

struct Event {
    int64_t id;
    EventKind kind;
};

struct Counters {
    int64_t steps = 0, scheduled_tokens = 0, prefill_tokens = 0, decode_tokens = 0;
    int64_t deferred_decodes = 0, deferred_prefills = 0, preemptions = 0, failures = 0, finished = 0;
    int64_t peak_pages_used = 0, aborted = 0;
};

class Scheduler {
public:
    Scheduler(CacheManager* cache, const SchedulerOptions& opt);

    // 0 ok; -1 refused (empty prompt, prompt longer than max_positions, max_new_tokens < 1); -2 duplicate id.
    int add_request(int64_t id, int prompt_len, int max_new_tokens);
    // Plans the next step. An empty plan means there is nothing to run.
    const std::vector<PlanEntry>& schedule();
    // After the model ran the plan: advances cached lengths and releases passed pages.
    void commit();
    // After commit(), for every planned entry with want_last: a token was sampled.
    // Returns 1 if the request is now finished (its pages are freed), 0 if it goes on, -2 if unknown.
    int on_token(int64_t id, bool is_eos);
    // Ends a request wherever it is; its pages are given back. 0 or -2.
    int abort(int64_t id);
    // The request is complete as of a token sampled earlier (the caller saw the end of sequence
    // only after the next step had been planned or run): it leaves the plan and the queues as
    // finished, not failed, and its pages are given back. 0 or -2.
    int stop(int64_t id);

    // Drops the record of a finished or failed request (its id may be used again). 0; -1 if the
    // request is still live; -2 if unknown.
    int forget(int64_t id);

    bool has_work() const;
    RequestState state(int64_t id) const;
    int generated(int64_t id) const;
    bool pop_event(Event* e);
    const Counters& counters() const { return counters_; }
    int n_known() const { return static_cast<int>(reqs_.size()); }
    int queue_length(int which) const;   // 0 waiting, 1 deferred_prefill, 2 prefill, 3 decode, 4 deferred_decode

private:
    struct Req {
        int64_t id;
        int total_len;       // prompt + generated tokens known so far
        int computed;        // tokens in the cache
        int max_new_tokens;
        int generated;
        RequestState state;
        uint64_t admit_seq;  // order of admission; the latest is preempted first
    };

    bool try_plan_tokens(Req& r, int n, int* budget, int* n_seqs);
    bool admit(Req& r);
    bool resolve_stall();
    void preempt(Req& victim);
    bool preempt_younger_than(const Req& r);
    void finish(Req& r, RequestState final_state);
    void remove_from(std::deque<int64_t>& q, int64_t id);

    CacheManager* cache_;
    SchedulerOptions opt_;
    std::unordered_map<int64_t, Req> reqs_;
    std::deque<int64_t> waiting_, deferred_prefill_, prefill_, decode_, deferred_decode_;
    std::vector<PlanEntry> plan_;
    std::deque<Event> events_;
    Counters counters_;
    uint64_t next_admit_seq_ = 1;
};

}  // namespace minillm
