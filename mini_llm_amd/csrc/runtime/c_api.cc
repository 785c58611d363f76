// C ABI of the host runtime (cache manager and scheduler), loaded from Python with ctypes.
#include <cstring>
#include <string>
#include <vector>

#include "cache_manager.h"
#include "scheduler.h"

using namespace minillm;

extern "C" {

void* mllm_cache_create(int n_groups, const int* page_size, const int* n_pages, const int* window,
                        int n_state_slots) {
    std::vector<GroupSpec> groups(n_groups);
    for (int g = 0; g < n_groups; ++g) {
        if (page_size[g] < 1 || n_pages[g] < 0 || window[g] < 0) return nullptr;
        groups[g].page_size = page_size[g];
        groups[g].n_pages = n_pages[g];
        groups[g].window = window[g];
    }
    if (n_state_slots < 0) return nullptr;
    return new CacheManager(groups, n_state_slots);
}
void mllm_cache_destroy(void* c) { delete static_cast<CacheManager*>(c); }
int mllm_cache_add_request(void* c, int64_t id) { return static_cast<CacheManager*>(c)->add_request(id); }
int mllm_cache_has_request(void* c, int64_t id) { return static_cast<CacheManager*>(c)->has_request(id) ? 1 : 0; }
int mllm_cache_pages_needed(void* c, int64_t id, int g, int new_len) {
    return static_cast<CacheManager*>(c)->pages_needed(id, g, new_len);
}
int mllm_cache_can_reserve(void* c, int64_t id, int new_len) {
    return static_cast<CacheManager*>(c)->can_reserve(id, new_len) ? 1 : 0;
}
int mllm_cache_reserve(void* c, int64_t id, int new_len) { return static_cast<CacheManager*>(c)->reserve(id, new_len); }
int mllm_cache_commit(void* c, int64_t id, int new_len) { return static_cast<CacheManager*>(c)->commit(id, new_len); }
int mllm_cache_free_request(void* c, int64_t id) { return static_cast<CacheManager*>(c)->free_request(id); }
int mllm_cache_length(void* c, int64_t id) { return static_cast<CacheManager*>(c)->length(id); }
int mllm_cache_state_slot(void* c, int64_t id) { return static_cast<CacheManager*>(c)->state_slot(id); }
int mllm_cache_block_table(void* c, int64_t id, int g, int* out, int cap) {
    return static_cast<CacheManager*>(c)->block_table(id, g, out, cap);
}
int mllm_cache_fill_step_common(void* c, const int64_t* ids, const int* n_tokens, int n, int* positions,
                                int* token_seq, int* cu_q, int* starts, int* ctx_len, int* state_slots) {
    return static_cast<CacheManager*>(c)->fill_step_common(ids, n_tokens, n, positions, token_seq, cu_q, starts,
                                                          ctx_len, state_slots);
}
int mllm_cache_fill_step_group(void* c, const int64_t* ids, const int* n_tokens, int n, int g, int max_blocks,
                               int* tables, int* slots) {
    return static_cast<CacheManager*>(c)->fill_step_group(ids, n_tokens, n, g, max_blocks, tables, slots);
}
int mllm_cache_free_pages(void* c, int g) { return static_cast<CacheManager*>(c)->free_pages(g); }
int mllm_cache_total_pages(void* c, int g) { return static_cast<CacheManager*>(c)->total_pages(g); }
int mllm_cache_free_state_slots(void* c) { return static_cast<CacheManager*>(c)->free_state_slots(); }
int mllm_cache_n_requests(void* c) { return static_cast<CacheManager*>(c)->n_requests(); }
// Writes the (possibly truncated) consistency report; returns its full length (0 = consistent).
int mllm_cache_check(void* c, char* out, int cap) {
    std::string s = static_cast<CacheManager*>(c)->check();
    if (cap > 0) {
        int n = static_cast<int>(s.size()) < cap - 1 ? static_cast<int>(s.size()) : cap - 1;
        std::memcpy(out, s.data(), n);
        out[n] = 0;
    }
    return static_cast<int>(s.size());
}

void* mllm_sched_create(void* cache, int max_num_seqs, int max_tokens_per_step, int prefill_chunk,
                        int max_positions, int preempt_for_decode) {
    SchedulerOptions o;
    o.max_num_seqs = max_num_seqs;
    o.max_tokens_per_step = max_tokens_per_step;
    o.prefill_chunk = prefill_chunk;
    o.max_positions = max_positions;
    o.preempt_for_decode = preempt_for_decode != 0;
    return new Scheduler(static_cast<CacheManager*>(cache), o);
}
void mllm_sched_destroy(void* s) { delete static_cast<Scheduler*>(s); }
int mllm_sched_add(void* s, int64_t id, int prompt_len, int max_new_tokens) {
    return static_cast<Scheduler*>(s)->add_request(id, prompt_len, max_new_tokens);
}
int mllm_sched_schedule(void* s, int64_t* ids, int* start, int* n_tokens, int* want_last, int cap) {
    const auto& plan = static_cast<Scheduler*>(s)->schedule();
    int n = static_cast<int>(plan.size());
    for (int i = 0; i < n && i < cap; ++i) {
        ids[i] = plan[i].id;
        start[i] = plan[i].start;
        n_tokens[i] = plan[i].n_tokens;
        want_last[i] = plan[i].want_last;
    }
    return n;
}
void mllm_sched_commit(void* s) { static_cast<Scheduler*>(s)->commit(); }
int mllm_sched_on_token(void* s, int64_t id, int is_eos) { return static_cast<Scheduler*>(s)->on_token(id, is_eos != 0); }
int mllm_sched_abort(void* s, int64_t id) { return static_cast<Scheduler*>(s)->abort(id); }
int mllm_sched_stop(void* s, int64_t id) { return static_cast<Scheduler*>(s)->stop(id); }
int mllm_sched_forget(void* s, int64_t id) { return static_cast<Scheduler*>(s)->forget(id); }
int mllm_sched_n_known(void* s) { return static_cast<Scheduler*>(s)->n_known(); }
int mllm_sched_has_work(void* s) { return static_cast<Scheduler*>(s)->has_work() ? 1 : 0; }
int mllm_sched_state(void* s, int64_t id) { return static_cast<int>(static_cast<Scheduler*>(s)->state(id)); }
int mllm_sched_generated(void* s, int64_t id) { return static_cast<Scheduler*>(s)->generated(id); }
int mllm_sched_pop_event(void* s, int64_t* id, int* kind) {
    Event e;
    if (!static_cast<Scheduler*>(s)->pop_event(&e)) return 0;
    *id = e.id;
    *kind = static_cast<int>(e.kind);
    return 1;
}
int mllm_sched_queue_length(void* s, int which) { return static_cast<Scheduler*>(s)->queue_length(which); }
void mllm_sched_counters(void* s, int64_t* out11) {
    const Counters& c = static_cast<Scheduler*>(s)->counters();
    out11[0] = c.steps; out11[1] = c.scheduled_tokens; out11[2] = c.prefill_tokens; out11[3] = c.decode_tokens;
    out11[4] = c.deferred_decodes; out11[5] = c.deferred_prefills; out11[6] = c.preemptions;
    out11[7] = c.failures; out11[8] = c.finished; out11[9] = c.peak_pages_used; out11[10] = c.aborted;
}

}  // extern "C"
