#include "scheduler.h"

#include <algorithm>

namespace minillm {

static inline bool is_final(RequestState s) {
    return s == RequestState::Finished || s == RequestState::Failed || s == RequestState::Aborted;
}


Scheduler::Scheduler(CacheManager* cache, const SchedulerOptions& opt) : cache_(cache), opt_(opt) {
    if (opt_.max_num_seqs < 1) opt_.max_num_seqs = 1;
    if (opt_.max_tokens_per_step < 1) opt_.max_tokens_per_step = 1;
    if (opt_.prefill_chunk < 1) opt_.prefill_chunk = 1;
}

int Scheduler::add_request(int64_t id, int prompt_len, int max_new_tokens) {
    if (reqs_.count(id)) return -2;
    if (prompt_len < 1 || max_new_tokens < 1) return -1;
    if (opt_.max_positions > 0 && prompt_len > opt_.max_positions) return -1;
    Req r{id, prompt_len, 0, max_new_tokens, 0, RequestState::WaitingPrefill, 0};
    reqs_.emplace(id, r);
    waiting_.push_back(id);
    return 0;
}

void Scheduler::remove_from(std::deque<int64_t>& q, int64_t id) {
    auto it = std::find(q.begin(), q.end(), id);
    if (it != q.end()) q.erase(it);
}

bool Scheduler::try_plan_tokens(Req& r, int n, int* budget, int* n_seqs) {
    if (cache_->reserve(r.id, r.computed + n) != 0) return false;
    plan_.push_back({r.id, r.computed, n, r.computed + n == r.total_len ? 1 : 0});
    *budget -= n;
    *n_seqs += 1;
    return true;
}

// A request is admitted when a state slot is free and the pages for ALL the tokens
// it has so far are free now and not promised to a prompt that is under way (the reference
// reserves the whole prompt, real_kv_allocator.cu:112-139). The pages themselves are taken
// portion by portion, so what a prompt under way has not taken yet counts as promised.
bool Scheduler::admit(Req& r) {
    if (cache_->free_state_slots() < 1) return false;
    for (int g = 0; g < cache_->n_groups(); ++g) {
        int promised = 0;
        for (int64_t id : prefill_) promised += cache_->pages_needed(id, g, reqs_.at(id).total_len);
        if (cache_->pages_needed_fresh(g, r.total_len) + promised > cache_->free_pages(g)) return false;
    }
    if (cache_->add_request(r.id) < 0) return false;
    r.state = RequestState::Prefill;
    r.admit_seq = next_admit_seq_++;
    r.computed = 0;
    prefill_.push_back(r.id);
    return true;
}

const std::vector<PlanEntry>& Scheduler::schedule() {
    plan_.clear();
    for (;;) {
        int budget = opt_.max_tokens_per_step;
        int n_seqs = 0;

        // Deferred decodes get another try, behind those that are ready.
        while (!deferred_decode_.empty()) {
            int64_t id = deferred_decode_.front();
            deferred_decode_.pop_front();
            reqs_.at(id).state = RequestState::DecodeReady;
            decode_.push_back(id);
        }

        // 1. One token for every request that is decoding.
        std::deque<int64_t> ready;
        const std::vector<int64_t> decoding(decode_.begin(), decode_.end());      // (a preemption below edits decode_)
        for (int64_t id : decoding) {
            Req& r = reqs_.at(id);
            if (r.state != RequestState::DecodeReady) continue;      // preempted a moment ago for an older one
            if (n_seqs >= opt_.max_num_seqs || budget < 1) {
                ready.push_back(id);          // waits for the next step, loses nothing
                continue;
            }
            bool planned = try_plan_tokens(r, 1, &budget, &n_seqs);
            while (!planned && opt_.preempt_for_decode && preempt_younger_than(r)) planned = try_plan_tokens(r, 1, &budget, &n_seqs);
            if (planned) {
                ready.push_back(id);
            } else {
                r.state = RequestState::DeferredDecode;
                deferred_decode_.push_back(id);
                ++counters_.deferred_decodes;
                events_.push_back({id, EventKind::Deferred});
            }
        }
        decode_.clear();
        for (int64_t id : ready)
            if (reqs_.at(id).state == RequestState::DecodeReady) decode_.push_back(id);      // (not those preempted meanwhile)

        // 2. The next portion of every prompt that is under way, first come first served.
        bool blocked = false;
        for (int64_t id : prefill_) {
            Req& r = reqs_.at(id);
            if (n_seqs >= opt_.max_num_seqs || budget < 1) { blocked = true; break; }
            int n = std::min({r.total_len - r.computed, opt_.prefill_chunk, budget});
            if (!try_plan_tokens(r, n, &budget, &n_seqs)) { blocked = true; break; }
        }

        // 3. Admission: deferred requests before new ones; the first refusal ends it.
        while (!blocked && !(deferred_prefill_.empty() && waiting_.empty())) {
            if (n_seqs >= opt_.max_num_seqs || budget < 1) break;
            bool from_deferred = !deferred_prefill_.empty();
            int64_t id = from_deferred ? deferred_prefill_.front() : waiting_.front();
            Req& r = reqs_.at(id);
            if (!admit(r)) {
                if (!from_deferred) {
                    waiting_.pop_front();
                    r.state = RequestState::DeferredPrefill;
                    deferred_prefill_.push_back(id);
                    ++counters_.deferred_prefills;
                    events_.push_back({id, EventKind::Deferred});
                }
                blocked = true;
                break;
            }
            if (from_deferred) deferred_prefill_.pop_front(); else waiting_.pop_front();
            int n = std::min({r.total_len, opt_.prefill_chunk, budget});
            if (!try_plan_tokens(r, n, &budget, &n_seqs)) { blocked = true; break; }
        }

        if (!plan_.empty() || !has_work()) break;
        if (!resolve_stall()) break;
    }
    if (!plan_.empty()) {
        ++counters_.steps;
        int64_t used = 0;
        for (int g = 0; g < cache_->n_groups(); ++g) used += cache_->total_pages(g) - cache_->free_pages(g);
        counters_.peak_pages_used = std::max(counters_.peak_pages_used, used);
    }
    return plan_;
}

// Nobody can take a step although work is pending.
bool Scheduler::resolve_stall() {
    std::vector<int64_t> running;
    for (int64_t id : prefill_) running.push_back(id);
    for (int64_t id : decode_) running.push_back(id);
    for (int64_t id : deferred_decode_) running.push_back(id);
    if (running.empty()) {
        // Nothing holds a page and the head still does not fit: it never will.
        if (deferred_prefill_.empty() && waiting_.empty()) return false;
        int64_t id = !deferred_prefill_.empty() ? deferred_prefill_.front() : waiting_.front();
        finish(reqs_.at(id), RequestState::Failed);
        return true;
    }
    if (running.size() == 1) {
        // It holds every used page and still cannot go on: the pool is too small for it.
        finish(reqs_.at(running[0]), RequestState::Failed);
        return true;
    }
    // Preempt the most recently admitted one; it is recomputed from its tokens later.
    Req* victim = nullptr;
    for (int64_t id : running) {
        Req& r = reqs_.at(id);
        if (!victim || r.admit_seq > victim->admit_seq) victim = &r;
    }
    preempt(*victim);
    return true;
}

void Scheduler::preempt(Req& victim) {
    remove_from(prefill_, victim.id);
    remove_from(decode_, victim.id);
    remove_from(deferred_decode_, victim.id);
    cache_->free_request(victim.id);
    victim.computed = 0;
    victim.state = RequestState::DeferredPrefill;
    deferred_prefill_.push_front(victim.id);
    ++counters_.preemptions;
    events_.push_back({victim.id, EventKind::Preempted});
}

// Frees the pages of the most recently admitted running request that was admitted after `r` and has no
// tokens in the plan under way. False if there is none.
bool Scheduler::preempt_younger_than(const Req& r) {
    Req* victim = nullptr;
    auto consider = [&](int64_t id) {
        Req& c = reqs_.at(id);
        if (c.id == r.id || c.admit_seq <= r.admit_seq) return;
        for (const PlanEntry& e : plan_)
            if (e.id == id) return;
        if (!victim || c.admit_seq > victim->admit_seq) victim = &c;
    };
    for (int64_t id : prefill_) consider(id);
    for (int64_t id : decode_) consider(id);
    for (int64_t id : deferred_decode_) consider(id);
    if (victim == nullptr) return false;
    preempt(*victim);
    return true;
}

void Scheduler::commit() {
    for (const PlanEntry& e : plan_) {
        auto it = reqs_.find(e.id);
        if (it == reqs_.end()) continue;
        Req& r = it->second;
        if (is_final(r.state)) continue;
        r.computed = e.start + e.n_tokens;
        cache_->commit(r.id, r.computed);
        counters_.scheduled_tokens += e.n_tokens;
        if (e.n_tokens == 1 && r.generated > 0) ++counters_.decode_tokens;
        else counters_.prefill_tokens += e.n_tokens;
    }
    plan_.clear();
}

int Scheduler::on_token(int64_t id, bool is_eos) {
    auto it = reqs_.find(id);
    if (it == reqs_.end()) return -2;
    Req& r = it->second;
    if (is_final(r.state)) return 1;
    r.total_len += 1;
    r.generated += 1;
    if (r.state == RequestState::Prefill) {
        remove_from(prefill_, id);
        r.state = RequestState::DecodeReady;
        decode_.push_back(id);
    }
    bool out_of_positions = opt_.max_positions > 0 && r.total_len > opt_.max_positions;
    if (is_eos || r.generated >= r.max_new_tokens || out_of_positions) {
        finish(r, RequestState::Finished);
        return 1;
    }
    return 0;
}

void Scheduler::finish(Req& r, RequestState final_state) {
    remove_from(waiting_, r.id);
    remove_from(deferred_prefill_, r.id);
    remove_from(prefill_, r.id);
    remove_from(decode_, r.id);
    remove_from(deferred_decode_, r.id);
    if (cache_->has_request(r.id)) cache_->free_request(r.id);
    r.state = final_state;
    if (final_state == RequestState::Failed) {
        ++counters_.failures;
        events_.push_back({r.id, EventKind::Failed});
    } else if (final_state == RequestState::Aborted) {
        ++counters_.aborted;             // (no event: the caller who aborts knows)
    } else {
        ++counters_.finished;
    }
}

int Scheduler::abort(int64_t id) {
    auto it = reqs_.find(id);
    if (it == reqs_.end()) return -2;
    Req& r = it->second;
    if (is_final(r.state)) return 0;
    plan_.erase(std::remove_if(plan_.begin(), plan_.end(),
                               [id](const PlanEntry& e) { return e.id == id; }), plan_.end());
    finish(r, RequestState::Aborted);
    return 0;
}

int Scheduler::stop(int64_t id) {
    auto it = reqs_.find(id);
    if (it == reqs_.end()) return -2;
    Req& r = it->second;
    if (is_final(r.state)) return 0;
    plan_.erase(std::remove_if(plan_.begin(), plan_.end(),
                               [id](const PlanEntry& e) { return e.id == id; }), plan_.end());
    finish(r, RequestState::Finished);
    return 0;
}

int Scheduler::forget(int64_t id) {
    auto it = reqs_.find(id);
    if (it == reqs_.end()) return -2;
    RequestState st = it->second.state;
    if (!is_final(st)) return -1;
    reqs_.erase(it);
    return 0;
}

bool Scheduler::has_work() const {
    return !(waiting_.empty() && deferred_prefill_.empty() && prefill_.empty() && decode_.empty() &&
             deferred_decode_.empty());
}

RequestState Scheduler::state(int64_t id) const {
    auto it = reqs_.find(id);
    return it == reqs_.end() ? RequestState::Unknown : it->second.state;
}

int Scheduler::generated(int64_t id) const {
    auto it = reqs_.find(id);
    return it == reqs_.end() ? -2 : it->second.generated;
}

bool Scheduler::pop_event(Event* e) {
    if (events_.empty()) return false;
    *e = events_.front();
    events_.pop_front();
    return true;
}

int Scheduler::queue_length(int which) const {
    switch (which) {
        case 0: return static_cast<int>(waiting_.size());
        case 1: return static_cast<int>(deferred_prefill_.size());
        case 2: return static_cast<int>(prefill_.size());
        case 3: return static_cast<int>(decode_.size());
        case 4: return static_cast<int>(deferred_decode_.size());
        default: return -1;
    }
}

}  // namespace minillm
