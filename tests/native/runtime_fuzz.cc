// A random workload through the C++ cache manager and scheduler, for a build with
// -fsanitize=address,undefined: requests of random lengths arrive while others decode, pools are small
// enough that requests are deferred and preempted, some requests are aborted or stopped late, a second
// group of caches has a window and gives pages back early. After every step the manager's own invariants
// are checked (every page free or held by exactly one block, every slot likewise), the step's index
// arrays are built and their page rows checked for collisions; at the end every page and slot is back.
// Exit code 0 and "ok" on success.
#include <cstdio>
#include <cstdlib>
#include <map>
#include <random>
#include <set>
#include <vector>

#include "cache_manager.h"
#include "scheduler.h"

using namespace minillm;

#define REQUIRE(cond, ...)                                                     \
    do {                                                                       \
        if (!(cond)) {                                                         \
            std::fprintf(stderr, "runtime_fuzz: line %d: ", __LINE__);         \
            std::fprintf(stderr, __VA_ARGS__);                                 \
            std::fprintf(stderr, "\n");                                        \
            std::exit(1);                                                      \
        }                                                                      \
    } while (0)

static Counters g_total;

static void one_run(unsigned seed) {
    std::mt19937 rng(seed);
    auto pick = [&](int lo, int hi) { return lo + static_cast<int>(rng() % static_cast<unsigned>(hi - lo + 1)); };
    const int page = 1 << pick(1, 4), max_pos = 96, n_slots = pick(2, 6);
    std::vector<GroupSpec> groups(2);
    groups[0].page_size = page; groups[0].n_pages = pick((max_pos + page - 1) / page + 1, 3 * max_pos / page + 2); groups[0].window = 0;
    groups[1].page_size = page; groups[1].n_pages = groups[0].n_pages; groups[1].window = pick(3, 40);
    CacheManager cache(groups, n_slots);
    SchedulerOptions opt;
    opt.max_num_seqs = pick(1, n_slots);
    opt.prefill_chunk = pick(2, 24);
    opt.max_tokens_per_step = opt.prefill_chunk + opt.max_num_seqs + pick(0, 16);
    opt.max_positions = max_pos;
    opt.preempt_for_decode = pick(0, 1) == 1;      // both policies for a decode that gets no page
    Scheduler sched(&cache, opt);
    int64_t next_id = 1;
    std::map<int64_t, int> want_new;            // live requests -> tokens still to come
    int to_add = pick(3, 14), steps = 0;
    std::vector<int> positions, token_seq, cu_q, starts, ctx_len, slots_of, tables, rows;
    while ((to_add > 0 || sched.has_work()) && steps < 5000) {
        ++steps;
        while (to_add > 0 && pick(0, 2) == 0) {
            const int prompt = pick(1, 60), new_tokens = pick(1, max_pos - prompt);
            const int rc = sched.add_request(next_id, prompt, new_tokens);
            REQUIRE(rc == 0, "add_request returned %d", rc);
            want_new[next_id++] = new_tokens;
            --to_add;
        }
        const std::vector<PlanEntry> plan = sched.schedule();
        Event ev;
        while (sched.pop_event(&ev))
            if (ev.kind == EventKind::Failed) want_new.erase(ev.id);
        REQUIRE(cache.check().empty(), "after schedule: %s", cache.check().c_str());
        if (plan.empty()) continue;
        // the step's index arrays, as the runner builds them
        const int n = static_cast<int>(plan.size());
        std::vector<int64_t> ids(n);
        std::vector<int> n_tok(n);
        int T = 0, budget = 0;
        std::set<int64_t> seen;
        for (int i = 0; i < n; ++i) {
            ids[i] = plan[i].id; n_tok[i] = plan[i].n_tokens; T += n_tok[i]; budget += n_tok[i];
            REQUIRE(seen.insert(plan[i].id).second, "request %lld twice in a plan", static_cast<long long>(plan[i].id));
            REQUIRE(plan[i].n_tokens >= 1 && plan[i].start == cache.length(plan[i].id), "plan entry does not continue its request");
            REQUIRE(plan[i].start + plan[i].n_tokens <= max_pos, "a plan passes the last position");
        }
        REQUIRE(n <= opt.max_num_seqs && budget <= opt.max_tokens_per_step, "a plan exceeds the step's limits");
        positions.assign(T, 0); token_seq.assign(T, 0); cu_q.assign(n + 1, 0); starts.assign(n, 0); ctx_len.assign(n, 0); slots_of.assign(n, 0);
        REQUIRE(cache.fill_step_common(ids.data(), n_tok.data(), n, positions.data(), token_seq.data(), cu_q.data(), starts.data(),
                                       ctx_len.data(), slots_of.data()) == 0, "fill_step_common failed");
        for (int g = 0; g < 2; ++g) {
            const int max_blocks = (max_pos + page - 1) / page;
            tables.assign(static_cast<size_t>(n) * max_blocks, 0); rows.assign(T, 0);
            REQUIRE(cache.fill_step_group(ids.data(), n_tok.data(), n, g, max_blocks, tables.data(), rows.data()) == 0, "fill_step_group failed");
            std::set<int> used;
            for (int t = 0; t < T; ++t) {
                REQUIRE(rows[t] >= 0 && rows[t] < groups[g].n_pages * page, "a page row lies outside the pool");
                REQUIRE(used.insert(rows[t]).second, "two tokens of a step share a page row");
            }
        }
        sched.commit();
        for (const PlanEntry& e : plan) {
            if (!e.want_last) continue;
            auto it = want_new.find(e.id);
            if (it == want_new.end()) continue;
            const int action = pick(0, 60);
            if (action == 0) { REQUIRE(sched.abort(e.id) == 0, "abort failed"); want_new.erase(it); continue; }
            if (action == 1 && sched.state(e.id) != RequestState::Finished) { REQUIRE(sched.stop(e.id) == 0, "stop failed"); want_new.erase(it); continue; }
            const int done = sched.on_token(e.id, pick(0, 40) == 0);
            REQUIRE(done == 0 || done == 1, "on_token returned %d", done);
            if (done == 1) { want_new.erase(it); REQUIRE(sched.forget(e.id) == 0, "forget failed"); }
            else --it->second;
        }
        REQUIRE(cache.check().empty(), "after the step: %s", cache.check().c_str());
    }
    REQUIRE(steps < 5000, "the workload did not drain");
    REQUIRE(!sched.has_work(), "work left");
    for (int g = 0; g < 2; ++g) REQUIRE(cache.free_pages(g) == cache.total_pages(g), "pages lost in group %d", g);
    REQUIRE(cache.free_state_slots() == n_slots && cache.n_requests() == 0, "slots or requests left");
    const Counters& c = sched.counters();
    g_total.steps += c.steps; g_total.preemptions += c.preemptions; g_total.deferred_decodes += c.deferred_decodes;
    g_total.deferred_prefills += c.deferred_prefills; g_total.failures += c.failures; g_total.finished += c.finished;
}

int main(int argc, char** argv) {
    const int runs = argc > 1 ? std::atoi(argv[1]) : 200;
    for (int r = 0; r < runs; ++r) one_run(1000u + static_cast<unsigned>(r));
    // (the pools are small enough that the pressure paths run)
    REQUIRE(runs < 50 || (g_total.preemptions > 0 && g_total.deferred_decodes > 0 && g_total.deferred_prefills > 0 && g_total.finished > 0),
            "the workload exercised no page pressure");
    std::printf("ok %d runs: %lld steps, %lld finished, %lld preemptions, %lld deferred decodes, %lld deferred prefills, %lld failures\n", runs,
                static_cast<long long>(g_total.steps), static_cast<long long>(g_total.finished), static_cast<long long>(g_total.preemptions),
                static_cast<long long>(g_total.deferred_decodes), static_cast<long long>(g_total.deferred_prefills),
                static_cast<long long>(g_total.failures));
    return 0;
}
