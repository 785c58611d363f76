"""The scheduler's decisions, driven without a model (the reference tests its scheduler with a
mock backend that emits 1000, 1001, ... : /root/reference/include/runtime/mock_backend.h:10-48,
/root/reference/tests/cpp/test_scheduler.cpp:160-221), and the engine under page pressure on
the CPU reference ops."""
import pytest
import torch

import plain_ops
from conftest import TINY
from mini_llm_amd.cache.manager import CacheManager, GroupSpec
from mini_llm_amd.engine.scheduler import Scheduler


def drive(s, eos_after=None, max_iters=10000):
    """Runs the loop with a fake model; returns per-request token counts and the plans."""
    produced, plans = {}, []
    for _ in range(max_iters):
        plan = s.schedule()
        if not plan:
            break
        plans.append(plan)
        s.commit()
        for e in plan:
            if e.want_last:
                n = produced.get(e.request_id, 0) + 1
                produced[e.request_id] = n
                s.on_token(e.request_id, eos_after is not None and n >= eos_after.get(e.request_id, 10 ** 9))
    return produced, plans


def make(n_pages=64, page=4, seqs=4, budget=32, chunk=16, max_pos=128, slots=None, preempt_for_decode=False):
    cm = CacheManager([GroupSpec(page, n_pages)], slots or seqs)
    return cm, Scheduler(cm, seqs, budget, chunk, max_pos, preempt_for_decode)


def test_single_request_lifecycle():
    cm, s = make()
    s.add_request(7, 5, 4)
    assert s.state(7) == "waiting_prefill"
    plan = s.schedule()
    assert [(e.request_id, e.start, e.n_tokens, e.want_last) for e in plan] == [(7, 0, 5, True)]
    assert s.state(7) == "prefill"
    s.commit()
    assert not s.on_token(7, False) and s.state(7) == "decode_ready"
    starts = []
    for i in range(3):
        (e,) = s.schedule()
        starts.append((e.start, e.n_tokens, e.want_last))
        s.commit()
        done = s.on_token(7, False)
        assert done == (i == 2)
    assert starts == [(5, 1, True), (6, 1, True), (7, 1, True)]       # the prefill's token is output #1
    assert s.state(7) == "finished" and s.generated(7) == 4 and not s.has_work()
    assert cm.free_pages() == 64 and cm.n_requests() == 0 and cm.check() == ""
    assert s.schedule() == []


def test_refused_requests():
    cm, s = make(max_pos=16)
    with pytest.raises(ValueError):
        s.add_request(1, 0, 4)
    with pytest.raises(ValueError):
        s.add_request(1, 17, 4)
    with pytest.raises(ValueError):
        s.add_request(1, 4, 0)
    s.add_request(1, 16, 4)
    with pytest.raises(KeyError):
        s.add_request(1, 3, 4)
    produced, _ = drive(s)
    assert produced == {1: 1}              # the prompt fills every position: one token, then the length cap


def test_pages_promised_to_a_prompt_under_way_are_not_given_to_the_next():
    """Two prompts of two portions each whose pages fit only one at a time: the second is admitted
    only when the first has finished, so nobody is preempted and recomputed."""
    cm, s = make(n_pages=12, page=4, budget=32, chunk=16)
    s.add_request(1, 32, 2)                # 8 pages for the prompt, 9 with its second token
    s.add_request(2, 32, 2)
    p = s.schedule()
    assert [(e.request_id, e.n_tokens) for e in p] == [(1, 16)]
    assert s.state(2) == "deferred_prefill"          # 4 pages free are promised to request 1
    s.commit()
    produced, plans = drive(s)
    assert produced == {1: 2, 2: 2}
    assert s.counters()["preemptions"] == 0
    assert all(len({e.request_id for e in plan}) == 1 for plan in plans)
    assert cm.free_pages() == 12 and cm.check() == ""


def test_finished_requests_can_be_forgotten():
    cm, s = make()
    s.add_request(1, 5, 1)
    s.add_request(2, 5, 3)
    s.schedule(); s.commit()
    assert s.on_token(1, False) and not s.on_token(2, False)
    assert s.n_known() == 2
    s.forget(1)
    s.forget(2)                            # still live: stays
    assert s.n_known() == 1 and s.state(1) == "unknown" and s.state(2) == "decode_ready"
    s.add_request(1, 3, 1)                 # the id is free again
    produced, _ = drive(s)
    assert produced == {1: 1, 2: 2}


def test_prompts_are_cut_under_the_budget_and_decodes_come_first():
    cm, s = make(budget=12, chunk=8)
    s.add_request(1, 20, 3)
    s.add_request(2, 6, 3)
    p1 = s.schedule()
    assert [(e.request_id, e.start, e.n_tokens, e.want_last) for e in p1] == [(1, 0, 8, False), (2, 0, 4, False)]
    s.commit()
    p2 = s.schedule()
    assert [(e.request_id, e.start, e.n_tokens, e.want_last) for e in p2] == [(1, 8, 8, False), (2, 4, 2, True)]
    s.commit(); s.on_token(2, False)
    p3 = s.schedule()          # request 2 decodes first, then request 1's last portion
    assert [(e.request_id, e.start, e.n_tokens, e.want_last) for e in p3] == [(2, 6, 1, True), (1, 16, 4, True)]
    s.commit(); s.on_token(2, False); s.on_token(1, False)
    produced, _ = drive(s)
    assert s.generated(1) == 3 and s.generated(2) == 3 and cm.free_pages() == 64


def test_max_num_seqs_limits_a_step_and_nobody_starves():
    cm, s = make(seqs=2, slots=8)
    for i in range(5):
        s.add_request(i, 3, 4)
    produced, plans = drive(s)
    assert all(len(p) <= 2 for p in plans)
    assert produced == {i: 4 for i in range(5)}
    c = s.counters()
    assert c["finished"] == 5 and c["prefill_tokens"] == 15 and c["decode_tokens"] == 15


def test_admission_waits_for_pages_first_come_first_served():
    cm, s = make(n_pages=6, page=4)             # 24 tokens of cache
    s.add_request(1, 16, 3)                     # 4 pages, 5 with its outputs
    s.add_request(2, 12, 2)                     # 3 pages: does not fit beside request 1
    s.add_request(3, 2, 2)                      # would fit, but may not overtake request 2
    plan = s.schedule()
    assert [e.request_id for e in plan] == [1]
    assert s.state(2) == "deferred_prefill" and s.state(3) == "waiting_prefill"
    assert (2, "deferred") in s.pop_events()
    produced, _ = drive(s)
    assert produced == {1: 3, 2: 2, 3: 2} and s.counters()["preemptions"] == 0
    assert cm.free_pages() == 6 and cm.check() == ""


def test_out_of_pages_defers_decodes_then_preempts_the_latest():
    cm, s = make(n_pages=4, page=4, budget=16, chunk=16)
    s.add_request(1, 7, 8)                      # 2 pages; needs a 3rd at length 9, a 4th at 13
    s.add_request(2, 7, 8)                      # 2 pages
    events = []
    produced = {}
    for _ in range(200):
        plan = s.schedule()
        events += s.pop_events()
        if not plan:
            break
        s.commit()
        for e in plan:
            if e.want_last:
                produced[e.request_id] = produced.get(e.request_id, 0) + 1
                s.on_token(e.request_id, False)
        assert cm.check() == ""
    # both need a third page at the same step: the later one is preempted, recomputed after the first ends
    assert (2, "preempted") in events
    assert produced == {1: 8, 2: 8}
    c = s.counters()
    assert c["preemptions"] >= 1 and c["deferred_decodes"] >= 1 and c["failures"] == 0
    assert cm.free_pages() == 4 and cm.n_requests() == 0


def test_a_decode_without_a_page_preempts_a_younger_request_at_once():
    """The engine's default policy: an older request never waits on its pages for a younger one. Three requests
    of 7 + 8 tokens through 7 pages of 4: all are admitted (2 pages each); both request 1 and request 2 need a third
    page at position 8 and one is free: request 1 takes it, and for request 2 the youngest, request 3, is preempted
    in that same iteration (no deferral). Later request 2 is the youngest that runs: it then waits (there is nobody
    younger to take pages from). Request 3 is recomputed once pages are free again, and everybody finishes."""
    cm, s = make(n_pages=7, page=4, budget=32, chunk=16, preempt_for_decode=True)
    for rid in (1, 2, 3):
        s.add_request(rid, 7, 8)
    events, produced, order = [], {}, []
    for it in range(200):
        plan = s.schedule()
        for ev in s.pop_events():
            events.append((it,) + ev)
        if not plan:
            break
        s.commit()
        for e in plan:
            if e.want_last:
                produced[e.request_id] = produced.get(e.request_id, 0) + 1
                if s.on_token(e.request_id, False):
                    order.append(e.request_id)
        assert cm.check() == ""
    kinds = [(rid, kind) for _, rid, kind in events]
    assert events[0] == (2, 3, "preempted")            # in the iteration in which request 2 found no page
    assert not any(rid == 1 for rid, _ in kinds)       # the oldest neither waits nor is preempted
    assert (2, "preempted") not in kinds and all(it > 2 for it, rid, kind in events if (rid, kind) == (2, "deferred"))
    assert produced == {1: 8, 2: 8, 3: 8} and order[:2] == [1, 2]
    c = s.counters()
    assert c["preemptions"] >= 1 and c["failures"] == 0 and cm.free_pages() == 7 and cm.n_requests() == 0
    # the reference's manner on the same workload: the decode waits (is deferred) instead
    cm2, s2 = make(n_pages=7, page=4, budget=32, chunk=16, preempt_for_decode=False)
    for rid in (1, 2, 3):
        s2.add_request(rid, 7, 8)
    produced2, _ = drive(s2)
    assert produced2 == {1: 8, 2: 8, 3: 8} and s2.counters()["deferred_decodes"] >= 1


def test_a_request_larger_than_the_pool_fails_alone():
    cm, s = make(n_pages=2, page=4)
    s.add_request(1, 9, 2)                      # 3 pages, the pool has 2
    s.add_request(2, 3, 2)
    produced, _ = drive(s)
    assert s.state(1) == "failed" and produced == {2: 2}
    assert (1, "failed") in s.pop_events()
    # one that fits at first and outgrows the pool fails when it is alone
    s.add_request(3, 7, 8)
    produced, _ = drive(s)
    assert s.state(3) == "failed" and produced[3] == 2 and cm.free_pages() == 2


def test_eos_and_abort_free_everything():
    cm, s = make()
    s.add_request(1, 5, 50)
    s.add_request(2, 5, 50)
    s.add_request(3, 40, 50)
    plan = s.schedule(); s.commit()
    for e in plan:
        if e.want_last:
            s.on_token(e.request_id, e.request_id == 1)
    assert s.state(1) == "finished" and s.state(3) == "prefill"
    s.abort(3)
    assert s.state(3) == "aborted" and s.counters()["aborted"] == 1 and s.counters()["failures"] == 0
    assert s.pop_events() == []                   # (no event: the caller who aborts knows)
    produced, _ = drive(s, eos_after={2: 3})
    assert s.generated(2) == 4 and cm.free_pages() == 64 and cm.n_requests() == 0 and not s.has_work()
