"""The cache manager: no page lost, held twice or freed twice, under random orders of
requests; groups with windows give pages back as the window passes; state slots."""
import random

import numpy as np
import pytest

from mini_llm_amd.cache.manager import CacheManager, GroupSpec, OutOfPages


def test_pages_are_taken_per_block_and_reused_lifo():
    cm = CacheManager([GroupSpec(4, 6)], 2)
    assert cm.add_request(10) == 0
    cm.reserve(10, 5)
    assert cm.block_table(10, 0).tolist() == [0, 1] and cm.free_pages() == 4
    cm.reserve(10, 8)                                   # still two blocks
    assert cm.free_pages() == 4
    cm.commit(10, 8)
    cm.reserve(10, 9)
    assert cm.block_table(10, 0).tolist() == [0, 1, 2]
    assert cm.add_request(11) == 1
    cm.reserve(11, 4)
    assert cm.block_table(11, 0).tolist() == [3]
    assert cm.free_request(10) == 3
    cm.reserve(11, 12)                                  # the pages just given back come first
    assert cm.block_table(11, 0).tolist() == [3, 2, 1]
    assert cm.check() == ""


def test_errors_are_reported_not_swallowed():
    cm = CacheManager([GroupSpec(4, 2)], 1)
    cm.add_request(1)
    with pytest.raises(KeyError):
        cm.add_request(1)
    with pytest.raises(OutOfPages):
        cm.add_request(2)                               # no slot left
    with pytest.raises(OutOfPages):
        cm.reserve(1, 9)                                # three pages, two exist
    assert cm.free_pages() == 2                         # all or nothing
    cm.reserve(1, 8)
    with pytest.raises(KeyError):
        cm.commit(1, 9)                                 # beyond what was reserved
    cm.commit(1, 8)
    with pytest.raises(KeyError):
        cm.reserve(1, 7)                                # below the committed length
    cm.free_request(1)
    with pytest.raises(KeyError, match="freed twice"):
        cm.free_request(1)
    with pytest.raises(KeyError):
        cm.length(1)
    assert cm.check() == "" and cm.free_pages() == 2 and cm.free_state_slots() == 1
    with pytest.raises(ValueError):
        CacheManager([GroupSpec(0, 2)], 1)


def test_window_group_gives_pages_back_as_it_passes():
    # group 0 keeps everything; group 1 needs the last 6 keys only
    cm = CacheManager([GroupSpec(4, 16, 0), GroupSpec(4, 4, 6)], 1)
    cm.add_request(1)
    held = []
    for n in range(1, 41):
        cm.reserve(1, n)
        cm.commit(1, n)
        t = cm.block_table(1, 1).tolist()
        live = [b for b, p in enumerate(t) if p >= 0]
        first_key = max(0, n - 6 + 1)                   # the next query (position n) needs keys >= this
        assert live == list(range(first_key // 4, (n + 3) // 4)), (n, t)
        held.append(len(live))
        assert cm.check() == ""
    assert max(held) <= 3 and cm.free_pages(1) >= 1
    assert (cm.block_table(1, 0) >= 0).all() and len(cm.block_table(1, 0)) == 10
    # a long portion needs pages for all of its tokens at once, then gives most back
    cm.free_request(1)
    cm.add_request(2)
    cm.reserve(2, 16)
    assert cm.free_pages(1) == 0
    cm.commit(2, 16)
    assert cm.free_pages(1) == 2 and cm.block_table(2, 1).tolist()[:2] == [-1, -1]
    with pytest.raises(OutOfPages):
        cm.reserve(2, 16 + 12)
    cm.reserve(2, 16 + 8)


@pytest.mark.parametrize("seed", range(6))
def test_random_orders_keep_every_page_accounted_for(seed):
    rng = random.Random(seed)
    groups = [GroupSpec(4, 40, 0), GroupSpec(8, 12, rng.choice([0, 5, 16])), GroupSpec(2, 30, 3)]
    cm = CacheManager(groups, 6)
    live = {}                     # id -> committed length
    next_id = 0
    for _ in range(600):
        op = rng.random()
        if op < 0.25 and len(live) < 6:
            cm.add_request(next_id)
            live[next_id] = 0
            next_id += 1
        elif op < 0.8 and live:
            rid = rng.choice(list(live))
            new_len = live[rid] + rng.choice([1, 1, 1, 2, 3, 7, 16])
            need = [cm.pages_needed(rid, g, new_len) for g in range(3)]
            free = [cm.free_pages(g) for g in range(3)]
            fits = all(n <= f for n, f in zip(need, free))
            assert cm.can_reserve(rid, new_len) == fits
            if fits:
                cm.reserve(rid, new_len)
                assert [cm.free_pages(g) for g in range(3)] == [f - n for f, n in zip(free, need)]
                if rng.random() < 0.9:
                    cm.commit(rid, new_len)
                    live[rid] = new_len
            else:
                with pytest.raises(OutOfPages):
                    cm.reserve(rid, new_len)
                assert [cm.free_pages(g) for g in range(3)] == free
        elif live:
            rid = rng.choice(list(live))
            cm.free_request(rid)
            del live[rid]
            with pytest.raises(KeyError):
                cm.free_request(rid)
        assert cm.check() == ""
        # a page id appears in one table only
        for g in range(3):
            seen = []
            for rid in live:
                seen += [p for p in cm.block_table(rid, g).tolist() if p >= 0]
            assert len(seen) == len(set(seen)) == cm.total_pages(g) - cm.free_pages(g)
    for rid in list(live):
        cm.free_request(rid)
    assert all(cm.free_pages(g) == groups[g].n_pages for g in range(3)) and cm.free_state_slots() == 6
