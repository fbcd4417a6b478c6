"""The cache manager's bookkeeping on the host: no page lost, held twice or freed twice, under
random orders of requests; windows give pages back; promises hold (CPU)."""
import random

import pytest
import torch

from zedinfer_amd.cache import CacheManager, IdPool, OutOfPages, OutOfSlots, PagePool
from zedinfer_amd.parts.mixers import attention_cache_request


def manager(pages=12, page_size=4, requests=4, window=0, max_step_tokens=8):
    kv = {0: attention_cache_request("full", 2, 16), 1: attention_cache_request("full", 2, 16)}
    if window:
        kv[2] = attention_cache_request("window", 1, 32, window)
    return CacheManager(kv, {}, pages, page_size, requests, torch.float32, None, max_step_tokens)


def test_pool_basics():
    # reference: tests/kvcache/test_block_pool.cpp:40-45 (a full pool refuses), :161-189 (free+used==total)
    p = PagePool(3)
    a, b, c = p.take(), p.take(), p.take()
    assert sorted([a, b, c]) == [0, 1, 2] and p.num_free == 0
    with pytest.raises(OutOfPages):
        p.take()
    p.give_back(b)
    assert p.take() == b                      # last in, first out: used again at once
    with pytest.raises(ValueError, match="not held"):
        p.give_back(b) or p.give_back(b)
    with pytest.raises(ValueError, match="outside"):
        p.give_back(7)
    p.check()
    s = IdPool(1, "state slot")
    s.take()
    with pytest.raises(OutOfSlots):
        s.take()


def test_groups_by_need():
    m = manager(window=6)
    assert [(g.kind, g.window, sorted(g.caches)) for g in m.groups] == [("full", 0, [0, 1]), ("window", 6, [2])]
    assert m.group_of_cache == {0: 0, 1: 0, 2: 1}


def test_grow_commit_close():
    m = manager()
    s = m.open("a")
    m.ensure(s, 5)
    assert s.held == [2] and s.pages[0] == [0, 1]
    m.commit(s, 5)
    m.ensure(s, 8)
    assert s.held == [2]
    m.ensure(s, 9)
    assert s.held == [3]
    assert m.token_slots(s, 0, 3, 3).tolist() == [3, 4, 5]
    m.check()
    m.close(s)
    assert m.groups[0].pool.num_free == 12 and m.slots.num_free == 4 and not m.live
    with pytest.raises(ValueError, match="closed"):
        m.close(s)
    m.check()


def test_ensure_is_all_or_nothing():
    m = manager(pages=4, window=6)
    a, b = m.open("a"), m.open("b")
    m.ensure(a, 12)                                  # 3 of 4 pages in both groups
    m.commit(a, 12)
    before = (list(b.pages[0]), list(b.pages[1]), b.held[:], b.promised[:],
              m.groups[0].pool.num_free, m.groups[1].pool.num_free)
    with pytest.raises(OutOfPages):
        m.ensure(b, 8)                               # the full group lacks a page
    assert before == (b.pages[0], b.pages[1], b.held, b.promised, m.groups[0].pool.num_free,
                      m.groups[1].pool.num_free)
    m.check()


def test_undo_gives_back_what_an_ensure_took():
    """A step that cannot grow one of its requests undoes the growth of the others (Engine.step does)."""
    m = manager(pages=6, window=6)
    a, b = m.open("a"), m.open("b")
    m.ensure(a, 5)
    m.commit(a, 5)
    before = (list(a.pages[0]), list(a.pages[1]), a.held[:], a.promised[:],
              m.groups[0].pool.num_free, m.groups[1].pool.num_free, m.groups[0].pool.committed)
    growth = m.ensure(a, 14)
    assert growth.taken and a.held[0] > before[2][0]
    with pytest.raises(OutOfPages):
        m.ensure(b, 20)
    m.undo(a, growth)
    assert before == (a.pages[0], a.pages[1], a.held, a.promised, m.groups[0].pool.num_free,
                      m.groups[1].pool.num_free, m.groups[0].pool.committed)
    m.check()
    m.ensure(a, 14)                                  # and it can be taken again
    m.commit(a, 14)
    m.check()


def test_window_gives_pages_back():
    m = manager(pages=6, page_size=4, window=6)
    s = m.open("a")
    seen_free = []
    for n in range(1, 41):
        m.ensure(s, n)
        m.commit(s, n)
        m.check()
        seen_free.append(m.groups[1].pool.num_free)
        if n <= 24:
            assert s.held[0] == -(-n // 4)
        # the window group holds only pages that a later token can still see
        first_needed = max(0, n - 6 + 1) // 4
        assert all(p < 0 for p in s.pages[1][:first_needed]) and all(p >= 0 for p in s.pages[1][first_needed:])
        assert s.held[1] <= 3
        if n == 24:
            break
    assert m.groups[1].pool.takes > 3            # window pages went round
    with pytest.raises(RuntimeError, match="no page"):
        m.token_slots(s, 1, 0, 4)                  # a position the window has passed
    m.close(s)
    m.check()


def test_promises():
    m = manager(pages=10, page_size=4, requests=8)
    assert m.can_open(40) and not m.can_open(41)
    a = m.open("a", expected_tokens=24)              # 6 pages promised
    assert not m.can_open(17) and m.can_open(16)
    b = m.open("b", expected_tokens=16)              # 4 pages: everything is promised
    with pytest.raises(OutOfPages):
        m.open("c", expected_tokens=1)
    m.ensure(b, 16)
    m.commit(b, 16)
    with pytest.raises(OutOfPages, match="all 10 are promised"):
        m.ensure(b, 17)                              # b may not take what a was promised
    m.ensure(a, 24)                                  # a's promise holds although b wanted more
    m.check()
    m.close(a)
    m.ensure(b, 17)                                  # now there is an unpromised page
    assert b.promised == [5]
    m.check()


def test_slots():
    m = manager(requests=2)
    a, b = m.open("a"), m.open("b")
    assert {a.slot, b.slot} == {0, 1}
    assert not m.can_open(1)
    with pytest.raises(OutOfSlots):
        m.open("c")
    with pytest.raises(ValueError, match="already holds"):
        m.open("a")
    m.close(a)
    assert m.open("c").slot == a.slot


@pytest.mark.parametrize("seed", range(6))
@pytest.mark.parametrize("window", [0, 10])
def test_random_orders(seed, window):
    rng = random.Random(seed)
    m = manager(pages=16, page_size=4, requests=4, window=window, max_step_tokens=9)
    live, n_id = {}, 0
    for _ in range(600):
        op = rng.random()
        if op < 0.2 and len(live) < 4:
            try:
                s = m.open(n_id, expected_tokens=rng.choice([0, 0, 8, 20]))
                live[n_id] = s
            except OutOfPages:
                pass
            n_id += 1
        elif op < 0.85 and live:
            s = live[rng.choice(list(live))]
            n = rng.choice([1, 1, 1, 2, 5, 9])
            try:
                m.ensure(s, s.length + n)
                m.commit(s, s.length + n)
            except OutOfPages:
                m.close(s)                            # what the scheduler does with a request that cannot grow
                del live[s.request_id]
        elif live:
            rid = rng.choice(list(live))
            m.close(live.pop(rid))
        m.check()
    for s in list(live.values()):
        m.close(s)
    m.check()
    assert all(g.pool.num_free == g.pool.total and g.pool.committed == 0 for g in m.groups)
    assert all(g.pool.takes > g.pool.total for g in m.groups)
