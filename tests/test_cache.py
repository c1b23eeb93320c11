"""The cache's bookkeeping, without a GPU: no slot or page lost, held twice or freed
twice; groups with and without a window; state rows; sharing between runs."""
import random

import pytest
import torch

from tq_kv_amd.cache import PAGE, Cache, CacheFull
from tq_kv_amd.parts.spec import KVNeed, StateNeed

FULL = KVNeed(2, 16, None)
WIN = KVNeed(2, 16, 100)


def make(needs, cache_of=None, max_tokens=PAGE * 8, max_slots=4):
    return Cache(needs, cache_of or [None] * len(needs), max_tokens, max_slots, torch.float32, "cpu")


def test_lengths_after_prompt_and_single_tokens():
    # prompt(8), +1, +1 -> 8, 9, 10 (tq-kv/src/candle_kv.rs:266-299)
    c = make([FULL, FULL])
    s = c.acquire()
    for n, want in [(8, 8), (1, 9), (1, 10)]:
        c.reserve([(s, n)])
        c.commit([(s, n)])
        assert c.length(s) == want
    c.release(s)
    assert c.acquire() == s and c.length(s) == 0     # the slot is used again, empty
    c.check()


def test_groups_have_storage_of_their_own():
    c = make([FULL, WIN, WIN, FULL])
    assert len(c.kv_groups) == 2
    full = next(g for g in c.kv_groups if g.need.window is None)
    win = next(g for g in c.kv_groups if g.need.window == 100)
    assert full.runs == [0, 3] and win.runs == [1, 2]
    assert full.keys.shape == (2, 8, 2, PAGE, 16) and win.values.shape == (2, 8, 2, 16, PAGE)
    assert c.entry(3).keys.data_ptr() == full.keys[1].data_ptr()
    assert c.entry(1).group is win and c.entry(1).writes


def test_window_group_gives_pages_back_early():
    c = make([FULL, WIN], max_tokens=PAGE * 8)
    full, win = c.kv_groups
    s = c.acquire()
    c.reserve([(s, 300)])
    assert full.pool.n_held == 5 and win.pool.n_held == 5      # a prompt needs all its positions in the step
    c.commit([(s, 300)])
    # next query is at 300 and sees 201..300: pages 0..2 (positions < 192) are dead
    assert win.pool.n_held == 2 and win.pages[s][:3] == [-1, -1, -1] and full.pool.n_held == 5
    t = c.page_table(win, [s])
    assert t.shape == (1, 5) and list(t[0, :3]) == [-1, -1, -1] and all(p >= 0 for p in t[0, 3:])
    for _ in range(100):
        c.reserve([(s, 1)])
        c.commit([(s, 1)])
    assert win.pool.n_held == 3 and full.pool.n_held == 7      # 400 positions: 7 pages, window holds 301..400
    c.check()
    c.release(s)
    assert win.pool.n_held == 0 and full.pool.n_held == 0
    c.check()


def test_reserve_is_all_or_nothing():
    c = make([FULL], max_tokens=PAGE * 4, max_slots=4)
    a, b = c.acquire(), c.acquire()
    c.reserve([(a, PAGE * 2)])
    c.commit([(a, PAGE * 2)])
    with pytest.raises(CacheFull):
        c.reserve([(a, 1), (b, PAGE * 2)])      # 1 + 2 pages wanted, 2 free
    assert c.kv_groups[0].pool.n_held == 2 and b not in c.kv_groups[0].pages
    c.check()
    c.reserve([(b, PAGE * 2)])
    c.commit([(b, PAGE * 2)])
    assert c.tokens_held() == PAGE * 4
    with pytest.raises(CacheFull):
        c.reserve([(a, 1)])
    c.release(a)
    c.reserve([(b, 1)])                          # a's pages are there for b now
    c.check()


def test_slots_run_out_and_come_back():
    c = make([FULL], max_slots=2)
    a, b = c.acquire(), c.acquire()
    with pytest.raises(CacheFull):
        c.acquire()
    c.release(a)
    with pytest.raises(AssertionError):
        c.release(a)
    assert c.acquire() == a
    c.check()


def test_random_walk_loses_nothing():
    rng = random.Random(0)
    c = make([FULL, WIN, FULL], max_tokens=PAGE * 16, max_slots=6)
    live = {}
    for _ in range(600):
        op = rng.random()
        if op < 0.25 and len(live) < 6:
            live[c.acquire()] = 0
        elif op < 0.4 and live:
            s = rng.choice(list(live))
            c.release(s)
            del live[s]
        elif live:
            batch = rng.sample(list(live), rng.randint(1, len(live)))
            items = [(s, rng.choice([1, 1, 1, 7, 70, 130])) for s in batch]
            try:
                c.reserve(items)
            except CacheFull:
                c.check()
                continue
            c.commit(items)
            for s, n in items:
                live[s] += n
                assert c.length(s) == live[s]
        c.check()
        assert c.tokens_held() <= PAGE * 16
        for g in c.kv_groups:
            for s in live:
                pages = g.pages.get(s, [])
                first = g.first_needed(live[s]) // PAGE
                assert all(p >= 0 for p in pages[first:]) and len(pages) >= (live[s] + PAGE - 1) // PAGE
    for s in list(live):
        c.release(s)
    c.check()
    assert all(g.pool.n_held == 0 for g in c.kv_groups) and c.slots.n_held == 0


def test_state_rows_are_zeroed_when_a_slot_is_taken():
    c = make([StateNeed((3,)), FULL, None])
    assert c.entry(2) is None
    st = c.entry(0)
    s = c.acquire()
    st.state[s] += 5.0
    c.release(s)
    s2 = c.acquire()
    assert s2 == s and torch.equal(st.state[s2], torch.zeros(3))
    assert st.state.shape == (4, 3)


def test_a_run_can_read_another_runs_cache():
    c = make([FULL, FULL, FULL], cache_of=[None, None, 0])
    assert len(c.kv_groups) == 1 and c.kv_groups[0].runs == [0, 1]
    assert c.entry(2).keys.data_ptr() == c.entry(0).keys.data_ptr() and not c.entry(2).writes and c.entry(0).writes
    with pytest.raises(ValueError, match="needs"):
        make([FULL, WIN], cache_of=[None, 0])
    with pytest.raises(ValueError, match="keeps none"):
        make([None, FULL], cache_of=[None, 0])


def test_sizes():
    with pytest.raises(ValueError):
        make([FULL], max_tokens=10)
    c = make([FULL], max_tokens=PAGE * 3 + 5, max_slots=100)
    assert c.n_pages == 3 and c.max_slots == 3        # never more slots than pages


def test_a_cache_of_state_alone_holds_no_pages_and_is_bounded_by_slots():
    from tq_kv_amd.engine.generate import plan_batches
    cache = Cache([StateNeed((4,)), None, StateNeed((4,), "int32")], [None, None, None], 10, 7, torch.float32, "cpu")
    assert not cache.holds_pages and cache.max_slots == 7 and cache.kv_groups == [] and len(cache.state_groups) == 2
    assert cache.state_groups[1].state.dtype == torch.int32
    slots = [cache.acquire() for _ in range(7)]
    cache.reserve([(s, 100000) for s in slots])           # no pages to run out of
    cache.commit([(s, 100000) for s in slots])
    assert cache.length(slots[3]) == 100000
    with pytest.raises(CacheFull):
        cache.acquire()
    for s in slots:
        cache.release(s)
    cache.check()
    # the loop plans such a model by slots alone
    assert plan_batches([500] * 5, 10, 64, 2, holds_pages=False) == [[0, 1], [2, 3], [4]]
    with pytest.raises(Exception, match="cache positions"):
        plan_batches([500] * 5, 10, 64, 2)
